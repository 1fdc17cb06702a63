// Definitions shared by the attention kernels (attention.hip, attention_pipe.hip): parameter block, mask helpers.
#pragma once

#include <math.h>

#include <type_traits>

#include "common.h"

namespace kernl {

static constexpr float kLog2eA = 1.4426950408889634f;
static constexpr float kNegBig = -1.0e30f;            // anything below: exp2(x - rowmax) is exactly 0
static constexpr float kClampFloor = -1.7014118e38f;  // scaled mask values are kept finite (-FLT_MAX / 2)
static constexpr float kRescaleThreshold = 8.0f;  // log2 units
static constexpr float kMaskedScore = -32768.0f;  // base-2 scores below this are mask values, not scores
// A mask value (base-2 domain) at or below this marks a dead key: added to any score a 16-bit model produces it stays
// below kMaskedScore, so the key weighs exactly 0 in every row that has an ordinary key, and a key tile of dead keys only
// is not visited at all.  -inf and the fp32 / bf16 "minimum" masks are far below it, and so is the fp16 one that models
// build in their own dtype (finfo(float16).min = -65504, -94505 in the base-2 domain) — which kNegBig does not catch.
static constexpr float kDeadMask = 2.0f * kMaskedScore;

enum { MASK_NONE = 0, MASK_VECTOR = 1, MASK_MATRIX = 2 };

struct AttnParams {
    const void *q, *k, *v, *mask;
    void *o;
    int B, H, M, N;
    int64_t qs[4], ks[4], vs[4], os[4];  // element strides {batch, head, row, col}
    int64_t ms[4];                       // mask strides, 0 on broadcast dims
    int mask_dtype;
    float scale_log2;  // sm_scale * log2(e)
    float sm_scale;
    float clamp;  // replacement for -inf mask entries
    int nq_tiles;
    int mask_fast;  // matrix mask rows: 1 = readable as aligned 4-element vectors through 32-bit offsets,
                    // 2 = 16-byte chunks of a row are aligned too (they can be staged through LDS)
    int xcd_by_batch;  // workgroups of one batch entry (all heads) share an XCD instead of those of one head
    int causal_off;  // causal: query row m sees keys 0 .. m + causal_off (0: top-left aligned)
};

__device__ __forceinline__ float load_mask_value(const void *mask, int dtype, int64_t off) {
    if (dtype == KERNL_F32) return static_cast<const float *>(mask)[off];
    if (dtype == KERNL_F16) return (float)static_cast<const f16 *>(mask)[off];
    return (float)static_cast<const bf16 *>(mask)[off];
}

// mask value -> additive term in the log2 domain, finite.
__device__ __forceinline__ float scale_mask(float mv, float clamp) {
    if (mv == -INFINITY) mv = clamp;
    return fmaxf(mv * kLog2eA, kClampFloor);
}


// Software-pipelined MFMA kernel (attention_pipe.hip).  Handles head sizes 64 and 128 with no mask or with a per-key
// mask of at most kPipeMaxMaskKeys keys (non-causal), and causal attention without a mask; taken from kPipeMinKeys keys
// on — head size 128 only for causal problems with few (batch, head) pairs — or whenever it applies, with `force`.
// Returns false when it does not take the problem.
static constexpr int kPipeMaxMaskKeys = 2048;
static constexpr int kPipeMinKeys = 1024;
bool launch_attention_pipe(const AttnParams &p, int D, int dtype, int mask_mode, bool causal, bool force, hipStream_t st);

}  // namespace kernl
