// Flash-attention forward for gfx950:  out = softmax(q·kᵀ·scale + causal + mask) · v.
//
// Semantics follow the reference kernel src/kernl/implementations/attention.py:122-435: scores and both
// accumulators in fp32, additive mask with -inf entries clamped to a finite minimum, top-left aligned causal
// masking, online softmax over key tiles, P rounded to the input dtype before P·V.  The softmax is kept
// un-normalised until the end (one division per output element instead of the reference's per-tile
// renormalisation, attention.py:399-417) — the same value up to fp32 rounding.
//
// MFMA path.  A workgroup of 4 waves owns 128 query rows of one (batch, head); each wave owns 32 of them.
// Key/value tiles are staged HBM -> VGPR -> LDS (double buffered, one barrier per tile):
//   K tile  [BN keys][D]      row-major, 16-byte chunks XOR-swizzled;
//   Vᵀ tile [D][BN keys]      transposed in registers on the way in (each thread holds a 4-key x 8-feature
//                             block), because P·V contracts over keys and an MFMA lane needs 8 consecutive
//                             values of the contraction index.
// Scores are computed TRANSPOSED: Sᵀ = K·Qᵀ with K on the MFMA "A" side, so a lane ends up with the scores of
// ONE query row (lane % 32) against BN/2 keys.  Row max and row sum are then lane-local loops plus a single
// exchange with lane ^ 32, and the fp32 score registers, once exponentiated and packed to 16 bit, already are
// the MFMA "B" operand of Oᵀ = Vᵀ·Pᵀ — P never touches LDS.  Vᵀ rows are stored through rowperm16, so each lane
// finishes with 16 consecutive output features of its query row and writes them as two 16-byte stores.
#include <math.h>

#include "common.h"

namespace kernl {

static constexpr float kLog2eA = 1.4426950408889634f;
static constexpr float kNegBig = -1.0e30f;            // anything below: exp2(x - rowmax) is exactly 0
static constexpr float kClampFloor = -1.7014118e38f;  // scaled mask values are kept finite (-FLT_MAX / 2)
static constexpr int kMaxTiles = 256;
static constexpr float kRescaleThreshold = 8.0f;  // log2 units

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

template <typename T, int D, int BN, int SUB, int WPE, int MASK_MODE, bool CAUSAL>
__global__ void __launch_bounds__(256, WPE) attention_mfma_kernel(const AttnParams p) {
    typedef typename Vec8<T>::type vec8;
    constexpr int BM = 128;
    constexpr int KROW = D * 2, VROW = BN * 2;           // LDS row bytes of the K and Vᵀ tiles
    constexpr int K_BYTES = BN * KROW, V_BYTES = D * VROW;
    constexpr int STAGE = K_BYTES + V_BYTES + BN * 4;    // + per-key additive term (fp32)
    constexpr int NBS = SUB / 32, DB = D / 32, KS = D / 16;
    constexpr int DC = D / 8;                            // 16-byte chunks per K/V row
    constexpr int KI = BN * DC / 256;                    // K chunks per thread per tile
    constexpr int VKEYS = BN * DC / 256;                 // every thread transposes a VKEYS-key x 8-feature block of V
    static_assert(VKEYS == 4 || VKEYS == 2, "V blocks of 4 or 2 keys");
    static_assert(BN * DC % 256 == 0, "K chunks must split evenly over the threads");

    __shared__ __attribute__((aligned(16))) unsigned char smem[2 * STAGE];
    __shared__ int tile_list[kMaxTiles];
    __shared__ int tile_cls[kMaxTiles];
    __shared__ int n_listed;

    // ---- which (batch, head, query tile): ids are dealt round-robin over 8 XCDs; keep all query tiles of a
    // head on one XCD and adjacent in time so K/V re-reads hit that XCD's L2.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int bh = (slot / p.nq_tiles) * 8 + xcd;
    int qt = slot % p.nq_tiles;
    if (bh >= p.B * p.H) return;
    if (CAUSAL) qt = p.nq_tiles - 1 - qt;  // longest rows first
    const int b = bh / p.H, h = bh % p.H;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lr = lane & 31, lh = lane >> 5;
    const int m_wave0 = qt * BM + wave * 32;
    const int my_m = m_wave0 + lr;
    const int M = p.M, N = p.N;

    const T *qp = static_cast<const T *>(p.q) + b * p.qs[0] + h * p.qs[1];
    const T *kp = static_cast<const T *>(p.k) + b * p.ks[0] + h * p.ks[1];
    const T *vp = static_cast<const T *>(p.v) + b * p.vs[0] + h * p.vs[1];
    T *op = static_cast<T *>(p.o) + b * p.os[0] + h * p.os[1];
    const int64_t mask_base = (MASK_MODE != MASK_NONE) ? b * p.ms[0] + h * p.ms[1] : 0;

    // ---- key range and tile list
    int n_end = N;
    if (CAUSAL) n_end = min(N, qt * BM + BM);
    const int nt_all = (n_end + BN - 1) / BN;

    if (MASK_MODE == MASK_VECTOR && !CAUSAL && nt_all <= kMaxTiles) {
        // classify key tiles from the per-key mask: 0 = all zero (no add needed), 1 = general,
        // 2 = every entry so negative that the tile contributes exactly 0 (skippable if some other tile is not).
        for (int t = wave; t < nt_all; t += 4) {
            bool nonzero = false, normal = false;
            for (int n = t * BN + lane; n < min(N, t * BN + BN); n += 64) {
                const float mv = scale_mask(load_mask_value(p.mask, p.mask_dtype, mask_base + n * p.ms[3]), p.clamp);
                nonzero |= (mv != 0.0f);
                normal |= (mv > kNegBig);
            }
            const bool any_nonzero = __ballot(nonzero) != 0, any_normal = __ballot(normal) != 0;
            if (lane == 0) tile_cls[t] = !any_normal ? 2 : (any_nonzero ? 1 : 0);
        }
        __syncthreads();
        if (tid == 0) {
            int cnt = 0;
            for (int t = 0; t < nt_all; ++t)
                if (tile_cls[t] != 2) tile_list[cnt++] = t;
            if (cnt == 0) {  // every key masked: keep them all, the result is the (finite) uniform average
                for (int t = 0; t < nt_all; ++t) {
                    tile_list[t] = t;
                    tile_cls[t] = 1;
                }
                cnt = nt_all;
            }
            n_listed = cnt;
        }
        __syncthreads();
    }
    const bool use_list = (MASK_MODE == MASK_VECTOR && !CAUSAL && nt_all <= kMaxTiles);
    const int nt = use_list ? __builtin_amdgcn_readfirstlane(n_listed) : nt_all;

    // ---- Q fragments (MFMA "B" side: lane holds its query row, 8 consecutive features per k-step)
    vec8 qf[KS];
    {
        const T *qrow = qp + (int64_t)min(my_m, M - 1) * p.qs[2] + lh * 8;
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const vec8 *>(qrow + s * 16);
    }

    // ---- global -> register staging of one K/V tile.  Buffer loads: a uniform resource covering this head's
    // K (V) rows, a loop-invariant 32-bit thread offset and the tile's first row as a scalar offset.  Rows past
    // the last key lie beyond the resource's extent and read as zero in hardware.
    const int v_dc = tid % DC, v_ng = tid / DC;  // this thread's VKEYS-key x 8-feature block of V
    const __amdgpu_buffer_rsrc_t krsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T *>(kp), 0, (int)((((int64_t)N - 1) * p.ks[2] + D) * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T *>(vp), 0, (int)((((int64_t)N - 1) * p.vs[2] + D) * 2), 0x00020000);
    uint32_t kg[KI], vg[VKEYS];  // byte offsets of this thread's chunks inside a tile
    int kl[KI], vl[8];       // LDS byte offsets inside a stage
#pragma unroll
    for (int i = 0; i < KI; ++i) {
        const int qd = tid + 256 * i;
        const int row = qd / DC, c = qd % DC;
        kg[i] = (uint32_t)(((int64_t)row * p.ks[2] + c * 8) * 2);
        kl[i] = swz_offset<KROW>(row, c);
    }
#pragma unroll
    for (int r = 0; r < VKEYS; ++r) vg[r] = (uint32_t)(((int64_t)(v_ng * VKEYS + r) * p.vs[2] + v_dc * 8) * 2);
    {
        // Vᵀ: feature d lives in LDS row (d & ~31) + inverse_rowperm16(d & 31); the VKEYS consecutive keys of this
        // thread stay adjacent at position pos of that row, where pos swaps bits 2 and 3 of the key index (see
        // header comment).
        const int nloc = v_ng * VKEYS;
        const int pos = (nloc & ~12) | ((nloc & 4) << 1) | ((nloc & 8) >> 1);
        const int chunk = pos >> 3, within = (pos & 7) * 2;  // 16-byte chunk, byte offset inside it
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int d = v_dc * 8 + e;
            const int x = d & 31;
            const int row = (d & ~31) + 8 * ((x >> 2) & 3) + 4 * (x >> 4) + (x & 3);
            vl[e] = K_BYTES + swz_offset<VROW>(row, chunk) + within;
        }
    }
    vec8 kst[KI], vst[VKEYS];
    float bias_st = 0.0f;
    auto gload = [&](int tile) {
        const int n0 = tile * BN;
        const int k_soff = (int)((int64_t)n0 * p.ks[2] * 2), v_soff = (int)((int64_t)n0 * p.vs[2] * 2);
#pragma unroll
        for (int i = 0; i < KI; ++i)
            kst[i] = __builtin_bit_cast(vec8, __builtin_amdgcn_raw_buffer_load_b128(krsrc, kg[i], k_soff, 0));
#pragma unroll
        for (int r = 0; r < VKEYS; ++r)
            vst[r] = __builtin_bit_cast(vec8, __builtin_amdgcn_raw_buffer_load_b128(vrsrc, vg[r], v_soff, 0));
        if (MASK_MODE == MASK_VECTOR || n0 + BN > N) {
            if (tid < BN) {
                const int n = n0 + tid;
                float bv = 0.0f;
                if (MASK_MODE == MASK_VECTOR)
                    bv = scale_mask(load_mask_value(p.mask, p.mask_dtype, mask_base + min(n, N - 1) * p.ms[3]), p.clamp);
                if (n >= N) bv = -INFINITY;
                bias_st = bv;
            }
        }
    };
    auto lstore = [&](int stage) {
        unsigned char *sb = smem + stage * STAGE;
#pragma unroll
        for (int i = 0; i < KI; ++i) *reinterpret_cast<vec8 *>(sb + kl[i]) = kst[i];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (VKEYS == 4) {
                T quad[4] = {vst[0][e], vst[1][e], vst[VKEYS - 2][e], vst[VKEYS - 1][e]};
                *reinterpret_cast<uint64_t *>(sb + vl[e]) = *reinterpret_cast<const uint64_t *>(quad);
            } else {
                T pair[2] = {vst[0][e], vst[1][e]};
                *reinterpret_cast<uint32_t *>(sb + vl[e]) = *reinterpret_cast<const uint32_t *>(pair);
            }
        }
        if (tid < BN) *reinterpret_cast<float *>(sb + K_BYTES + V_BYTES + tid * 4) = bias_st;
    };

    // ---- running state of this lane's query row
    float m_i = -INFINITY, l_i = 0.0f;
    f32x16 o_acc[DB];
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) o_acc[d][v] = 0.0f;

    const float c = p.scale_log2;

    // LDS byte offsets of this lane's operand fragments inside a sub-tile, minus the 32-row block term
    // (a compile-time constant that folds into the instruction offset).  The swizzle phase of a row depends
    // only on its low bits, so it is the same in every 32-row block.
    int k_off[KS], v_off[SUB / 16];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_off[ks] = swz_offset<KROW>(lr, 2 * ks + lh);
#pragma unroll
    for (int ps = 0; ps < SUB / 16; ++ps) v_off[ps] = swz_offset<VROW>(lr, 2 * ps + lh);
    const int64_t mask_row = mask_base + (int64_t)min(my_m, M - 1) * (MASK_MODE == MASK_MATRIX ? p.ms[2] : 0);

    if (nt > 0) {
        gload(use_list ? __builtin_amdgcn_readfirstlane(tile_list[0]) : 0);
        lstore(0);
    }
    // Every load issued so far (Q fragments included) has to have landed before the loop: otherwise the
    // compiler must assume they may still be in flight at the first MFMA of each iteration and waits there for
    // the vector-memory counter to drain, which also drains the prefetch of the next tile issued just before.
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    __syncthreads();

    for (int it = 0; it < nt; ++it) {
        // tile indices come from LDS: tell the compiler they are wave-uniform, otherwise every buffer load that
        // takes them as a scalar offset is wrapped in a waterfall loop
        const int tile = use_list ? __builtin_amdgcn_readfirstlane(tile_list[it]) : it;
        const int n0 = tile * BN;
        if (it + 1 < nt) gload(use_list ? __builtin_amdgcn_readfirstlane(tile_list[it + 1]) : it + 1);

        const unsigned char *kb = smem + (it & 1) * STAGE;
        const unsigned char *vb = kb + K_BYTES;
        const float *colbias = reinterpret_cast<const float *>(kb + K_BYTES + V_BYTES);

        // The tile is consumed in sub-tiles of SUB keys, each a complete online-softmax step, which keeps
        // the live score registers at SUB/2 per lane.
        const bool tile_general = (MASK_MODE == MASK_MATRIX) || (n0 + BN > N) ||
                                  (MASK_MODE == MASK_VECTOR && (use_list ? (__builtin_amdgcn_readfirstlane(tile_cls[tile]) != 0) : true));
#pragma nounroll
        for (int sub = 0; sub < BN / SUB; ++sub) {
            const int ns0 = n0 + sub * SUB;  // first key of the sub-tile
            // a wave whose 32 rows all lie above this causal sub-tile has nothing to do in it
            if (CAUSAL && ns0 > m_wave0 + 31) break;
            if (ns0 >= N) break;
            const unsigned char *ksub = kb + sub * SUB * KROW;
            // along a Vᵀ row the sub-tile is SUB/8 chunks further; under the XOR swizzle that is an XOR too
            const int vsub_xor = sub * (SUB / 8) * 16;

            // ---- Sᵀ = K · Qᵀ.  MFMA phases run at raised wave priority: a wave that is ready to feed the matrix
            // pipe goes first, the other waves of the SIMD fill the gaps with their softmax VALU work.
            f32x16 s_acc[NBS];
            __builtin_amdgcn_s_setprio(2);
#pragma unroll
            for (int nb = 0; nb < NBS; ++nb) {
#pragma unroll
                for (int v = 0; v < 16; ++v) s_acc[nb][v] = 0.0f;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const vec8 kf = *reinterpret_cast<const vec8 *>(ksub + nb * 32 * KROW + k_off[ks]);
                    s_acc[nb] = mfma32(kf, qf[ks], s_acc[nb]);
                }
            }

            __builtin_amdgcn_s_setprio(0);

            // ---- online softmax on this lane's row; key of s_acc[nb][v] is ns0 + 32 nb + 8 (v/4) + 4 lh + (v%4)
            const bool general = tile_general || (CAUSAL && (ns0 + SUB - 1 > m_wave0));
            float mx = -INFINITY;
            if (general) {
#pragma unroll
                for (int nb = 0; nb < NBS; ++nb) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const int nl = sub * SUB + nb * 32 + g * 8 + lh * 4;  // key index inside the tile
                        const f32x4 cb = *reinterpret_cast<const f32x4 *>(colbias + nl);
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            float sv = s_acc[nb][g * 4 + r] * c + cb[r];
                            if (MASK_MODE == MASK_MATRIX) {
                                const int n = min(n0 + nl + r, N - 1);
                                sv += scale_mask(load_mask_value(p.mask, p.mask_dtype, mask_row + n * p.ms[3]), p.clamp);
                            }
                            if (CAUSAL && (n0 + nl + r > my_m)) sv = -INFINITY;
                            s_acc[nb][g * 4 + r] = sv;
                            mx = fmaxf(mx, sv);
                        }
                    }
                }
            } else {
#pragma unroll
                for (int nb = 0; nb < NBS; ++nb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s_acc[nb][v]);
                mx *= c;  // c > 0 on this path (checked by the host)
            }
            mx = halves32_max(mx);  // the other 16-key half of every 32-key block lives in lane ^ 32
            // m_i is the exponent REFERENCE of this row, not necessarily its running maximum: it is only moved (and
            // the accumulator and row sum rescaled) when the new maximum exceeds it by more than 2^8, so probabilities
            // stay <= 256 — exact in fp32 and well inside the 16-bit range — and after the first tiles the rescale
            // almost never runs.  The final O / l is independent of the reference.
            if (__builtin_amdgcn_ballot_w64(mx > m_i + kRescaleThreshold) != 0) {
                const float m_new = fmaxf(m_i, mx);
                const float alpha = __builtin_amdgcn_exp2f(m_i - ((m_new == -INFINITY) ? 0.0f : m_new));
                l_i *= alpha;
#pragma unroll
                for (int d = 0; d < DB; ++d)
#pragma unroll
                    for (int v = 0; v < 16; ++v) o_acc[d][v] *= alpha;
                m_i = m_new;
            }
            const float m_use = (m_i == -INFINITY) ? 0.0f : m_i;
            // exponentiate in place; the row sum is taken below from the ROUNDED probabilities (two per
            // v_dot2c), i.e. from exactly the values that enter P·V
            if (general) {
#pragma unroll
                for (int nb = 0; nb < NBS; ++nb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) s_acc[nb][v] = __builtin_amdgcn_exp2f(s_acc[nb][v] - m_use);
            } else {
#pragma unroll
                for (int nb = 0; nb < NBS; ++nb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) s_acc[nb][v] = __builtin_amdgcn_exp2f(s_acc[nb][v] * c - m_use);
            }
            float rs = 0.0f;

            // ---- Oᵀ += Vᵀ · Pᵀ
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int ps = 0; ps < SUB / 16; ++ps) {
                const int nb = ps >> 1, half8 = (ps & 1) * 8;
                u32x4 pk;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    pk[j] = pack2<T>(s_acc[nb][half8 + 2 * j], s_acc[nb][half8 + 2 * j + 1]);
                    rs = pair_sum_acc<T>(pk[j], rs);
                }
                const vec8 pf = __builtin_bit_cast(vec8, pk);
#pragma unroll
                for (int d = 0; d < DB; ++d) {
                    const vec8 vf = *reinterpret_cast<const vec8 *>(vb + d * 32 * VROW + (v_off[ps] ^ vsub_xor));
                    o_acc[d] = mfma32(vf, pf, o_acc[d]);
                }
            }
            __builtin_amdgcn_s_setprio(0);
            l_i += rs;
        }

        if (it + 1 < nt) lstore((it + 1) & 1);
        __syncthreads();
    }

    // ---- normalise and store: lane holds features 32 d + 16 lh + (0..15) of row my_m
    const float l_tot = halves32_sum(l_i);
    const float inv_l = 1.0f / l_tot;
    if (my_m < M) {
        T *orow = op + (int64_t)my_m * p.os[2] + lh * 16;
#pragma unroll
        for (int d = 0; d < DB; ++d) {
            u32x4 p0, p1;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                p0[j] = pack2<T>(o_acc[d][2 * j] * inv_l, o_acc[d][2 * j + 1] * inv_l);
                p1[j] = pack2<T>(o_acc[d][8 + 2 * j] * inv_l, o_acc[d][8 + 2 * j + 1] * inv_l);
            }
            *reinterpret_cast<u32x4 *>(orow + d * 32) = p0;
            *reinterpret_cast<u32x4 *>(orow + d * 32 + 8) = p1;
        }
    }
}

// ----------------------------------------------------------------------------------------------------
// Scalar kernel: any strides, any head size up to 256.  One wave per query row; keys are taken 64 at a time
// (lane <-> key for the scores, lane <-> feature for the output).
// ----------------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(64) attention_scalar_kernel(const AttnParams p, int D, int mask_mode, int causal) {
    __shared__ float qs[256];
    __shared__ float ps[64];
    const int m = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x;
    const T *qp = static_cast<const T *>(p.q) + b * p.qs[0] + h * p.qs[1] + (int64_t)m * p.qs[2];
    const T *kp = static_cast<const T *>(p.k) + b * p.ks[0] + h * p.ks[1];
    const T *vp = static_cast<const T *>(p.v) + b * p.vs[0] + h * p.vs[1];
    T *op = static_cast<T *>(p.o) + b * p.os[0] + h * p.os[1] + (int64_t)m * p.os[2];
    const int64_t mask_base = mask_mode != MASK_NONE ? b * p.ms[0] + h * p.ms[1] + (mask_mode == MASK_MATRIX ? (int64_t)m * p.ms[2] : 0) : 0;
    for (int d = lane; d < D; d += 64) qs[d] = to_float(qp[d * p.qs[3]]);
    __syncthreads();
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    float m_i = -INFINITY, l_i = 0.0f;
    const int n_end = causal ? min(p.N, m + 1) : p.N;
    for (int n0 = 0; n0 < n_end; n0 += 64) {
        const int n = n0 + lane;
        float s = -INFINITY;
        if (n < n_end) {
            float dot = 0.0f;
            const T *kr = kp + (int64_t)n * p.ks[2];
            for (int d = 0; d < D; ++d) dot += qs[d] * to_float(kr[d * p.ks[3]]);
            s = dot * p.scale_log2;
            if (mask_mode != MASK_NONE)
                s += scale_mask(load_mask_value(p.mask, p.mask_dtype, mask_base + n * p.ms[3]), p.clamp);
        }
        float mx = s;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        const float m_new = fmaxf(m_i, mx);
        const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
        const float alpha = __builtin_amdgcn_exp2f(m_i - m_use);
        float pv = __builtin_amdgcn_exp2f(s - m_use);
        // P is rounded to the storage dtype before P·V, the row sum uses the unrounded value (as the reference)
        const float rs = wave_sum(pv);
        l_i = l_i * alpha + rs;
        m_i = m_new;
        __syncthreads();
        ps[lane] = to_float(from_float<T>(pv));
        __syncthreads();
        const int cnt = min(64, n_end - n0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int d = lane + 64 * j;
            if (d < D) {
                float a = acc[j] * alpha;
                for (int i = 0; i < cnt; ++i) a += ps[i] * to_float(vp[(int64_t)(n0 + i) * p.vs[2] + d * p.vs[3]]);
                acc[j] = a;
            }
        }
    }
    const float inv_l = 1.0f / l_i;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int d = lane + 64 * j;
        if (d < D) op[d * p.os[3]] = from_float<T>(acc[j] * inv_l);
    }
}

// ----------------------------------------------------------------------------------------------------
// host dispatch
// ----------------------------------------------------------------------------------------------------
template <typename T, int D, int BN, int SUB, int WPE>
static void launch_mfma(const AttnParams &p, int mask_mode, bool causal, hipStream_t st) {
    const int bh_padded = ((p.B * p.H + 7) / 8) * 8;
    dim3 grid((unsigned)(bh_padded * p.nq_tiles)), block(256);
#define KERNL_ATTN_LAUNCH(MM, C) hipLaunchKernelGGL((attention_mfma_kernel<T, D, BN, SUB, WPE, MM, C>), grid, block, 0, st, p)
    if (mask_mode == MASK_NONE) {
        if (causal) KERNL_ATTN_LAUNCH(MASK_NONE, true);
        else KERNL_ATTN_LAUNCH(MASK_NONE, false);
    } else if (mask_mode == MASK_VECTOR) {
        if (causal) KERNL_ATTN_LAUNCH(MASK_VECTOR, true);
        else KERNL_ATTN_LAUNCH(MASK_VECTOR, false);
    } else {
        if (causal) KERNL_ATTN_LAUNCH(MASK_MATRIX, true);
        else KERNL_ATTN_LAUNCH(MASK_MATRIX, false);
    }
#undef KERNL_ATTN_LAUNCH
}

int g_attention_force_scalar = 0;  // test hook: route everything through the scalar kernel
int g_attention_variant = 0;       // tuning hook: tile shape of the head-size-64 MFMA kernel

}  // namespace kernl

extern "C" void kernl_attention_force_scalar(int on) { kernl::g_attention_force_scalar = on; }
extern "C" void kernl_attention_set_variant(int which) { kernl::g_attention_variant = which; }

extern "C" int kernl_attention_fwd(const void *q, const void *k, const void *v, void *out, const void *mask,
                                   int64_t B, int64_t H, int64_t M, int64_t N, int64_t D,
                                   const int64_t q_strides[4], const int64_t k_strides[4],
                                   const int64_t v_strides[4], const int64_t o_strides[4],
                                   const int64_t mask_sizes[4], const int64_t mask_strides[4], int mask_dtype,
                                   float sm_scale, int is_causal, float mask_min_clamp, int dtype, void *stream) {
    using namespace kernl;
    if (q == nullptr || k == nullptr || v == nullptr || out == nullptr || q_strides == nullptr ||
        k_strides == nullptr || v_strides == nullptr || o_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "attention: q, k, v, out and their strides must not be NULL");
    if (B < 0 || H <= 0 || M < 0 || N <= 0 || D <= 0)
        return set_error(KERNL_ERR_INVALID_ARG, "attention: bad sizes B=%lld H=%lld M=%lld N=%lld D=%lld",
                         (long long)B, (long long)H, (long long)M, (long long)N, (long long)D);
    if (dtype != KERNL_F16 && dtype != KERNL_BF16)
        return set_error(KERNL_ERR_UNSUPPORTED, "attention: only f16 and bf16 are supported, got dtype %d", dtype);
    if (B * H > (1 << 24) || M > (1 << 24) || N > (1 << 24))
        return set_error(KERNL_ERR_UNSUPPORTED, "attention: sizes too large");
    int mask_mode = MASK_NONE;
    AttnParams p;
    if (mask != nullptr) {
        if (mask_sizes == nullptr || mask_strides == nullptr)
            return set_error(KERNL_ERR_INVALID_ARG, "attention: mask given without sizes/strides");
        if (mask_sizes[0] != B && mask_sizes[0] != 1)
            return set_error(KERNL_ERR_INVALID_ARG, "attention: incompatible broadcast batch dimension of the mask");
        if (mask_sizes[1] != H && mask_sizes[1] != 1)
            return set_error(KERNL_ERR_INVALID_ARG, "attention: incompatible broadcast heads dimension of the mask");
        if (mask_sizes[2] != M && mask_sizes[2] != 1)
            return set_error(KERNL_ERR_INVALID_ARG, "attention: incompatible broadcast m_size dimension of the mask");
        if (mask_sizes[3] != N)
            return set_error(KERNL_ERR_INVALID_ARG, "attention: last size of the mask must equal the key count");
        if (mask_dtype != KERNL_F16 && mask_dtype != KERNL_BF16 && mask_dtype != KERNL_F32)
            return set_error(KERNL_ERR_UNSUPPORTED, "attention: unknown mask dtype %d", mask_dtype);
        // a query dimension of size 1 — or one that is a stride-0 broadcast — means one value per key
        mask_mode = (mask_sizes[2] == 1 || mask_strides[2] == 0) ? MASK_VECTOR : MASK_MATRIX;
        p.ms[0] = mask_sizes[0] == 1 ? 0 : mask_strides[0];
        p.ms[1] = mask_sizes[1] == 1 ? 0 : mask_strides[1];
        p.ms[2] = mask_sizes[2] == 1 ? 0 : mask_strides[2];
        p.ms[3] = mask_strides[3];
    } else {
        p.ms[0] = p.ms[1] = p.ms[2] = p.ms[3] = 0;
    }
    if (B == 0 || M == 0) return KERNL_OK;

    p.q = q; p.k = k; p.v = v; p.o = out; p.mask = mask;
    p.B = (int)B; p.H = (int)H; p.M = (int)M; p.N = (int)N;
    for (int i = 0; i < 4; ++i) {
        p.qs[i] = q_strides[i]; p.ks[i] = k_strides[i]; p.vs[i] = v_strides[i]; p.os[i] = o_strides[i];
    }
    p.mask_dtype = mask_dtype;
    p.sm_scale = sm_scale;
    p.scale_log2 = sm_scale * 1.4426950408889634f;
    p.clamp = mask_min_clamp;
    p.nq_tiles = (int)((M + 127) / 128);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool causal = is_causal != 0;

    auto rows_ok = [](const void *ptr, const int64_t s[4]) {
        return s[3] == 1 && s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0 && aligned16(ptr);
    };
    const bool mfma_ok = !g_attention_force_scalar && (D == 64 || D == 128) && sm_scale > 0.0f &&
                         rows_ok(q, q_strides) && rows_ok(k, k_strides) && rows_ok(v, v_strides) &&
                         rows_ok(out, o_strides) && (int64_t)((B * H + 7) / 8) * 8 * p.nq_tiles < (1ll << 31) &&
                         k_strides[2] > 0 && v_strides[2] > 0 &&  // one head's K / V extent must fit 31-bit byte offsets
                         (N + 128) * k_strides[2] < (1ll << 30) && (N + 128) * v_strides[2] < (1ll << 30);
    if (mfma_ok) {
        if (dtype == KERNL_F16) {
            if (D == 64) {
                // measured on config 1: 64-key tiles at 3 waves/SIMD win without causal masking (finer skipping of
                // padded key tiles, more waves to interleave), 128-key tiles at 2 waves/SIMD win with it
                int variant = g_attention_variant;
                if (variant == 0) variant = (causal || mask_mode == MASK_MATRIX) ? 3 : 1;
                if (variant == 1) launch_mfma<f16, 64, 64, 64, 3>(p, mask_mode, causal, st);
                else if (variant == 2) launch_mfma<f16, 64, 64, 64, 2>(p, mask_mode, causal, st);
                else launch_mfma<f16, 64, 128, 64, 2>(p, mask_mode, causal, st);
            }
            else launch_mfma<f16, 128, 64, 32, 2>(p, mask_mode, causal, st);
        } else {
            if (D == 64) launch_mfma<bf16, 64, 128, 64, 2>(p, mask_mode, causal, st);
            else launch_mfma<bf16, 128, 64, 32, 2>(p, mask_mode, causal, st);
        }
        return check_launch("attention (mfma)");
    }
    if (D > 256) return set_error(KERNL_ERR_UNSUPPORTED, "attention: head size %lld > 256", (long long)D);
    if (H > 65535 || B > 65535)
        return set_error(KERNL_ERR_UNSUPPORTED, "attention: scalar path needs B, H <= 65535");
    dim3 grid((unsigned)M, (unsigned)H, (unsigned)B);
    if (dtype == KERNL_F16)
        hipLaunchKernelGGL((attention_scalar_kernel<f16>), grid, dim3(64), 0, st, p, (int)D, mask_mode, (int)causal);
    else
        hipLaunchKernelGGL((attention_scalar_kernel<bf16>), grid, dim3(64), 0, st, p, (int)D, mask_mode, (int)causal);
    return check_launch("attention (scalar)");
}
