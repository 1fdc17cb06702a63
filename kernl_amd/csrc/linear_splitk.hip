// Linear layer for a FEW rows of x (at most 64: batched decoding steps, pooled outputs), as a stream-K product.
//
//     out[M,N] = act(x[M,K] · w[N,K]ᵀ + bias[N]) (+ residual[M,N])
//
// Same semantics as the fused linear kernels (reference: src/kernl/implementations/linear_layer.py:92-210: fp32
// accumulation, bias added in fp32, activation on the fp32 value, one rounding).  The decomposition is the one of the
// reference's stream-K experiment (experimental/streamk/kernel_streamk.py: every workgroup takes an equal, contiguous
// share of the (output tile, k-step) iteration space and tiles cut by a share boundary are completed from partial
// sums), with a second small kernel instead of its spin locks.
//
// The weight is the only large operand and the job is to stream it ONCE at HBM speed with every CU — but with this many
// rows x matters too: a workgroup that owns few columns re-reads all of x from L2 (the kernel that gives every workgroup
// 16 to 64 columns and all of K moves 2 to 4 times the weight's bytes in x, and L2 delivers them at about 11 TB/s).
// Work is cut into UNITS: one 64-wide chunk of K for one tile of 128 output columns.  The units, tile after tile, are
// dealt in equal contiguous runs to at most 256 workgroups — one round of one workgroup per CU (measured: a grid of
// 1.25 or 1.5 rounds takes up to 1.5x the time of one round, and a grid that leaves a third of the CUs idle 1.3x).
// A workgroup of 8 waves walks its run: the x rows of two (16 rows: four) units at a time go through LDS (16-byte pieces,
// XOR-swizzled for the MFMA operand reads; two stages, one barrier per group) and every wave feeds the 16 weight rows it owns
// of the unit's tile from global memory straight into v_mfma_f32_16x16x32 — weights on the A side, x on the B side,
// lane (r = lane % 16, g = lane / 16) supplying k = 16 g + 8 s .. + 7 of the chunk in step s on both sides.  The
// prefetch depth is in registers: a ring of 4 (8) units of weight fragments per wave and the thread's share of the next
// group of x.
//
// Where a run ends or crosses into the next tile, the workgroup writes its fp32 partial tile to the workspace (slot
// `workgroup + tile`: unique, because runs and tiles advance together; lane-major, 16 bytes per lane and block, coalesced
// both ways) and the second kernel adds a tile's slots in workgroup order and runs the epilogue: the result does not
// depend on timing.  When a run is exactly one tile (about 200 to 256 tiles), the first kernel runs the epilogue itself
// and nothing else is launched.  (One launch with a ticket per tile — the last workgroup to arrive adds — was measured
// too: partial tiles then have to travel as agent-scope stores and loads, and the three dependent round trips store /
// ticket / load cost what the second launch costs, 4 to 5 us; a release fence instead walks the whole L2 and costs 5x
// the kernel.  Two launches need no counters, hence no workspace that must stay zeroed between calls.)
#include <type_traits>

#include "activations.h"
#include "common.h"

namespace kernl {

static constexpr int kFewRowWaves = 8;                      // waves per workgroup
static constexpr int kFewRowTile = 16 * kFewRowWaves;      // output columns per tile
static constexpr int kFewRowMaxGrid = 256;                 // one workgroup per CU

struct FewRowPlan {
    int tiles;        // column tiles
    int nch;          // chunks of 64 k per tile
    int run;          // units per workgroup
    int grid;         // workgroups
    bool direct;      // every run is exactly one tile: no partial sums
    int64_t partial_bytes;
};

static inline int fewrow_row_blocks(int64_t M) { return M <= 16 ? 1 : M <= 32 ? 2 : 4; }

static FewRowPlan fewrow_plan(int64_t M, int64_t N, int64_t K) {
    FewRowPlan p;
    p.nch = (int)(K / 64);
    p.tiles = (int)((N + kFewRowTile - 1) / kFewRowTile);
    const int64_t total = (int64_t)p.tiles * p.nch;
    int64_t run = (total + kFewRowMaxGrid - 1) / kFewRowMaxGrid;
    if (run < 4) run = 4;
    // whole tiles per workgroup where that costs at most a fifth of the CUs: no partial sums, one launch
    if (p.tiles <= kFewRowMaxGrid && p.tiles * 5 >= kFewRowMaxGrid * 4) run = p.nch;
    p.run = (int)run;
    p.grid = (int)((total + run - 1) / run);
    p.direct = p.run == p.nch;
    p.partial_bytes = p.direct ? 0 : (int64_t)(p.grid + p.tiles) * kFewRowTile * 16 * fewrow_row_blocks(M) * 4;
    return p;
}

// Epilogue of one 16 x 16 block of one lane: elements e = 0..3 of `acc` are output columns n .. n + 3 of x row m.
template <typename T>
__device__ __forceinline__ void fewrow_epilogue(const f32x4_acc &acc, int m, int n, const T *__restrict__ bias,
                                                T *__restrict__ out, int M, int N, int64_t out_rs, int64_t out_cs, int act,
                                                const T *__restrict__ residual, int64_t res_rs, int64_t res_cs) {
    if (n >= N || m >= M) return;
    float y[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float b = bias != nullptr ? to_float(bias[min(n + e, N - 1)]) : 0.0f;
        y[e] = apply_act16(acc[e] + b, act);
        if (residual != nullptr && n + e < N) y[e] += to_float(residual[(int64_t)m * res_rs + (int64_t)(n + e) * res_cs]);
    }
    if (out_cs == 1 && (out_rs & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0 && n + 3 < N) {
        uint2 v;
        v.x = pack2<T>(y[0], y[1]);
        v.y = pack2<T>(y[2], y[3]);
        *reinterpret_cast<uint2 *>(out + (int64_t)m * out_rs + n) = v;
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (n + e < N) out[(int64_t)m * out_rs + (int64_t)(n + e) * out_cs] = from_float<T>(y[e]);
    }
}

template <typename T, int MB, int WAVES, int GC, int RING>
__global__ void __launch_bounds__(64 * WAVES)
linear_fewrow_kernel(const T *__restrict__ X, const T *__restrict__ W, const T *__restrict__ bias, T *__restrict__ out,
                     float *__restrict__ part, int M, int N, int K, int64_t ldx, int64_t out_rs, int64_t out_cs, int act,
                     int tiles, int run, int direct, const T *__restrict__ residual, int64_t res_rs, int64_t res_cs) {
    typedef typename Vec8<T>::type vec8;
    static_assert(RING % (2 * GC) == 0, "a round of RING units is a whole number of stage pairs");
    constexpr int THREADS = 64 * WAVES;
    constexpr int MP = 16 * MB;                 // rows of x, padded to whole MFMA blocks
    constexpr int CHUNK_BYTES = MP * 128;       // one staged chunk of x
    constexpr int XP = GC * MP * 8 / THREADS;   // 16-byte pieces of a group of x per thread
    static_assert(GC * MP * 8 % THREADS == 0 && XP >= 1, "every thread stages the same number of pieces");
    __shared__ __attribute__((aligned(16))) unsigned char xs[2][GC * CHUNK_BYTES];

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int nch = K / 64;
    const int total = tiles * nch;              // the host keeps the number of units below 2^31
    const int u_begin = (int)blockIdx.x * run;
    const int n_units = min(run, total - u_begin);
    const int first_tile = u_begin / nch, first_chunk = u_begin - first_tile * nch;

    // ---- weights: a ring of RING units per wave.  The request cursor walks the run and stops at its last unit
    // (requests past the end fetch that unit again and are never used): no branch around a load, so the compiler's
    // wait counts are exact and the ring really is in flight.  Columns beyond N repeat the last weight row.
    vec8 wf[RING][2];
    int rq_left = n_units - 1;                  // units the cursor may still advance by
    int rq_tile = first_tile, rq_chunk = first_chunk;
    auto weight_row = [&](int tile) __attribute__((always_inline)) -> const T * {
        return W + (int64_t)min(tile * (16 * WAVES) + 16 * wave + r, N - 1) * K + 16 * g;
    };
    const T *wrow = weight_row(rq_tile);
    auto request_w = [&](int slot) __attribute__((always_inline)) {
        const T *src = wrow + (int64_t)rq_chunk * 64;
        wf[slot][0] = *reinterpret_cast<const vec8 *>(src);
        wf[slot][1] = *reinterpret_cast<const vec8 *>(src + 8);
        if (rq_left > 0) {      // uniform; address arithmetic only
            --rq_left;
            if (++rq_chunk == nch) {
                rq_chunk = 0;
                wrow = weight_row(++rq_tile);
            }
        }
    };

    // ---- x: piece i of a thread is 16-byte piece (q & 7) of row (q >> 3) % MP of the group's unit q / (8 MP),
    // q = tid + THREADS i.  Rows beyond M repeat the last row; units past the end of the run repeat its last unit.
    vec8 xr[XP];
    const T *xrow[XP];
    int xunit[XP], xdst[XP];
#pragma unroll
    for (int i = 0; i < XP; ++i) {
        const int q = tid + THREADS * i, j = q / (MP * 8), row = (q >> 3) % MP, piece = q & 7;
        xrow[i] = X + (int64_t)min(row, M - 1) * ldx + piece * 8;
        xunit[i] = __builtin_amdgcn_readfirstlane(j);   // a wave's 64 pieces belong to one unit
        xdst[i] = j * CHUNK_BYTES + swz_offset<128>(row, piece);
    }
    // (the chunk of a group's first unit is kept as a running value: no division in the loop)
    const int last_chunk = (first_chunk + n_units - 1) % nch;
    int xg_unit = 0, xg_chunk = first_chunk;    // first unit of the group the next request is for, and its chunk
    auto request_x = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            int c = xg_chunk + xunit[i];
            c = c >= nch ? c - nch : c;
            c = xg_unit + xunit[i] < n_units ? c : last_chunk;
            xr[i] = *reinterpret_cast<const vec8 *>(xrow[i] + (int64_t)c * 64);
        }
        xg_unit += GC;
        xg_chunk += GC;
        xg_chunk = xg_chunk >= nch ? xg_chunk - nch : xg_chunk;
    };
    auto stage_x = [&](int stage) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < XP; ++i) *reinterpret_cast<vec8 *>(xs[stage] + xdst[i]) = xr[i];
    };
    int xoff[MB][2];   // this lane's operand fragments inside a staged chunk
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int s = 0; s < 2; ++s) xoff[mb][s] = swz_offset<128>(16 * mb + r, 2 * g + s);

    f32x4_acc acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = f32x4_acc{0.0f, 0.0f, 0.0f, 0.0f};

    // ---- consumer: unit i of the run is chunk `c_chunk` of tile `c_tile`
    int c_tile = first_tile, c_chunk = first_chunk;
    // Partial tile of this workgroup for tile `tile`: slot blockIdx + tile.  The stores are issued from assembly: a
    // store the compiler knows of, inside a branch of the loop, makes it wait for EVERY outstanding load at the next
    // use of a fragment (loads and stores share one counter that it then treats as unordered).
    auto flush_partial = [&](int tile) __attribute__((always_inline)) {
        float4 *dst = reinterpret_cast<float4 *>(part) + (((int64_t)blockIdx.x + tile) * (WAVES * MB) + wave * MB) * 64 + lane;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 1" ::"v"(dst + mb * 64), "v"(acc[mb]) : "memory");
            acc[mb] = f32x4_acc{0.0f, 0.0f, 0.0f, 0.0f};
        }
    };
    // unit i of the run sits in ring slot i % RING; its x is chunk (i % RING) % GC of stage ((i % RING) / GC) % 2
    auto unit_step = [&](int i, int slot) __attribute__((always_inline)) {
        if (i < n_units) {   // uniform over the workgroup; no load of global memory inside
            const unsigned char *chunk = xs[(slot / GC) & 1] + (slot % GC) * CHUNK_BYTES;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const vec8 x0 = *reinterpret_cast<const vec8 *>(chunk + xoff[mb][0]);
                const vec8 x1 = *reinterpret_cast<const vec8 *>(chunk + xoff[mb][1]);
                acc[mb] = mfma16(wf[slot][0], x0, acc[mb]);
                acc[mb] = mfma16(wf[slot][1], x1, acc[mb]);
            }
            if (++c_chunk == nch || i == n_units - 1) {
                if (!direct) flush_partial(c_tile);
                c_chunk = 0;
                ++c_tile;
            }
        }
    };

    // prologue: x of group 0 into stage 0, x of group 1 on its way, RING units of weights requested
    request_x();
#pragma unroll
    for (int slot = 0; slot < RING; ++slot) request_w(slot);
    stage_x(0);
    request_x();
    __syncthreads();
    // rounds of RING units that refill the ring ...
    int i0 = 0;
    for (; i0 + RING < n_units; i0 += RING) {
#pragma unroll
        for (int slot = 0; slot < RING; ++slot) {
            unit_step(i0 + slot, slot);
            request_w(slot);   // the unit RING further on
            if ((slot + 1) % GC == 0) {
                // end of a group: the other stage was last read one group ago and every wave has passed a barrier since
                stage_x(((slot / GC) & 1) ^ 1);
                request_x();
                __syncthreads();
            }
        }
    }
    // ... and the last round, which requests nothing
#pragma unroll
    for (int slot = 0; slot < RING; ++slot) {
        unit_step(i0 + slot, slot);
        if ((slot + 1) % GC == 0 && slot + 1 < RING) {
            // (the request stays outside the run-time test: a load inside a branch costs exact wait counts after it)
            const bool more = i0 + slot + 1 < n_units;   // uniform
            if (more) stage_x(((slot / GC) & 1) ^ 1);
            if (slot + 1 + GC < RING) request_x();
            if (more) __syncthreads();
        }
    }
    if (!direct) return;
    // a run of exactly one tile: element e of a lane is output column n + e of x row 16 mb + r
    const int n = first_tile * (16 * WAVES) + 16 * wave + 4 * g;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
        fewrow_epilogue<T>(acc[mb], 16 * mb + r, n, bias, out, M, N, out_rs, out_cs, act, residual, res_rs, res_cs);
}

// Adds the partial tiles of every tile in workgroup order and runs the epilogue.  One thread per 16-byte element of a
// tile (the same lane-to-element map as above).  Tile t holds units [t nch, (t + 1) nch), i.e. it was touched by
// workgroups (t nch) / run .. ((t + 1) nch - 1) / run, and workgroup w left its share in slot w + t.
template <typename T, int MB, int WAVES>
__global__ void __launch_bounds__(256)
linear_fewrow_reduce_kernel(const float *__restrict__ part, const T *__restrict__ bias, T *__restrict__ out, int M, int N,
                            int64_t out_rs, int64_t out_cs, int act, int tiles, int nch, int run,
                            const T *__restrict__ residual, int64_t res_rs, int64_t res_cs) {
    constexpr int TILE_ELEMS = WAVES * MB * 64;                      // 16-byte elements of one partial tile
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)tiles * TILE_ELEMS) return;
    const int tile = (int)(idx / TILE_ELEMS), e = (int)(idx - (int64_t)tile * TILE_ELEMS);
    const int lane = e & 63, mb = (e >> 6) % MB, wave = (e >> 6) / MB;
    const int w_first = (tile * nch) / run, w_last = ((tile + 1) * nch - 1) / run;   // units fit 31 bits
    const float4 *theirs = reinterpret_cast<const float4 *>(part) + ((int64_t)w_first + tile) * TILE_ELEMS + e;
    f32x4_acc acc = {0.0f, 0.0f, 0.0f, 0.0f};
    const int n_slots = w_last - w_first + 1;
    int s = 0;
    for (; s + 4 <= n_slots; s += 4) {   // four loads in flight, added in workgroup order
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = theirs[(int64_t)(s + u) * TILE_ELEMS];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            acc[0] += v[u].x;
            acc[1] += v[u].y;
            acc[2] += v[u].z;
            acc[3] += v[u].w;
        }
    }
    for (; s < n_slots; ++s) {
        const float4 v = theirs[(int64_t)s * TILE_ELEMS];
        acc[0] += v.x;
        acc[1] += v.y;
        acc[2] += v.z;
        acc[3] += v.w;
    }
    fewrow_epilogue<T>(acc, 16 * mb + (lane & 15), tile * (16 * WAVES) + 16 * wave + 4 * (lane >> 4), bias, out, M, N, out_rs,
                       out_cs, act, residual, res_rs, res_cs);
}

template <typename T>
static void launch_fewrow(const void *x, const void *w, const void *bias, const void *residual, void *out, void *workspace,
                          const FewRowPlan &p, int M, int N, int K, int64_t ldx, int64_t out_rs, int64_t out_cs,
                          int64_t res_rs, int64_t res_cs, int act, hipStream_t st) {
    float *part = static_cast<float *>(workspace);
    // x groups of 2 units and a ring of 4 measured best (by 0.5 to 1.4 us against 4 and 8); 16 rows of x are too few
    // pieces for 512 threads to stage 2 units at a time
#define KERNL_FEWROW(MBV)                                                                                               \
    do {                                                                                                                \
        hipLaunchKernelGGL((linear_fewrow_kernel<T, MBV, kFewRowWaves, (MBV == 1 ? 4 : 2), (MBV == 1 ? 8 : 4)>),        \
                           dim3((unsigned)p.grid),                                                                      \
                           dim3(64 * kFewRowWaves), 0, st, static_cast<const T *>(x), static_cast<const T *>(w),        \
                           static_cast<const T *>(bias), static_cast<T *>(out), part, M, N, K, ldx, out_rs, out_cs,    \
                           act, p.tiles, p.run, p.direct ? 1 : 0, static_cast<const T *>(residual), res_rs, res_cs);   \
        if (!p.direct)                                                                                                  \
            hipLaunchKernelGGL((linear_fewrow_reduce_kernel<T, MBV, kFewRowWaves>),                                     \
                               dim3((unsigned)(((int64_t)p.tiles * kFewRowWaves * MBV * 64 + 255) / 256)), dim3(256), 0, \
                               st, part, static_cast<const T *>(bias), static_cast<T *>(out), M, N, out_rs, out_cs,     \
                               act, p.tiles, p.nch, p.run, static_cast<const T *>(residual), res_rs, res_cs);           \
    } while (0)
    if (M <= 16) KERNL_FEWROW(1);
    else if (M <= 32) KERNL_FEWROW(2);
    else KERNL_FEWROW(4);
#undef KERNL_FEWROW
}

}  // namespace kernl

extern "C" int64_t kernl_linear_fewrow_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    using namespace kernl;
    if (M <= 0 || M > 64 || N <= 0 || K < 256 || K % 64 != 0) return 0;
    return fewrow_plan(M, N, K).partial_bytes;
}

extern "C" int kernl_linear_fewrow_fwd(const void *x, const void *w, const void *bias, const void *residual, void *out,
                                       void *workspace, int64_t workspace_bytes, int64_t M, int64_t N, int64_t K,
                                       const int64_t x_strides[2], const int64_t out_strides[2],
                                       const int64_t residual_strides[2], int activation, int dtype, void *stream) {
    using namespace kernl;
    if (x == nullptr || w == nullptr || out == nullptr || x_strides == nullptr || out_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "few-row linear: x, w, out and their strides must not be NULL");
    if (residual != nullptr && residual_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "few-row linear: residual given without strides");
    if (M < 0 || N <= 0 || K <= 0 || workspace_bytes < 0)
        return set_error(KERNL_ERR_INVALID_ARG, "few-row linear: bad sizes M=%lld N=%lld K=%lld workspace=%lld", (long long)M,
                         (long long)N, (long long)K, (long long)workspace_bytes);
    if (activation < KERNL_ACT_NONE || activation > KERNL_ACT_SILU)
        return set_error(KERNL_ERR_INVALID_ARG, "few-row linear: unknown activation %d", activation);
    if (dtype != KERNL_F16 && dtype != KERNL_BF16)
        return set_error(KERNL_ERR_UNSUPPORTED, "few-row linear: only f16 and bf16 are supported, got dtype %d", dtype);
    if (M > 64 || K % 64 != 0 || K < 256 || N > (1 << 30) || K > INT32_MAX)
        return set_error(KERNL_ERR_UNSUPPORTED, "few-row linear: at most 64 rows of x and K a multiple of 64, at least 256 "
                         "(M=%lld K=%lld)", (long long)M, (long long)K);
    if (x_strides[1] != 1 || x_strides[0] % 8 != 0 || !aligned16(x) || !aligned16(w))
        return set_error(KERNL_ERR_UNSUPPORTED, "few-row linear: x needs unit feature stride and 16-byte aligned rows, the "
                         "weight a 16-byte aligned base");
    if (workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15) != 0)
        return set_error(KERNL_ERR_UNSUPPORTED, "few-row linear: the workspace must be 16-byte aligned");
    if (M == 0) return KERNL_OK;
    if (((N + kFewRowTile - 1) / kFewRowTile) * (K / 64) >= (int64_t)1 << 30)
        return set_error(KERNL_ERR_UNSUPPORTED, "few-row linear: N * K too large");
    const FewRowPlan p = fewrow_plan(M, N, K);
    if (!p.direct && (workspace == nullptr || workspace_bytes < p.partial_bytes))
        return set_error(KERNL_ERR_INVALID_ARG, "few-row linear: the workspace must hold %lld bytes "
                         "(kernl_linear_fewrow_workspace_bytes), got %lld", (long long)p.partial_bytes,
                         (long long)(workspace == nullptr ? 0 : workspace_bytes));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t res_rs = residual ? residual_strides[0] : 0, res_cs = residual ? residual_strides[1] : 0;
    if (dtype == KERNL_F16)
        launch_fewrow<f16>(x, w, bias, residual, out, workspace, p, (int)M, (int)N, (int)K, x_strides[0], out_strides[0],
                           out_strides[1], res_rs, res_cs, activation, st);
    else
        launch_fewrow<bf16>(x, w, bias, residual, out, workspace, p, (int)M, (int)N, (int)K, x_strides[0], out_strides[0],
                            out_strides[1], res_rs, res_cs, activation, st);
    return check_launch("linear (few rows, split K)");
}
