// Kernels and launchers of the fused linear layer, shared by linear.hip (dispatch, entry points, the 8-wave, skinny
// and FMA kernels), linear_wide.hip and linear_wide_half.hip.
#pragma once

// Fused linear layer for gfx950:  out[M,N] = act(x[M,K] · w[N,K]ᵀ + bias[N]).
//
// Semantics follow the reference kernel src/kernl/implementations/linear_layer.py:92-210: fp32 accumulation,
// bias added in fp32, optional store of the pre-activation, activation applied to the fp32 accumulator, one
// rounding to the output dtype.
//
// MFMA path (16-bit inputs, K-contiguous x): both operands are K-major, which is exactly what
// v_mfma_f32_32x32x16 wants (each lane supplies 8 consecutive k of one row), so tiles go HBM -> VGPR -> LDS
// with 16-byte accesses and no transposition.  The weight rows feed the MFMA "A" side and the activations the
// "B" side, i.e. the instruction produces a 32(n) x 32(m) block of outᵀ; together with the row permutation
// rowperm16 on the weight tile this leaves every lane holding 16 consecutive output columns of one output
// row, so bias loads and output stores are 16-byte vectors without any shuffle through LDS.
#include <type_traits>

#include "activations.h"
#include "common.h"

namespace kernl {

// The wide kernels are heavy to compile (dozens of fully unrolled instantiations): their launchers live in translation
// units of their own (linear_wide.hip, linear_wide_half.hip) behind these functions, so that a build runs them in parallel.
// dtype: KERNL_F16 / KERNL_BF16; cols: 256 or 192 output columns per tile.
struct LinearArgs;
struct HalfSplitPlan;
void run_wide(const LinearArgs &a, int dtype, int cols);             // 256-row tiles; the gated epilogue when a.act says so
void run_wide_w8(const LinearArgs &a);                               // fp8 e5m2 weights, fp16 activations
void run_wide_half(const LinearArgs &a, int dtype, int cols);        // 128-row tiles
void run_wide_half_w8(const LinearArgs &a);
void run_half_split(const LinearArgs &a, const HalfSplitPlan &p, float *part, int dtype);
void run_small(const LinearArgs &a, int dtype, int rows, int cols);  // 32 x 64, 64 x 64 or 64 x 128 tiles over the whole K (linear_small.hip)
void run_small_dealt(const LinearArgs &a, int dtype, int rows);      // 16-, 32- or 64-row, 32-column tiles, k-tiles dealt to the waves


// ----------------------------------------------------------------------------------------------------
// Epilogue shared by the MFMA kernels: lane (lr, lh) holds, for 32x32 block (i, j) of its wave's tile, output row
// m_wave + 32 i + lr and the 16 consecutive columns starting at n_wave + 32 j + 16 lh.  Bias add, optional store of
// the pre-activation, activation, one rounding to the output dtype, 16-byte stores where the layout allows.
//
// Gated form (ACT has kGluBit set): the weight rows alternate in blocks of 32 between the gate and the value
// projection, so blocks (i, 2p) and (i, 2p + 1) of a lane hold the gate and the value of the SAME 16 output elements;
// out[m, n] = act(gate + bias_gate) * (value + bias_value) with N counting the interleaved rows (twice the output
// width).  The same product as the reference's fused feed-forward kernel forms from two accumulators
// (experimental/llama-v2/kernel/fused_kernel_ff.py:36-75).
// ----------------------------------------------------------------------------------------------------
static constexpr int kGluBit = 8;

// Bias of a wave's TN column blocks as packed 16-bit values: raw[j] holds the 16 consecutive entries starting at
// n_wave + 32 j + 16 lh.  Fetched ONCE per tile and ahead of time: with one or two waves per SIMD a load issued where
// its value is needed stalls the whole epilogue for a memory round trip.
template <typename T, int TN>
__device__ __forceinline__ void bias_fetch(const T *__restrict__ bias, int n_wave, int lh, int N, int bias_vec_ok,
                                           u32x4 (&raw)[TN][2]) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int n = n_wave + j * 32 + lh * 16;
        if (bias == nullptr) {
            raw[j][0] = u32x4{0, 0, 0, 0};
            raw[j][1] = u32x4{0, 0, 0, 0};
        } else if (bias_vec_ok && n + 16 <= N) {
            raw[j][0] = *reinterpret_cast<const u32x4 *>(bias + n);
            raw[j][1] = *reinterpret_cast<const u32x4 *>(bias + n + 8);
        } else {
#pragma unroll
            for (int v = 0; v < 16; v += 2) {
                const uint32_t lo = n + v < N ? (uint32_t)__builtin_bit_cast(uint16_t, bias[n + v]) : 0u;
                const uint32_t hi = n + v + 1 < N ? (uint32_t)__builtin_bit_cast(uint16_t, bias[n + v + 1]) : 0u;
                raw[j][v >> 3][(v & 7) >> 1] = lo | (hi << 16);
            }
        }
    }
}
template <typename T>
__device__ __forceinline__ float bias_elem(const u32x4 (&raw)[2], int v) {
    const uint32_t word = raw[v >> 3][(v & 7) >> 1];
    const uint16_t bits = (uint16_t)((v & 1) ? (word >> 16) : (word & 0xFFFFu));
    return to_float(__builtin_bit_cast(T, bits));
}

// ROW0 / ROWS select the 32-row blocks handled by one call (the wide kernel calls once per block so that each call
// unrolls completely).  Waves whose blocks lie inside the matrix and whose output rows take 16-byte stores run a
// straight-line path; edge tiles, strided outputs and the pre-activation side output run the general one.
template <typename T, int ACT, int TM, int TN, int ROW0 = 0, int ROWS = TM>
__device__ __forceinline__ void linear_epilogue(f32x16 (&acc)[TM][TN], int m_wave, int n_wave, int lr, int lh,
                                                const T *__restrict__ bias, T *__restrict__ out,
                                                T *__restrict__ act_in, int M, int N, int64_t out_rs, int64_t out_cs,
                                                int64_t ai_rs, int64_t ai_cs, int out_vec_ok, int ai_vec_ok,
                                                int bias_vec_ok, const u32x4 (&braw)[TN][2]) {
    auto store16 = [&](T *p, const float (&r)[16]) __attribute__((always_inline)) {
        u32x4 p0, p1;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            p0[v] = pack2<T>(r[2 * v], r[2 * v + 1]);
            p1[v] = pack2<T>(r[8 + 2 * v], r[8 + 2 * v + 1]);
        }
        *reinterpret_cast<u32x4 *>(p) = p0;
        *reinterpret_cast<u32x4 *>(p + 8) = p1;
    };
    const bool rows_inside = m_wave + (ROW0 + ROWS) * 32 <= M;
    if constexpr ((ACT & kGluBit) != 0) {
        static_assert(TN % 2 == 0, "gated epilogue pairs neighbouring 32-column blocks");
        constexpr int BASE = ACT & (kGluBit - 1);
        const int n_total = N >> 1;
        const bool interior = rows_inside && (n_wave >> 1) + TN * 16 <= n_total && out_vec_ok;
        if (__builtin_amdgcn_readfirstlane((int)interior)) {
#pragma unroll
            for (int pr = 0; pr < TN / 2; ++pr) {
                T *col = out + (int64_t)(m_wave + lr) * out_rs + (n_wave >> 1) + pr * 32 + lh * 16;
#pragma unroll
                for (int i = ROW0; i < ROW0 + ROWS; ++i) {
                    float r[16];
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        r[v] = apply_act16(acc[i][2 * pr][v] + bias_elem<T>(braw[2 * pr], v), BASE) *
                               (acc[i][2 * pr + 1][v] + bias_elem<T>(braw[2 * pr + 1], v));
                    store16(col + (int64_t)(i * 32) * out_rs, r);
                }
            }
            return;
        }
#pragma unroll
        for (int pr = 0; pr < TN / 2; ++pr) {
            const int n = (n_wave >> 1) + pr * 32 + lh * 16;         // output column
#pragma unroll
            for (int i = ROW0; i < ROW0 + ROWS; ++i) {
                const int m = m_wave + i * 32 + lr;
                if (m >= M || n >= n_total) continue;  // n_total is a multiple of 32: a block is in or out as a whole
                float r[16];
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    r[v] = apply_act16(acc[i][2 * pr][v] + bias_elem<T>(braw[2 * pr], v), BASE) *
                           (acc[i][2 * pr + 1][v] + bias_elem<T>(braw[2 * pr + 1], v));
                if (out_vec_ok) {
                    store16(out + (int64_t)m * out_rs + n, r);
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v) out[(int64_t)m * out_rs + (int64_t)(n + v) * out_cs] = from_float<T>(r[v]);
                }
            }
        }
        return;
    }
    const bool interior = rows_inside && n_wave + TN * 32 <= N && out_vec_ok && act_in == nullptr;
    if (__builtin_amdgcn_readfirstlane((int)interior)) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            T *col = out + (int64_t)(m_wave + lr) * out_rs + n_wave + j * 32 + lh * 16;
#pragma unroll
            for (int i = ROW0; i < ROW0 + ROWS; ++i) {
                float r[16];
#pragma unroll
                for (int v = 0; v < 16; ++v) r[v] = apply_act16(acc[i][j][v] + bias_elem<T>(braw[j], v), ACT);
                store16(col + (int64_t)(i * 32) * out_rs, r);
            }
        }
        return;
    }
    const bool SAVE_ACT_IN = act_in != nullptr;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int n = n_wave + j * 32 + lh * 16;
#pragma unroll
        for (int i = ROW0; i < ROW0 + ROWS; ++i) {
            const int m = m_wave + i * 32 + lr;
            if (m >= M || n >= N) continue;
            float r[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) r[v] = acc[i][j][v] + bias_elem<T>(braw[j], v);  // zeros without a bias
            if (SAVE_ACT_IN) {
                if (ai_vec_ok && n + 16 <= N) {
                    store16(act_in + (int64_t)m * ai_rs + n, r);
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        if (n + v < N) act_in[(int64_t)m * ai_rs + (int64_t)(n + v) * ai_cs] = from_float<T>(r[v]);
                }
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) r[v] = apply_act16(r[v], ACT);
            if (out_vec_ok && n + 16 <= N) {
                store16(out + (int64_t)m * out_rs + n, r);
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    if (n + v < N) out[(int64_t)m * out_rs + (int64_t)(n + v) * out_cs] = from_float<T>(r[v]);
            }
        }
    }
}

// ----------------------------------------------------------------------------------------------------
// MFMA kernel
// ----------------------------------------------------------------------------------------------------
template <int BM_, int BN_, int BK_, int WAVES_M_, int WAVES_N_, int MIN_BLOCKS_>
struct LinearTile {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int MIN_BLOCKS = MIN_BLOCKS_;
    static constexpr int THREADS = 64 * WAVES_M * WAVES_N;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // per-wave output tile
    static constexpr int TM = WM / 32, TN = WN / 32;            // 32x32 MFMA blocks per wave
    static constexpr int ROW_BYTES = BK * 2;
    static constexpr int CPR = BK / 8;  // 16-byte chunks per tile row
    static constexpr int X_BYTES = BM * ROW_BYTES, W_BYTES = BN * ROW_BYTES;
    static constexpr int STAGE_BYTES = X_BYTES + W_BYTES;
    static constexpr int LDS_BYTES = 2 * STAGE_BYTES;
    static constexpr int XI = BM * CPR / THREADS, WI = BN * CPR / THREADS;  // chunks per thread per stage
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be made of 32x32 blocks");
    static_assert(BM * CPR % THREADS == 0 && BN * CPR % THREADS == 0, "tile rows must split over threads");
    static constexpr int GROUP_M = 4;  // m-tiles walked together so one XCD's L2 sees a compact block
};

// W8: the weight is stored as one byte per element (fp8 e5m2, the upper byte of the fp16 encoding); a thread fetches
// 8 bytes where it would fetch a 16-byte chunk and widens them on the way into LDS, so everything after the LDS
// store is the 16-bit kernel.
template <typename T, typename Cfg, int ACT, bool W8 = false>
__global__ void __launch_bounds__(Cfg::THREADS, Cfg::MIN_BLOCKS)
linear_mfma_kernel(const T *__restrict__ X, const T *__restrict__ W, const T *__restrict__ bias,
                   T *__restrict__ out, T *__restrict__ act_in, int M, int N, int K, int64_t ldx,
                   int64_t out_rs, int64_t out_cs, int64_t ai_rs, int64_t ai_cs, int tiles_m, int tiles_n,
                   int out_vec_ok, int ai_vec_ok, int bias_vec_ok) {
    typedef typename Vec8<T>::type vec8;
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
    constexpr int TM = Cfg::TM, TN = Cfg::TN, CPR = Cfg::CPR, RB = Cfg::ROW_BYTES;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    // ---- tile assignment: workgroup ids are dealt round-robin to the 8 XCDs, so give each XCD a
    // contiguous run of the (grouped) tile order; its private L2 then sees neighbouring tiles.
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) >> 3;
    const int t = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per_xcd || t >= total) return;
    const int group_span = Cfg::GROUP_M * tiles_n;
    const int group = t / group_span;
    const int first_m = group * Cfg::GROUP_M;
    const int gsize = min(tiles_m - first_m, Cfg::GROUP_M);
    const int in_group = t - group * group_span;
    const int tile_m = first_m + in_group % gsize;
    const int tile_n = in_group / gsize;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave % Cfg::WAVES_M, wave_n = wave / Cfg::WAVES_M;
    const int lr = lane & 31, lh = lane >> 5;

    // ---- global -> register staging: thread owns chunks q = tid + THREADS*i, row q / CPR, chunk q % CPR.
    // Loads are buffer loads: a wave-uniform resource (tile origin, extent up to the end of the last valid row),
    // a loop-invariant per-thread 32-bit byte offset and the k position in a scalar register.  Anything past the
    // extent — rows beyond M or N, k-tiles beyond K — reads as zero without touching memory, so the loop needs
    // neither clamps nor branches; only a chunk that starts beyond K INSIDE a valid row is redirected by hand.
    constexpr uint32_t kOutOfRange = 0x80000000u;
    const int rows_x = min(BM, M - m0), rows_w = min(BN, N - n0);
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<T *>(X + (int64_t)m0 * ldx), 0, (int)((((int64_t)rows_x - 1) * ldx + K) * 2), 0x00020000);
    constexpr int WB = W8 ? 1 : 2;  // bytes per weight element in memory
    const __amdgpu_buffer_rsrc_t wrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char *>(reinterpret_cast<const char *>(W) + (int64_t)n0 * K * WB), 0, (int)((int64_t)rows_w * K * WB),
        0x00020000);
    uint32_t xg[Cfg::XI], wg[Cfg::WI];  // byte offsets from the tile origins
    int xl[Cfg::XI], wl[Cfg::WI];       // LDS byte offsets inside a stage
#pragma unroll
    for (int i = 0; i < Cfg::XI; ++i) {
        const int q = tid + Cfg::THREADS * i;
        const int row = q / CPR, c = q % CPR;
        xg[i] = row < rows_x ? (uint32_t)(((int64_t)row * ldx + c * 8) * 2) : kOutOfRange;
        xl[i] = swz_offset<RB>(row, c);
    }
#pragma unroll
    for (int i = 0; i < Cfg::WI; ++i) {
        const int q = tid + Cfg::THREADS * i;
        const int row = q / CPR, c = q % CPR;
        // LDS row `row` feeds MFMA row (row % 32) of its 32-block and carries weight row rowperm16(row % 32).
        const int wrow = (row & ~31) + rowperm16(row & 31);
        wg[i] = wrow < rows_w ? (uint32_t)(((int64_t)wrow * K + c * 8) * WB) : kOutOfRange;
        wl[i] = Cfg::X_BYTES + swz_offset<RB>(row, c);
    }
    const int kchunk = (tid % CPR) * 8;  // same for every i because THREADS % CPR == 0

    // ---- software pipeline over k-tiles of BK:
    //   registers hold tile kt+1 (fetched from HBM/L2 during iteration kt-1), LDS stage kt&1 holds tile kt.
    //   Iteration kt, k-step s:  read the operand fragments of step s+1 from LDS, store a quarter of tile kt+1
    //   from registers into the other LDS stage, run the MFMAs of step s, and re-issue the global loads of the
    //   same quarter for tile kt+2.  Global latency gets a whole iteration to hide, LDS stores ride under the
    //   MFMAs, and there is one barrier per k-tile.  The loop body is branch-free (past the last k-tile the loads
    //   return zeros and the stores fill a stage nobody reads), which keeps the number of loads in flight known
    //   at compile time: the memory counters are waited on by count.
    constexpr int KSTEPS = BK / 16;
    vec8 xs[Cfg::XI], ws[Cfg::WI];
    const int nk = (K + BK - 1) / BK;

    auto gload_part = [&](int k0, int part) {  // chunks i with i % KSTEPS == part
        const bool inside = k0 + kchunk < K;   // K % 8 == 0: a 16-byte chunk is entirely inside or outside
#pragma unroll
        for (int i = 0; i < Cfg::XI; ++i)
            if (i % KSTEPS == part)
                xs[i] = __builtin_bit_cast(
                    vec8, __builtin_amdgcn_raw_buffer_load_b128(xrsrc, inside ? xg[i] : kOutOfRange, k0 * 2, 0));
#pragma unroll
        for (int i = 0; i < Cfg::WI; ++i)
            if (i % KSTEPS == part) {
                if constexpr (W8) {
                    const u32x2 raw = __builtin_amdgcn_raw_buffer_load_b64(wrsrc, inside ? wg[i] : kOutOfRange, k0, 0);
                    const u32x4 wide = {__builtin_amdgcn_perm(0u, raw[0], 0x010c000cu), __builtin_amdgcn_perm(0u, raw[0], 0x030c020cu),
                                        __builtin_amdgcn_perm(0u, raw[1], 0x010c000cu), __builtin_amdgcn_perm(0u, raw[1], 0x030c020cu)};
                    ws[i] = __builtin_bit_cast(vec8, wide);
                } else {
                    ws[i] = __builtin_bit_cast(
                        vec8, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, inside ? wg[i] : kOutOfRange, k0 * 2, 0));
                }
            }
    };
    auto lstore_part = [&](int stage, int part) {
        unsigned char *base = smem + stage * Cfg::STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < Cfg::XI; ++i)
            if (i % KSTEPS == part) *reinterpret_cast<vec8 *>(base + xl[i]) = xs[i];
#pragma unroll
        for (int i = 0; i < Cfg::WI; ++i)
            if (i % KSTEPS == part) *reinterpret_cast<vec8 *>(base + wl[i]) = ws[i];
    };

    f32x16 acc[TM][TN];
    // this wave's bias entries: in flight during the main loop where the tile shape leaves registers for them,
    // fetched in one go after it otherwise
    constexpr bool EARLY_BIAS = BM * BN < 256 * 256;
    u32x4 braw[TN][2];
    if (EARLY_BIAS) bias_fetch<T, TN>(bias, n0 + wave_n * Cfg::WN, lh, N, bias_vec_ok, braw);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // LDS byte offsets of this lane's operand fragments for k-step 0.  Chunk index 2*step + lh and the XOR swizzle
    // only touch bits 4..6 of the offset, so step s is the same offset XOR 32*s.
    static_assert(RB == 128 || RB == 64, "fragment addressing below assumes 64- or 32-element k-tiles");
    int xoff[TM], woff[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) xoff[i] = swz_offset<RB>(wave_m * Cfg::WM + i * 32 + lr, lh);
#pragma unroll
    for (int j = 0; j < TN; ++j) woff[j] = Cfg::X_BYTES + swz_offset<RB>(wave_n * Cfg::WN + j * 32 + lr, lh);

#pragma unroll
    for (int part = 0; part < KSTEPS; ++part) gload_part(0, part);
#pragma unroll
    for (int part = 0; part < KSTEPS; ++part) lstore_part(0, part);
#pragma unroll
    for (int part = 0; part < KSTEPS; ++part) gload_part(BK, part);
    __syncthreads();

    vec8 fa[2][TN], fb[2][TM];
    for (int kt = 0; kt < nk; ++kt) {
        const unsigned char *cur = smem + (kt & 1) * Cfg::STAGE_BYTES;
        const int nxt = (kt + 1) & 1;
#pragma unroll
        for (int j = 0; j < TN; ++j) fa[0][j] = *reinterpret_cast<const vec8 *>(cur + woff[j]);
#pragma unroll
        for (int i = 0; i < TM; ++i) fb[0][i] = *reinterpret_cast<const vec8 *>(cur + xoff[i]);
#pragma unroll
        for (int st = 0; st < KSTEPS; ++st) {
            if (st + 1 < KSTEPS) {
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    fa[(st + 1) & 1][j] = *reinterpret_cast<const vec8 *>(cur + (woff[j] ^ (32 * (st + 1))));
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    fb[(st + 1) & 1][i] = *reinterpret_cast<const vec8 *>(cur + (xoff[i] ^ (32 * (st + 1))));
            }
            lstore_part(nxt, st);
            __builtin_amdgcn_sched_barrier(0);  // keep the order: fragment reads, LDS stores, MFMAs, global loads
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = mfma32(fa[st & 1][j], fb[st & 1][i], acc[i][j]);
            __builtin_amdgcn_sched_barrier(0);
            gload_part((kt + 2) * BK, st);
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
    }

    if (!EARLY_BIAS) bias_fetch<T, TN>(bias, n0 + wave_n * Cfg::WN, lh, N, bias_vec_ok, braw);
    linear_epilogue<T, ACT, TM, TN>(acc, m0 + wave_m * Cfg::WM, n0 + wave_n * Cfg::WN, lr, lh, bias, out, act_in, M, N, out_rs,
                                    out_cs, ai_rs, ai_cs, out_vec_ok, ai_vec_ok, bias_vec_ok, braw);
}

// ----------------------------------------------------------------------------------------------------
// Wide MFMA kernel for K % 8 == 0 (K % 64 == 0 with one-byte weights): 256x256 output tile, 4 waves, ONE wave per SIMD owning a 128x128 sub-tile as
// 8x8 blocks of v_mfma_f32_16x16x32 (256 accumulator registers, kept in the accumulation half of the register file).
// Per 32-wide k-step a wave runs 64 MFMAs on 16 operand fragments — half the LDS traffic per flop of the 8-wave
// kernel above.  Operand tiles go HBM -> LDS directly (buffer loads with the LDS flag), two 64 KB stages.  With a
// single wave per SIMD nothing else can fill a stall, so the instruction stream is laid out by hand: LDS reads and
// tile loads issue in the shadow of the MFMAs (at most one every other MFMA), fragments are read one k-step (64
// MFMAs) ahead, and the one barrier per k-tile sits in front of its second k-step, after which the stage just
// consumed takes the next-but-one k-tile, one load every fourth MFMA.  (A burst of 16 loads followed by a wait for
// all of them stalls a lone wave: 64 KB need >= 1024 cycles to pass the CU's 64 B/clk fill path.)
//
// Weight rows are placed in LDS so that a lane ends up with consecutive output columns of a row (see WideLane below and
// wide_weight_row): stores need no regrouping and 16 adjacent lanes cover a whole row of the wave's sub-tile.
// ----------------------------------------------------------------------------------------------------
// Lane geometry of the wide kernels' results.  The x fragment is the matrix instruction's A operand and the weight
// fragment its B operand: element v of accumulator [i][j] in lane (l16 = lane % 16, g = lane / 16) is output row
// 16 i + 4 g + v of the wave's sub-tile and the output column whose weight row sits in LDS row 16 j + l16 of the wave's
// weight rows.  The placement of weight rows in LDS (wide_weight_row) makes those the lane's CONSECUTIVE columns:
//   plain   LDS row 16 j + r carries weight row NBN r + j: lane l16 holds columns NBN l16 .. NBN l16 + NBN - 1 of each
//           of its four rows — one 16-byte (256-column tiles) or 12-byte (192-column tiles) store per row, and the 16
//           lanes of a group cover the 256 (192) contiguous bytes of the row: a store instruction writes four whole
//           rows of the sub-tile
//   gated   blocks 0 .. 3 carry the gate rows and blocks 4 .. 7 the value rows of output columns 4 l16 .. 4 l16 + 3 (of
//           the wave's 64): one 8-byte store per row
// With the operands the other way round (weights on the A side) adjacent lanes hold different ROWS and every 16-byte
// store reaches memory as 64 separate pieces; regrouping the packed results so that adjacent lanes write contiguous
// bytes (inside quads of lanes with DPP moves, or through LDS) cost 64 vector instructions per 16-row block or the LDS
// bandwidth all four waves want at once.  Here the epilogue of a block is: read, add bias, activate, round, store.
template <bool GATED, int NBN>
struct WideLane {
    static constexpr int NV = GATED ? 4 : NBN;  // output values per lane and row
    // first output column of lane l16 in a wave whose weight rows start at fused row n_wave
    static __device__ __forceinline__ int col(int n_wave, int l16) { return GATED ? (n_wave >> 1) + 4 * l16 : n_wave + NBN * l16; }
};

// The lane's bias entries, fetched as packed 16-bit values (`raw`: entry j of accumulator block j in half j % 2 of dword
// j / 2; zeros without a bias and beyond N) and converted to fp32 once per output tile.  The fetch is issued in front of
// a tile's main loop and the conversion after it, so that no wave waits for a memory round trip between its last
// product and its epilogue.  `N` is the number of weight rows (gated: gate and value rows together; the fused weight
// holds 32 gate rows, then the 32 value rows of the same output columns, and so on).
template <typename T, bool GATED, int NBN>
__device__ __forceinline__ void wide_bias_fetch(const T *__restrict__ bias, int n_wave, int l16, int N, int bias_vec_ok,
                                                uint32_t (&raw)[NBN / 2]) {
#pragma unroll
    for (int e = 0; e < NBN / 2; ++e) raw[e] = 0u;
    if (bias == nullptr) return;
    auto entry = [&](int row) __attribute__((always_inline)) -> uint32_t {
        return row < N ? (uint32_t)__builtin_bit_cast(uint16_t, bias[row]) : 0u;
    };
    if constexpr (GATED) {
        const int c = 4 * l16;                              // first of the lane's 4 output columns inside the wave's 64
        const int row = n_wave + 64 * (c >> 5) + (c & 31);  // its gate row; the value row is 32 further
        if (bias_vec_ok && row + 36 <= N) {
            const u32x2 gt = *reinterpret_cast<const u32x2 *>(bias + row), vl = *reinterpret_cast<const u32x2 *>(bias + row + 32);
            raw[0] = gt[0], raw[1] = gt[1], raw[2] = vl[0], raw[3] = vl[1];
        } else {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                raw[e] = entry(row + 2 * e) | (entry(row + 2 * e + 1) << 16);
                raw[2 + e] = entry(row + 32 + 2 * e) | (entry(row + 33 + 2 * e) << 16);
            }
        }
    } else {
        const int n = n_wave + NBN * l16;
        if (bias_vec_ok && n + NBN <= N) {
            if constexpr (NBN == 8) {
                const u32x4 v = *reinterpret_cast<const u32x4 *>(bias + n);
                raw[0] = v[0], raw[1] = v[1], raw[2] = v[2], raw[3] = v[3];
            } else {
#pragma unroll
                for (int e = 0; e < NBN / 2; ++e) raw[e] = reinterpret_cast<const uint32_t *>(bias + n)[e];
            }
        } else {
#pragma unroll
            for (int e = 0; e < NBN / 2; ++e) raw[e] = entry(n + 2 * e) | (entry(n + 2 * e + 1) << 16);
        }
    }
}
template <typename T, int NBN>
__device__ __forceinline__ void wide_bias_unpack(const uint32_t (&raw)[NBN / 2], float (&bf)[NBN]) {
#pragma unroll
    for (int j = 0; j < NBN; ++j) bf[j] = to_float(__builtin_bit_cast(T, (uint16_t)(raw[j >> 1] >> (16 * (j & 1)))));
}

// Optional per-row factors of the finished sums (fp32, one per row of x: the inverse root mean square when an RMSNorm
// has been folded into the weight): rs[i][v] belongs to row 16 i + 4 g + v of the wave's sub-tile, 1 without factors and
// beyond M.  Fetched in front of a tile's main loop, like the bias.
template <int NBM>
__device__ __forceinline__ void wide_row_scale_fetch(const float *__restrict__ row_scale, int m_lane, int M, float (&rs)[NBM][4]) {
#pragma unroll
    for (int i = 0; i < NBM; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) rs[i][v] = 1.0f;
    if (row_scale == nullptr) return;
#pragma unroll
    for (int i = 0; i < NBM; ++i) {
        const int m = m_lane + 16 * i;  // a multiple of 4: 16-byte aligned in an aligned vector
        if (m + 4 <= M) {
            const float4 v4 = *reinterpret_cast<const float4 *>(row_scale + m);
            rs[i][0] = v4.x, rs[i][1] = v4.y, rs[i][2] = v4.z, rs[i][3] = v4.w;
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (m + v < M) rs[i][v] = row_scale[m + v];
        }
    }
}

// NV rounded values of one row -> one 16-, 12- or 8-byte store
// (RES: `res` holds the packed residual entries of the same elements; they are added to the ROUNDED values and the sum
// is rounded again — what `round(linear) + residual` gives as an addition of two 16-bit tensors)
template <typename T, int NV, bool RES = false, bool PACKED = true>
__device__ __forceinline__ void wide_store_row(T *p, const float (&r)[NV], const uint32_t (&res)[NV / 2]) {
    static_assert(NV == 8 || NV == 6 || NV == 4, "values per lane and row");
    uint32_t w[NV / 2];
#pragma unroll
    for (int e = 0; e < NV / 2; ++e) {
        w[e] = pack2<T>(r[2 * e], r[2 * e + 1]);
        if constexpr (RES) {
            if constexpr (std::is_same<T, f16>::value && PACKED) {
                typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
                w[e] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2_t, w[e]) + __builtin_bit_cast(half2_t, res[e]));
            } else if constexpr (std::is_same<T, f16>::value) {
                typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
                const half2_t a = __builtin_bit_cast(half2_t, w[e]), b = __builtin_bit_cast(half2_t, res[e]);
                w[e] = pack2<T>((float)a[0] + (float)b[0], (float)a[1] + (float)b[1]);
            } else {
                // bf16 -> fp32 is a shift
                const float lo = __builtin_bit_cast(float, w[e] << 16) + __builtin_bit_cast(float, res[e] << 16);
                const float hi = __builtin_bit_cast(float, w[e] & 0xFFFF0000u) + __builtin_bit_cast(float, res[e] & 0xFFFF0000u);
                w[e] = pack2<T>(lo, hi);
            }
        }
    }
    if constexpr (NV == 8) *reinterpret_cast<u32x4 *>(p) = u32x4{w[0], w[1], w[2], w[3]};
    else if constexpr (NV == 6) *reinterpret_cast<u32x3 *>(p) = u32x3{w[0], w[1], w[2]};
    else *reinterpret_cast<u32x2 *>(p) = u32x2{w[0], w[1]};
}

// Optional residual of the plain wide kernels: out = act(...) + residual[m, n], a matrix of the output's shape and dtype
// (the `hidden + projection(...)` of a transformer layer; no counterpart in the reference, whose models add in eager
// PyTorch).  `vec_ok`: unit column stride, rows that keep the lane's 16- or 12-byte pieces aligned.
struct WideResidual {
    const void *ptr = nullptr;
    int64_t rs = 0, cs = 0;
    int vec_ok = 0;
};
// The lane's residual entries of one 16-row block — rows m_first .. m_first + 3, its NBN consecutive columns from n on —
// as packed 16-bit values (zeros outside the matrix).  Issued one block ahead of the epilogue that adds them (block 0:
// in front of the tile's main loop, like the bias), so that no epilogue waits for a memory round trip.
template <typename T, int NBN>
__device__ __forceinline__ void wide_residual_fetch(const WideResidual &res, int m_first, int n, int M, int N,
                                                    uint32_t (&raw)[4][NBN / 2]) {
    const T *base = static_cast<const T *>(res.ptr);
    if (res.vec_ok && m_first + 4 <= M && n + NBN <= N) {
        const T *p = base + (int64_t)m_first * res.rs + n;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            if constexpr (NBN == 8) {
                const u32x4 t = *reinterpret_cast<const u32x4 *>(p + v * res.rs);
                raw[v][0] = t[0], raw[v][1] = t[1], raw[v][2] = t[2], raw[v][3] = t[3];
            } else {
                const u32x3 t = *reinterpret_cast<const u32x3 *>(p + v * res.rs);
                raw[v][0] = t[0], raw[v][1] = t[1], raw[v][2] = t[2];
            }
        }
        return;
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) {
#pragma unroll
        for (int e = 0; e < NBN / 2; ++e) raw[v][e] = 0u;
#pragma unroll
        for (int c = 0; c < NBN; ++c)
            if (m_first + v < M && n + c < N)
                raw[v][c >> 1] |= (uint32_t)__builtin_bit_cast(uint16_t, base[(int64_t)(m_first + v) * res.rs + (int64_t)(n + c) * res.cs]) << (16 * (c & 1));
    }
}

template <typename T, int NV>
__device__ __forceinline__ void wide_store_row(T *p, const float (&r)[NV]) {
    const uint32_t none[NV / 2] = {};
    wide_store_row<T, NV, false>(p, r, none);
}

// Epilogue of m-block IB (16 rows) of a wave of the wide kernels: out = act(sum * row factor + bias) (+ residual, RES:
// added to the ROUNDED value and rounded again, as a separate addition of two 16-bit tensors would).  Blocks that lie
// inside the matrix, with contiguous 16-byte aligned output rows and no pre-activation side output, run a straight-line path.
template <typename T, int ACT, int IB, int NBN, int NBM = 8, bool SCALED = false, bool RES = false>
__device__ __forceinline__ void wide_epilogue(f32x4_acc (&acc)[NBM][NBN], int m_wave, int n_wave, int l16, int g,
                                              T *__restrict__ out, T *__restrict__ act_in, int M, int N,
                                              int64_t out_rs, int64_t out_cs, int64_t ai_rs, int64_t ai_cs,
                                              int out_vec_ok, int ai_vec_ok, const float (&bf)[NBN], const float (&rs)[4],
                                              const uint32_t (&rres)[4][NBN / 2]) {
    constexpr bool GATED = (ACT & kGluBit) != 0;
    static_assert(!GATED || NBN == 8, "gated epilogues: four gate and four value blocks");
    static_assert(!RES || !GATED, "the residual form is for plain epilogues");
    constexpr int BASE = ACT & (kGluBit - 1), NV = WideLane<GATED, NBN>::NV;
    const int n = WideLane<GATED, NBN>::col(n_wave, l16);
    const int n_total = GATED ? N >> 1 : N;  // output columns
    const int m_first = m_wave + 16 * IB + 4 * g;
    // pre-activation values of row 4 g + v (gated: the gate; `value` then holds what it is multiplied with)
    auto sums = [&](int v, float (&r)[NV], float (&value)[NV]) __attribute__((always_inline)) {
#pragma unroll
        for (int c = 0; c < NV; ++c) {
            r[c] = SCALED ? fmaf(acc[IB][c][v], rs[v], bf[c]) : acc[IB][c][v] + bf[c];
            if (GATED) value[c] = SCALED ? fmaf(acc[IB][(4 + c) % NBN][v], rs[v], bf[(4 + c) % NBN]) : acc[IB][(4 + c) % NBN][v] + bf[(4 + c) % NBN];
            else value[c] = 1.0f;
        }
    };
    const bool interior = m_wave + 16 * IB + 16 <= M && (GATED ? (n_wave >> 1) + 64 <= n_total : n_wave + NBN * 16 <= N) &&
                          out_vec_ok && (GATED || act_in == nullptr);
    if (__builtin_amdgcn_readfirstlane((int)interior)) {
        T *p = out + (int64_t)m_first * out_rs + n;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            float r[NV], value[NV];
            sums(v, r, value);
#pragma unroll
            for (int c = 0; c < NV; ++c) r[c] = GATED ? apply_act16(r[c], BASE) * value[c] : apply_act16(r[c], ACT);
            if constexpr (RES) wide_store_row<T, NV, true>(p + v * out_rs, r, rres[v]);
            else wide_store_row<T, NV>(p + v * out_rs, r);
        }
        return;
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int m = m_first + v;
        if (m >= M || n >= n_total) continue;
        float r[NV], value[NV];
        sums(v, r, value);
        if (!GATED && act_in != nullptr) {
            if (ai_vec_ok && n + NV <= n_total) {
                wide_store_row<T, NV>(act_in + (int64_t)m * ai_rs + n, r);
            } else {
#pragma unroll
                for (int c = 0; c < NV; ++c)
                    if (n + c < n_total) act_in[(int64_t)m * ai_rs + (int64_t)(n + c) * ai_cs] = from_float<T>(r[c]);
            }
        }
#pragma unroll
        for (int c = 0; c < NV; ++c) r[c] = GATED ? apply_act16(r[c], BASE) * value[c] : apply_act16(r[c], ACT);
        if (out_vec_ok && n + NV <= n_total) {
            if constexpr (RES) wide_store_row<T, NV, true>(out + (int64_t)m * out_rs + n, r, rres[v]);
            else wide_store_row<T, NV>(out + (int64_t)m * out_rs + n, r);
        } else {
#pragma unroll
            for (int c = 0; c < NV; ++c) {
                if (n + c >= n_total) continue;
                T o = from_float<T>(r[c]);
                if constexpr (RES) o = from_float<T>(to_float(o) + to_float(__builtin_bit_cast(T, (uint16_t)(rres[v][c >> 1] >> (16 * (c & 1))))));
                out[(int64_t)m * out_rs + (int64_t)(n + c) * out_cs] = o;
            }
        }
    }
}

template <typename T, int ACT, int IB, int NBN, int NBM = 8, bool SCALED = false>
__device__ __forceinline__ void wide_epilogue(f32x4_acc (&acc)[NBM][NBN], int m_wave, int n_wave, int l16, int g,
                                              T *__restrict__ out, T *__restrict__ act_in, int M, int N,
                                              int64_t out_rs, int64_t out_cs, int64_t ai_rs, int64_t ai_cs,
                                              int out_vec_ok, int ai_vec_ok, const float (&bf)[NBN], const float (&rs)[4]) {
    const uint32_t none[4][NBN / 2] = {};
    wide_epilogue<T, ACT, IB, NBN, NBM, SCALED, false>(acc, m_wave, n_wave, l16, g, out, act_in, M, N, out_rs, out_cs, ai_rs,
                                                       ai_cs, out_vec_ok, ai_vec_ok, bf, rs, none);
}

// W8: the weight is stored as one byte per element (fp8 e5m2, the upper byte of the fp16 encoding).  Its tile travels
// HBM -> LDS as bytes (half the loads, 64-byte rows, chunks swizzled for 8-byte reads), a fragment is read as 8 bytes
// and widened by four byte-permutes two read slots later, all in the shadow of the MFMAs; everything else is unchanged.
// SCALED: the finished sums are multiplied by a factor per row of x (row_scale, fp32 [M]) before the bias is added.
// RES: a residual matrix is added to the rounded results (plain epilogues only).
template <typename T, int ACT, int NBN, bool W8 = false, bool SCALED = false, bool RES = false>
__global__ void __launch_bounds__(256, 1)
linear_wide_kernel(const T *__restrict__ X, const T *__restrict__ W, const T *__restrict__ bias, T *__restrict__ out,
                   T *__restrict__ act_in, int M, int N, int K, int64_t ldx, int64_t out_rs, int64_t out_cs,
                   int64_t ai_rs, int64_t ai_cs, int tiles_m, int tiles_n, int out_vec_ok, int ai_vec_ok,
                   int bias_vec_ok, const float *__restrict__ row_scale, const WideResidual residual) {
    typedef typename Vec8<T>::type vec8;
    constexpr bool GATED = (ACT & kGluBit) != 0;
    static_assert(NBN == 8 || (NBN == 6 && !GATED), "256 or 192 columns per tile; gated epilogues need 256");
    constexpr int BM = 256, BN = 32 * NBN, BK = 64, RB = BK * 2, CPR = BK / 8, NB = 8, KSTEPS = BK / 32;
    // LDS: [x stage 0 | x stage 1 | w stage 0 | w stage 1], 32 KB each: every fragment address is one per-lane register
    // plus an immediate of 0 or 32 KB for the stage (the immediate field of an LDS read ends at 64 KB - 1).
    constexpr int X_BYTES = BM * RB, W_BYTES = 32768, W_BASE = 2 * X_BYTES;
    static_assert(X_BYTES == 32768 && BN * RB <= W_BYTES, "stage immediates");
    static_assert(!W8 || (std::is_same<T, f16>::value && NBN == 8 && !GATED), "one-byte weights: fp16, 256 columns, plain");
    constexpr int WB = W8 ? 1 : 2;                                   // bytes per weight element in memory and in LDS
    constexpr int RBW = BK * WB, CPRW = RBW / 16;                    // weight tile: row bytes, 16-byte chunks per row
    constexpr int LOADS = BM * CPR / 256, LOADS_W = BN * CPRW / 256;  // 1 KB loads per wave for the x and the w tile
    constexpr int NL = LOADS + LOADS_W;                             // tile loads per wave and k-tile
    constexpr int GROUP_M = 4;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    // Persistent workgroups: one per CU (at most), each walking the output tiles  slot, slot + slots, ...  of its
    // XCD's contiguous run of the grouped tile order.  The k-tile stream runs THROUGH tile boundaries: while the last
    // k-tiles of one output tile are multiplied, the first two k-tiles of the next are already on their way into LDS,
    // and the epilogue's stores drain under the next tile's main loop.
    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) >> 3;
    const int xcd = (int)(blockIdx.x & 7), slots = (int)(gridDim.x >> 3);
    auto tile_origin = [&](int idx, int &m0, int &n0) __attribute__((always_inline)) -> bool {
        const int t = xcd * per_xcd + idx;
        if (idx >= per_xcd || t >= total) return false;
        const int group_span = GROUP_M * tiles_n;
        const int group = t / group_span;
        const int first_m = group * GROUP_M;
        const int gsize = min(tiles_m - first_m, GROUP_M);
        const int in_group = t - group * group_span;
        m0 = (first_m + in_group % gsize) * BM;
        n0 = (in_group / gsize) * BN;
        return true;
    };

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave & 1, wave_n = wave >> 1;
    const int l16 = lane & 15, g = lane >> 4;

    // ---- tile loads: load i of a wave fills the 1 KB of 16-byte chunks [256 i + 64 wave, +64) of an operand tile;
    // every lane fetches the chunk that belongs at its LDS position under the swizzle.  Rows beyond M / N lie outside
    // the buffer resource and arrive as zeros.  A wave's loads of one operand tile land in one contiguous 8 KB block
    // (load i at +1 KB i), so that groups of 4 loads share one write of the LDS base register and differ only in the
    // instruction's immediate offset.  That immediate is added to the memory address too, hence it is subtracted from
    // the per-lane offsets here.
    constexpr uint32_t kOutOfRange = 0x80000000u;
    u32x4 xrsrc = {0, 0, 0, 0x00020000u}, wrsrc = {0, 0, 0, 0x00020000u};
    uint32_t xd[LOADS], wd[LOADS_W];
    // points the tile loads at the output tile with origin (m0, n0); `valid` false switches them off
    auto set_load_tile = [&](bool valid, int m0, int n0) __attribute__((always_inline)) {
        const int rows_x = valid ? min(BM, M - m0) : 0, rows_w = valid ? min(BN, N - n0) : 0;
        if (valid) {
            const uint64_t xaddr = (uint64_t)(uintptr_t)(X + (int64_t)m0 * ldx);
            const uint64_t waddr = (uint64_t)(uintptr_t)(reinterpret_cast<const char *>(W) + (int64_t)n0 * K * WB);
            xrsrc[0] = (uint32_t)xaddr;
            xrsrc[1] = (uint32_t)(xaddr >> 32) & 0xFFFFu;
            xrsrc[2] = (uint32_t)((((int64_t)rows_x - 1) * ldx + K) * 2);
            wrsrc[0] = (uint32_t)waddr;
            wrsrc[1] = (uint32_t)(waddr >> 32) & 0xFFFFu;
            wrsrc[2] = (uint32_t)((int64_t)rows_w * K * WB);
        }
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int q = (wave * LOADS + i) * 64 + lane;  // 16-byte chunk index inside the tile
            const int row = q / CPR, c = swz_chunk<RB>(row, q % CPR);
            xd[i] = row < rows_x ? (uint32_t)(((int64_t)row * ldx + c * 8) * 2) - (uint32_t)(i & 3) * 1024u : kOutOfRange;
        }
#pragma unroll
        for (int i = 0; i < LOADS_W; ++i) {
            const int q = (wave * LOADS_W + i) * 64 + lane;
            const int row = q / CPRW, c = swz_chunk<RBW>(row, q % CPRW);
            // LDS row `row` is MFMA row r = row % 16 of n-block row / 16; see the placement rule above the kernel
            const int wrow = wide_weight_row<GATED, NBN>(row);
            wd[i] = wrow < rows_w ? (uint32_t)((int64_t)wrow * K * WB + c * 16) - (uint32_t)(i & 3) * 1024u : kOutOfRange;
        }
    };
    typedef __attribute__((address_space(3))) void lds_void;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void *)smem;
    // inline assembly on purpose: the compiler would make every later LDS read wait for loads it sees writing LDS.
    // `group` (0 or 1) selects loads 4 group .. 4 group + 3; its first load writes the LDS base register.
    auto load4 = [&](const u32x4 &rsrc, uint32_t off, uint32_t lds, int group, int part, int kbytes) __attribute__((always_inline)) {
        if (part == 0)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :: "s"(lds + group * 4096), "v"(off), "s"(rsrc), "s"(kbytes) : "memory", "m0");
        else if (part == 1)
            asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:1024 lds" :: "v"(off), "s"(rsrc), "s"(kbytes) : "memory");
        else if (part == 2)
            asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:2048 lds" :: "v"(off), "s"(rsrc), "s"(kbytes) : "memory");
        else
            asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:3072 lds" :: "v"(off), "s"(rsrc), "s"(kbytes) : "memory");
    };
    // K % 64 != 0: the last k-tile of every output tile is ragged.  Bit l of `tail_bits` says whether the chunk that
    // load l of this lane fetches starts below K in that k-tile; the others are pointed out of range and arrive as
    // zeros, in BOTH operands (a zero weight against whatever follows a row of x would still turn an infinity there
    // into a NaN here).  The chunk a (lane, load) pair fetches is the same for every tile.
    const int nk = (K + BK - 1) / BK;
    const int k_last = K - (nk - 1) * BK;  // 8 .. 64 valid k in the last k-tile
    uint32_t tail_bits = 0;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int q = (wave * LOADS + i) * 64 + lane;
        if (swz_chunk<RB>(q / CPR, q % CPR) * 8 < k_last) tail_bits |= 1u << i;
    }
#pragma unroll
    for (int i = 0; i < LOADS_W; ++i) {
        const int q = (wave * LOADS_W + i) * 64 + lane;
        if (swz_chunk<RBW>(q / CPRW, q % CPRW) * (16 / WB) < k_last) tail_bits |= 1u << (LOADS + i);
    }
    // The offsets are clipped IN PLACE when the ragged k-tile is the next one to request (it is the last k-tile of its
    // output tile: the next tile's offsets are computed afresh) — a branch taken once per output tile, and never when
    // K % 64 == 0; a select per load would put three VALU instructions per load into every k-tile of every shape.
    const int tail_kt = (K % BK) != 0 ? nk - 1 : -1;
    auto clip_tail = [&]() __attribute__((always_inline)) {
        asm volatile("" ::: "memory");  // keeps this a branch: without it the compiler turns the block into selects
#pragma unroll
        for (int i = 0; i < LOADS; ++i) xd[i] = ((tail_bits >> i) & 1u) != 0 ? xd[i] : kOutOfRange;
#pragma unroll
        for (int i = 0; i < LOADS_W; ++i) wd[i] = ((tail_bits >> (LOADS + i)) & 1u) != 0 ? wd[i] : kOutOfRange;
    };
    // load l (0 .. NL-1) of a k-tile: the x loads, then the w loads
    auto tile_load = [&](int l, int stage, int k0) __attribute__((always_inline)) {
        const uint32_t off = l < LOADS ? xd[l] : wd[l - LOADS];
        if (l < LOADS) load4(xrsrc, off, lds_base + stage * X_BYTES + wave * (LOADS * 1024), l >> 2, l & 3, k0 * 2);
        else load4(wrsrc, off, lds_base + W_BASE + stage * W_BYTES + wave * (LOADS_W * 1024), (l - LOADS) >> 2, (l - LOADS) & 3, k0 * WB);
    };

    // LDS addresses of this lane's operand fragments in stage 0, one register per (k-step, block): with a whole
    // register file per wave there is room to keep them all, and no address arithmetic is left in the loop
    typedef __attribute__((address_space(3))) const unsigned char *lds_bytes;
    typedef __attribute__((address_space(3))) const vec8 *lds_frag;
    const lds_bytes lds0 = (lds_bytes)smem;
    lds_frag xfrag[KSTEPS][NB], wfrag[KSTEPS][NBN];
#pragma unroll
    for (int st = 0; st < KSTEPS; ++st) {
#pragma unroll
        for (int i = 0; i < NB; ++i) xfrag[st][i] = (lds_frag)(lds0 + swz_offset<RB>(wave_m * 128 + i * 16 + l16, 4 * st + g));
#pragma unroll
        for (int j = 0; j < NBN; ++j) {
            const int row = wave_n * (NBN * 16) + j * 16 + l16, unit = 4 * st + g;   // 8 k-values per unit
            wfrag[st][j] = W8 ? (lds_frag)(lds0 + W_BASE + swz_offset<RBW>(row, unit >> 1) + (unit & 1) * 8)
                              : (lds_frag)(lds0 + W_BASE + swz_offset<RBW>(row, unit));
        }
    }
    constexpr int STAGE_FRAGS = X_BYTES / 16;  // pointer increment that selects stage 1
    // one-byte weights: 8 bytes per fragment, widened (byte b of a dword becomes the 16-bit value b << 8)
    typedef __attribute__((address_space(3))) const u32x2 *lds_frag8;
    auto read8 = [&](lds_frag ptr) __attribute__((always_inline)) -> u32x2 { return *(lds_frag8)ptr; };
    auto widen8 = [&](u32x2 raw) __attribute__((always_inline)) -> vec8 {
        const u32x4 wide = {__builtin_amdgcn_perm(0u, raw[0], 0x010c000cu), __builtin_amdgcn_perm(0u, raw[0], 0x030c020cu),
                            __builtin_amdgcn_perm(0u, raw[1], 0x010c000cu), __builtin_amdgcn_perm(0u, raw[1], 0x030c020cu)};
        return __builtin_bit_cast(vec8, wide);
    };
    u32x2 wraw[W8 ? NBN : 1];

    int idx = (int)(blockIdx.x >> 3);  // position of the tile being multiplied in this XCD's run
    int m0 = 0, n0 = 0;
    if (!tile_origin(idx, m0, n0)) return;

    // the load side runs ahead of the multiply side: (load_idx, load_kt) is the next k-tile to request
    int load_idx = idx, load_kt = 0;
    set_load_tile(true, m0, n0);
    if (tail_kt == 0) clip_tail();
    auto advance_load = [&]() __attribute__((always_inline)) {
        if (++load_kt == nk) {
            load_kt = 0;
            load_idx += slots;
            int lm0 = 0, ln0 = 0;
            const bool more = tile_origin(load_idx, lm0, ln0);
            set_load_tile(more, lm0, ln0);
        }
        if (load_kt == tail_kt) clip_tail();
    };
#pragma unroll
    for (int l = 0; l < NL; ++l) tile_load(l, 0, load_kt * BK);
    advance_load();
#pragma unroll
    for (int l = 0; l < NL; ++l) tile_load(l, 1, load_kt * BK);
    advance_load();
    // vmcnt(NL): the first k-tile has landed, the second may still be in flight
    __builtin_amdgcn_s_waitcnt(0x0F70 | (NL & 15) | ((NL >> 4) << 14));
    __syncthreads();

    vec8 fa[KSTEPS][NBN], fb[KSTEPS][NB];  // weight and activation fragments, one register set per k-step
#pragma unroll
    for (int j = 0; j < NBN; ++j) {
        if constexpr (W8) fa[0][j] = widen8(read8(wfrag[0][j]));
        else fa[0][j] = *wfrag[0][j];
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) fb[0][i] = *xfrag[0][i];

    f32x4_acc acc[NB][NBN];  // [m-block][n-block]

    // One k-tile held in stage CUR (a compile-time constant, so that stage offsets fold into instruction offsets).
    // `landed`: the loads of the next k-tile are known to have arrived (a wait for later loads has been passed), and
    // waiting for "everything outstanding" would only wait for the previous tile's output stores.
    auto k_tile = [&](auto cur_c, bool landed, auto first_c) __attribute__((always_inline)) {
        constexpr int CUR = decltype(cur_c)::value;
        constexpr bool FIRST = decltype(first_c)::value;  // the first k-tile of an output tile: its first k-step starts the sums
        const int k0 = load_kt * BK;
#pragma unroll
        for (int st = 0; st < KSTEPS; ++st) {
            const int sn = st ^ 1;                               // k-step whose fragments are fetched now
            const int src = (st == 0 ? CUR : CUR ^ 1) * STAGE_FRAGS;  // stage holding those fragments
            if (st == 1) {
                if (!landed) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's loads of the next k-tile are in
                __syncthreads();                                  // ... everyone's are, and nobody reads stage CUR any more
            }
            constexpr int PERIOD = NBN == 8 ? 4 : 3;  // MFMAs per LDS read / tile load: 64 / 4 = 48 / 3 = 16 issue slots
#pragma unroll
            for (int m = 0; m < NB * NBN; ++m) {
                const int i = m / NBN, j = m % NBN;
                // x on the A side: rows of the result are rows of x
                if (FIRST && st == 0) mfma16_start(fb[st][i], fa[st][j], acc[i][j]);
                else mfma16_inplace(fb[st][i], fa[st][j], acc[i][j]);
                const int slot = m / PERIOD;
                if (m % PERIOD == 0 && slot < NBN + NB) {
                    // the weight fragments first: the first MFMAs of the next k-step need all of them
                    if (slot < NBN) {
                        // (stage offsets are in 16-byte units of the 16-bit layout: a byte-weight stage is W_BYTES further all the same)
                        if constexpr (W8) wraw[slot] = read8(wfrag[sn][slot] + src);
                        else fa[sn][slot] = *(wfrag[sn][slot] + src);
                    } else {
                        fb[sn][slot - NBN] = *(xfrag[sn][slot - NBN] + src);
                    }
                } else if (W8 && m % PERIOD == 1 && slot >= 2 && slot - 2 < NBN) {
                    fa[sn][slot - 2] = widen8(wraw[slot - 2]);  // two read slots later: the bytes have arrived
                } else if (m % PERIOD == PERIOD - 2 && st == 1 && slot < NL) {
                    tile_load(slot, CUR, k0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    // Every output tile starts in stage 0: the host launches one workgroup per tile when the number of k-tiles is odd.
    bool landed = false;
    while (true) {
        // the tile's bias entries travel under its main loop
        const int n_wave = n0 + wave_n * (NBN * 16);
        uint32_t braw[NBN / 2];
        wide_bias_fetch<T, GATED, NBN>(bias, n_wave, l16, N, bias_vec_ok, braw);
        float rsc[SCALED ? NB : 1][4];
        if constexpr (SCALED) wide_row_scale_fetch<NB>(row_scale, m0 + wave_m * 128 + 4 * g, M, rsc);
        // the residual entries of the first 16-row blocks too; those of block I + RD - 1 are requested in front of block
        // I's epilogue (a ring of RD blocks: inside a model the residual was written several hundred MB of traffic ago
        // and comes from HBM, two or three block epilogues away)
        constexpr int RD = RES ? (NBN == 6 ? 4 : 3) : 1;
        uint32_t rres[RD][4][NBN / 2];
        const int n_lane = WideLane<GATED, NBN>::col(n_wave, l16);
        if constexpr (RES) {
#pragma unroll
            for (int i = 0; i < RD - 1; ++i)
                wide_residual_fetch<T, NBN>(residual, m0 + wave_m * 128 + 16 * i + 4 * g, n_lane, M, N, rres[i]);
        }
        // (no zeroing of the accumulators: the first k-step of the tile writes them)
        k_tile(IntC<0>(), landed, BoolC<true>());
        advance_load();
        landed = false;
        int kt = 1;
        for (; kt + 1 < nk; kt += 2) {
            k_tile(IntC<1>(), false, BoolC<false>());
            advance_load();
            k_tile(IntC<0>(), false, BoolC<false>());
            advance_load();
        }
        if (kt < nk) {
            k_tile(IntC<1>(), false, BoolC<false>());
            advance_load();
        }
        mfma16_inplace_results_landed(acc);

        // the loads of the next k-tile were issued earlier: after this wait they are known to have landed
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        landed = true;
        float bf[NBN];
        wide_bias_unpack<T, NBN>(braw, bf);
        // one call per 16-row block: each stays small enough for the compiler to unroll completely, so the
        // accumulators are only ever indexed by constants and never leave the register file
#define KERNL_WIDE_EPILOGUE(I)                                                                                         \
    if constexpr (RES && I + RD - 1 < 8)                                                                               \
        wide_residual_fetch<T, NBN>(residual, m0 + wave_m * 128 + 16 * (I + RD - 1) + 4 * g, n_lane, M, N, rres[(I + RD - 1) % RD]); \
    wide_epilogue<T, ACT, I, NBN, 8, SCALED, RES>(acc, m0 + wave_m * 128, n_wave, l16, g, out, act_in, M, N, out_rs, out_cs,   \
                                                  ai_rs, ai_cs, out_vec_ok, ai_vec_ok, bf, rsc[SCALED ? I : 0], rres[I % RD])
        KERNL_WIDE_EPILOGUE(0);
        KERNL_WIDE_EPILOGUE(1);
        KERNL_WIDE_EPILOGUE(2);
        KERNL_WIDE_EPILOGUE(3);
        KERNL_WIDE_EPILOGUE(4);
        KERNL_WIDE_EPILOGUE(5);
        KERNL_WIDE_EPILOGUE(6);
        KERNL_WIDE_EPILOGUE(7);
#undef KERNL_WIDE_EPILOGUE
        idx += slots;
        if (!tile_origin(idx, m0, n0)) break;
    }
}

// ----------------------------------------------------------------------------------------------------
// Half-height variant of the wide kernel for outputs that leave CUs idle with 256-row tiles (M = 2048 against
// N = 4096 gives 128 tiles of 256x256 but 256 of 128x256): 128 x (256 | 192) tile, 4 waves as 2 x 2, a 64-row
// sub-tile per wave (4 x NBN blocks of v_mfma_f32_16x16x32).  A k-tile is only 2 x 32 (24) MFMAs long here, too short
// to cover the load latency with two stages, and the smaller x tile leaves room for a third: THREE stages of
// 16 KB (x) + 32 KB (w), k-tile T + 3 requested while k-tile T is multiplied, the wait in front of the second k-step
// only for k-tile T + 1 (vmcnt(NL): the loads of T + 2 may still be in flight).  One workgroup per output tile.
// ----------------------------------------------------------------------------------------------------
// Tile t of the half-height kernels' grouped order (GROUP_M row tiles side by side) -> origin of the tile.
__device__ __forceinline__ void half_tile_origin(int t, int tiles_m, int tiles_n, int BM, int BN, int &m0, int &n0) {
    constexpr int GROUP_M = 8;
    const int group_span = GROUP_M * tiles_n;
    const int group = t / group_span;
    const int first_m = group * GROUP_M;
    const int gsize = min(tiles_m - first_m, GROUP_M);
    const int in_group = t - group * group_span;
    m0 = (first_m + in_group % gsize) * BM;
    n0 = (in_group / gsize) * BN;
}

// SPLIT: blockIdx.y selects one of `splits` ranges of k-tiles; the workgroup leaves its fp32 partial tile in `part`
// (slot blockIdx.y * tiles + t; per wave and 16 x 16 block 64 lanes x 16 bytes: coalesced, and the same lane reads it
// back in linear_wide_half_reduce_kernel, which adds the ranges in order and runs the epilogue).
template <typename T, int ACT, int NBN, bool W8 = false, bool SPLIT = false, bool SCALED = false, bool RES = false>
__global__ void __launch_bounds__(256, 1)
linear_wide_half_kernel(const T *__restrict__ X, const T *__restrict__ W, const T *__restrict__ bias,
                        T *__restrict__ out, T *__restrict__ act_in, int M, int N, int K, int64_t ldx, int64_t out_rs,
                        int64_t out_cs, int64_t ai_rs, int64_t ai_cs, int tiles_m, int tiles_n, int out_vec_ok,
                        int ai_vec_ok, int bias_vec_ok, float *__restrict__ part, int splits,
                        const float *__restrict__ row_scale, const WideResidual residual) {
    static_assert(!RES || !SPLIT, "the split form leaves its epilogue to the reduction launch");
    typedef typename Vec8<T>::type vec8;
    static_assert((ACT & kGluBit) == 0 && (NBN == 8 || NBN == 6), "plain epilogues, 256 or 192 columns");
    constexpr int NBM = 4, BM = 32 * NBM, BN = 32 * NBN, BK = 64, RB = BK * 2, CPR = BK / 8, KSTEPS = BK / 32;
    constexpr int X_STAGE = BM * RB, W_STAGE = 32768, W_BASE = 3 * X_STAGE;  // [x0|x1|x2|w0|w1|w2]
    static_assert(X_STAGE == 16384 && BN * RB <= W_STAGE, "stage immediates");
    static_assert(!W8 || (std::is_same<T, f16>::value && NBN == 8), "one-byte weights: fp16, 256 columns");
    constexpr int WB = W8 ? 1 : 2, RBW = BK * WB, CPRW = RBW / 16;  // weight tile: bytes per element, row bytes, chunks per row
    constexpr int LOADS_X = BM * CPR / 256, LOADS_W = BN * CPRW / 256, NL = LOADS_X + LOADS_W;
    static_assert(LOADS_X == 4, "one group of four loads for the x tile");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int total = tiles_m * tiles_n;
    const int per_xcd = (total + 7) >> 3;
    const int t = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= per_xcd || t >= total) return;
    int m0, n0;
    half_tile_origin(t, tiles_m, tiles_n, BM, BN, m0, n0);

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave & 1, wave_n = wave >> 1;
    const int l16 = lane & 15, g = lane >> 4;
    // per-row factors of the finished sums, if any: they travel under the main loop
    float rsc[SCALED ? NBM : 1][4];
    if constexpr (SCALED) wide_row_scale_fetch<NBM>(row_scale, m0 + wave_m * (NBM * 16) + 4 * g, M, rsc);

    // tile loads, as in the wide kernel: every lane fetches the chunk that belongs at its LDS position
    constexpr uint32_t kOutOfRange = 0x80000000u;
    const int rows_x = min(BM, M - m0), rows_w = min(BN, N - n0);
    const uint64_t xaddr = (uint64_t)(uintptr_t)(X + (int64_t)m0 * ldx);
    const uint64_t waddr = (uint64_t)(uintptr_t)(reinterpret_cast<const char *>(W) + (int64_t)n0 * K * WB);
    const u32x4 xrsrc = {(uint32_t)xaddr, (uint32_t)(xaddr >> 32) & 0xFFFFu,
                         (uint32_t)((((int64_t)rows_x - 1) * ldx + K) * 2), 0x00020000u};
    const u32x4 wrsrc = {(uint32_t)waddr, (uint32_t)(waddr >> 32) & 0xFFFFu, (uint32_t)((int64_t)rows_w * K * WB),
                         0x00020000u};
    uint32_t xd[LOADS_X], wd[LOADS_W];
#pragma unroll
    for (int i = 0; i < LOADS_X; ++i) {
        const int q = (wave * LOADS_X + i) * 64 + lane;
        const int row = q / CPR, c = swz_chunk<RB>(row, q % CPR);
        xd[i] = row < rows_x ? (uint32_t)(((int64_t)row * ldx + c * 8) * 2) - (uint32_t)(i & 3) * 1024u : kOutOfRange;
    }
#pragma unroll
    for (int i = 0; i < LOADS_W; ++i) {
        const int q = (wave * LOADS_W + i) * 64 + lane;
        const int row = q / CPRW, c = swz_chunk<RBW>(row, q % CPRW);
        const int wrow = wide_weight_row<false, NBN>(row);
        wd[i] = wrow < rows_w ? (uint32_t)((int64_t)wrow * K * WB + c * 16) - (uint32_t)(i & 3) * 1024u : kOutOfRange;
    }
    typedef __attribute__((address_space(3))) void lds_void;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void *)smem;
    auto load4 = [&](const u32x4 &rsrc, uint32_t off, uint32_t lds, int group4, int part, int kbytes) __attribute__((always_inline)) {
        if (part == 0)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :: "s"(lds + group4 * 4096), "v"(off), "s"(rsrc), "s"(kbytes) : "memory", "m0");
        else if (part == 1)
            asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:1024 lds" :: "v"(off), "s"(rsrc), "s"(kbytes) : "memory");
        else if (part == 2)
            asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:2048 lds" :: "v"(off), "s"(rsrc), "s"(kbytes) : "memory");
        else
            asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:3072 lds" :: "v"(off), "s"(rsrc), "s"(kbytes) : "memory");
    };
    // K % 64 != 0: chunks of the last k-tile that start at or beyond K are pointed out of range and arrive as zeros,
    // in both operands (as in the wide kernel); bit l of `tail_bits`: load l of this lane stays inside
    const int nk_all = (K + BK - 1) / BK;
    const int k_last = K - (nk_all - 1) * BK;
    uint32_t tail_bits = 0;
#pragma unroll
    for (int i = 0; i < LOADS_X; ++i) {
        const int q = (wave * LOADS_X + i) * 64 + lane;
        if (swz_chunk<RB>(q / CPR, q % CPR) * 8 < k_last) tail_bits |= 1u << i;
    }
#pragma unroll
    for (int i = 0; i < LOADS_W; ++i) {
        const int q = (wave * LOADS_W + i) * 64 + lane;
        if (swz_chunk<RBW>(q / CPRW, q % CPRW) * (16 / WB) < k_last) tail_bits |= 1u << (LOADS_X + i);
    }
    // clipped in place when the ragged k-tile is the next one to request: every request after it is for that k-tile
    // again.  A branch that K % 64 == 0 never takes; a select per load would cost every k-tile of every shape.
    const int tail_k0 = (K % BK) != 0 ? (nk_all - 1) * BK : -1;
    auto clip_tail = [&]() __attribute__((always_inline)) {
        asm volatile("" ::: "memory");  // keeps this a branch: without it the compiler turns the block into selects
#pragma unroll
        for (int i = 0; i < LOADS_X; ++i) xd[i] = ((tail_bits >> i) & 1u) != 0 ? xd[i] : kOutOfRange;
#pragma unroll
        for (int i = 0; i < LOADS_W; ++i) wd[i] = ((tail_bits >> (LOADS_X + i)) & 1u) != 0 ? wd[i] : kOutOfRange;
    };
    auto tile_load = [&](int l, int stage, int k0) __attribute__((always_inline)) {
        const uint32_t off = l < LOADS_X ? xd[l] : wd[l - LOADS_X];
        if (l < LOADS_X) load4(xrsrc, off, lds_base + stage * X_STAGE + wave * (LOADS_X * 1024), 0, l, k0 * 2);
        else load4(wrsrc, off, lds_base + W_BASE + stage * W_STAGE + wave * (LOADS_W * 1024), (l - LOADS_X) >> 2, (l - LOADS_X) & 3, k0 * WB);
    };

    // fragment addresses: x stages are 16 KB apart (immediates 0 / 16 K / 32 K); w stages 32 KB apart, and an LDS
    // read's immediate ends at 64 KB - 1, so the third w stage has address registers of its own
    typedef __attribute__((address_space(3))) const unsigned char *lds_bytes;
    typedef __attribute__((address_space(3))) const vec8 *lds_frag;
    const lds_bytes lds0 = (lds_bytes)smem;
    lds_frag xfrag[KSTEPS][NBM], wfrag[KSTEPS][NBN], wfrag2[KSTEPS][NBN];
#pragma unroll
    for (int st = 0; st < KSTEPS; ++st) {
#pragma unroll
        for (int i = 0; i < NBM; ++i) xfrag[st][i] = (lds_frag)(lds0 + swz_offset<RB>(wave_m * (NBM * 16) + i * 16 + l16, 4 * st + g));
#pragma unroll
        for (int j = 0; j < NBN; ++j) {
            const int row = wave_n * (NBN * 16) + j * 16 + l16, unit = 4 * st + g;   // 8 k-values per unit
            wfrag[st][j] = W8 ? (lds_frag)(lds0 + W_BASE + swz_offset<RBW>(row, unit >> 1) + (unit & 1) * 8)
                              : (lds_frag)(lds0 + W_BASE + swz_offset<RBW>(row, unit));
            wfrag2[st][j] = wfrag[st][j] + 2 * (W_STAGE / 16);
        }
    }

    // Every k-tile slot issues its NL loads, so that the counter waits stay exact up to the end; requests past the
    // last k-tile fetch that tile again (into a stage nobody reads any more) instead of running past the row ends.
    int nk = nk_all, kb = 0;   // k-tiles of this workgroup: kb .. kb + nk - 1
    if constexpr (SPLIT) {
        const int per_split = (nk + splits - 1) / splits;
        kb = (int)blockIdx.y * per_split;
        nk = min(per_split, nk - kb);   // the host keeps every range non-empty
    }
#pragma unroll
    for (int s3 = 0; s3 < 3; ++s3) {
        const int k0 = (kb + min(s3, nk - 1)) * BK;
        if (k0 == tail_k0) clip_tail();   // (clipping twice changes nothing)
#pragma unroll
        for (int l = 0; l < NL; ++l) tile_load(l, s3, k0);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70 | ((2 * NL) & 15) | (((2 * NL) >> 4) << 14));  // vmcnt(2 NL): k-tile 0 has landed
    __syncthreads();

    // one-byte weights: 8 bytes per fragment, widened (byte b of a dword becomes the 16-bit value b << 8)
    typedef __attribute__((address_space(3))) const u32x2 *lds_frag8;
    auto widen8 = [&](u32x2 raw) __attribute__((always_inline)) -> vec8 {
        const u32x4 wide = {__builtin_amdgcn_perm(0u, raw[0], 0x010c000cu), __builtin_amdgcn_perm(0u, raw[0], 0x030c020cu),
                            __builtin_amdgcn_perm(0u, raw[1], 0x010c000cu), __builtin_amdgcn_perm(0u, raw[1], 0x030c020cu)};
        return __builtin_bit_cast(vec8, wide);
    };
    u32x2 wraw[W8 ? NBN : 1];
    vec8 fa[KSTEPS][NBN], fb[KSTEPS][NBM];
#pragma unroll
    for (int j = 0; j < NBN; ++j) {
        if constexpr (W8) fa[0][j] = widen8(*(lds_frag8)wfrag[0][j]);
        else fa[0][j] = *wfrag[0][j];
    }
#pragma unroll
    for (int i = 0; i < NBM; ++i) fb[0][i] = *xfrag[0][i];

    f32x4_acc acc[NBM][NBN];
#pragma unroll
    for (int i = 0; i < NBM; ++i)
#pragma unroll
        for (int j = 0; j < NBN; ++j) acc[i][j] = f32x4_acc{0.0f, 0.0f, 0.0f, 0.0f};

    // fragment reads of stage S3 for k-step st (compile-time stage: immediates, or the second register set)
    auto read_w = [&](auto s3_c, int st, int j) __attribute__((always_inline)) -> vec8 {
        constexpr int S3 = decltype(s3_c)::value;
        return S3 == 2 ? *wfrag2[st][j] : *(wfrag[st][j] + S3 * (W_STAGE / 16));
    };
    auto read_w8 = [&](auto s3_c, int st, int j) __attribute__((always_inline)) -> u32x2 {
        constexpr int S3 = decltype(s3_c)::value;
        return S3 == 2 ? *(lds_frag8)wfrag2[st][j] : *(lds_frag8)(wfrag[st][j] + S3 * (W_STAGE / 16));
    };
    auto read_x = [&](auto s3_c, int st, int i) __attribute__((always_inline)) -> vec8 {
        constexpr int S3 = decltype(s3_c)::value;
        return *(xfrag[st][i] + S3 * (X_STAGE / 16));
    };
    auto k_tile = [&](auto cur_c, int kt) __attribute__((always_inline)) {
        constexpr int CUR = decltype(cur_c)::value, NXT = (CUR + 1) % 3;
        const int k_next = (kb + min(kt + 3, nk - 1)) * BK;
        if (k_next == tail_k0 && kt + 3 == nk - 1) clip_tail();   // once: later requests are for this k-tile again
#pragma unroll
        for (int st = 0; st < KSTEPS; ++st) {
            const int sn = st ^ 1;
            if (st == 1) {
                __builtin_amdgcn_s_waitcnt(0x0F70 | (NL & 15) | ((NL >> 4) << 14));  // vmcnt(NL): k-tile kt + 1 has landed
                __syncthreads();
            }
#pragma unroll
            for (int m = 0; m < NBM * NBN; ++m) {
                const int i = m / NBN, j = m % NBN;
                mfma16_inplace(fb[st][i], fa[st][j], acc[i][j]);  // x on the A side
                const int slot = m >> 1;
                if ((m & 1) == 0 && slot < NBN + NBM) {
                    if (st == 0) {
                        if (slot < NBN) {
                            if constexpr (W8) wraw[slot] = read_w8(IntC<CUR>(), sn, slot);
                            else fa[sn][slot] = read_w(IntC<CUR>(), sn, slot);
                        } else {
                            fb[sn][slot - NBN] = read_x(IntC<CUR>(), sn, slot - NBN);
                        }
                    } else {
                        if (slot < NBN) {
                            if constexpr (W8) wraw[slot] = read_w8(IntC<NXT>(), sn, slot);
                            else fa[sn][slot] = read_w(IntC<NXT>(), sn, slot);
                        } else {
                            fb[sn][slot - NBN] = read_x(IntC<NXT>(), sn, slot - NBN);
                        }
                    }
                } else if ((m & 1) == 1) {
                    if (st == 1 && slot < NL) tile_load(slot, CUR, k_next);
                    // one-byte weights: widened two read slots after the read, when the bytes have arrived
                    if (W8 && slot >= 2 && slot - 2 < NBN) fa[sn][slot - 2] = widen8(wraw[slot - 2]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    int kt = 0;
    for (; kt + 2 < nk; kt += 3) {
        k_tile(IntC<0>(), kt);
        k_tile(IntC<1>(), kt + 1);
        k_tile(IntC<2>(), kt + 2);
    }
    if (kt < nk) k_tile(IntC<0>(), kt);
    if (kt + 1 < nk) k_tile(IntC<1>(), kt + 1);
    mfma16_inplace_results_landed(acc);
    // the residual entries of the wave's four 16-row blocks (one tile per workgroup and a long K: this one round trip
    // is not worth registers held through the main loop)
    uint32_t rres_a[4][NBN / 2] = {}, rres_b[4][NBN / 2] = {}, rres_c[4][NBN / 2] = {}, rres_d[4][NBN / 2] = {};
    const int n_lane = n0 + wave_n * (NBN * 16) + NBN * l16;
    if constexpr (RES) {
        wide_residual_fetch<T, NBN>(residual, m0 + wave_m * (NBM * 16) + 4 * g, n_lane, M, N, rres_a);
        wide_residual_fetch<T, NBN>(residual, m0 + wave_m * (NBM * 16) + 16 + 4 * g, n_lane, M, N, rres_b);
        wide_residual_fetch<T, NBN>(residual, m0 + wave_m * (NBM * 16) + 32 + 4 * g, n_lane, M, N, rres_c);
        wide_residual_fetch<T, NBN>(residual, m0 + wave_m * (NBM * 16) + 48 + 4 * g, n_lane, M, N, rres_d);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): no load may still be writing LDS when the workgroup ends

    if constexpr (SPLIT) {
        float4 *dst = reinterpret_cast<float4 *>(part) + ((((int64_t)blockIdx.y * total + t) * 4 + wave) * (NBM * NBN)) * 64 + lane;
#pragma unroll
        for (int i = 0; i < NBM; ++i)
#pragma unroll
            for (int j = 0; j < NBN; ++j)
                dst[(i * NBN + j) * 64] = float4{acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
        return;
    }
    const int n_wave = n0 + wave_n * (NBN * 16);
    uint32_t braw[NBN / 2];
    float bf[NBN];
    wide_bias_fetch<T, false, NBN>(bias, n_wave, l16, N, bias_vec_ok, braw);
    wide_bias_unpack<T, NBN>(braw, bf);
#define KERNL_HALF_EPILOGUE(I)                                                                                         \
    wide_epilogue<T, ACT, I, NBN, NBM, SCALED, RES>(acc, m0 + wave_m * (NBM * 16), n_wave, l16, g, out, act_in, M, N, out_rs, \
                                                    out_cs, ai_rs, ai_cs, out_vec_ok, ai_vec_ok, bf, rsc[SCALED ? I : 0],  \
                                                    I == 0 ? rres_a : I == 1 ? rres_b : I == 2 ? rres_c : rres_d)
    KERNL_HALF_EPILOGUE(0);
    KERNL_HALF_EPILOGUE(1);
    KERNL_HALF_EPILOGUE(2);
    KERNL_HALF_EPILOGUE(3);
#undef KERNL_HALF_EPILOGUE
}

// Second launch of the split form: workgroup (t, I) adds the k ranges' partial sums of 16-row block I of every wave of
// tile t, in range order, and runs the epilogue the unsplit kernel runs (same wave and lane geometry).
template <typename T, int ACT, int NBN>
__global__ void __launch_bounds__(256)
linear_wide_half_reduce_kernel(const float *__restrict__ part, const T *__restrict__ bias, T *__restrict__ out,
                               T *__restrict__ act_in, int M, int N, int64_t out_rs, int64_t out_cs, int64_t ai_rs,
                               int64_t ai_cs, int tiles_m, int tiles_n, int out_vec_ok, int ai_vec_ok, int bias_vec_ok,
                               int splits) {
    constexpr int NBM = 4, BM = 32 * NBM, BN = 32 * NBN;
    const int t = (int)blockIdx.x, I = (int)blockIdx.y, total = tiles_m * tiles_n;
    int m0, n0;
    half_tile_origin(t, tiles_m, tiles_n, BM, BN, m0, n0);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave & 1, wave_n = wave >> 1;
    const int l16 = lane & 15, g = lane >> 4;
    f32x4_acc acc[NBM][NBN];
#pragma unroll
    for (int i = 0; i < NBM; ++i)
#pragma unroll
        for (int j = 0; j < NBN; ++j) acc[i][j] = f32x4_acc{0.0f, 0.0f, 0.0f, 0.0f};
    const float4 *src = reinterpret_cast<const float4 *>(part) + (((int64_t)t * 4 + wave) * (NBM * NBN) + I * NBN) * 64 + lane;
    const int64_t split_stride = (int64_t)total * 4 * (NBM * NBN) * 64;
    for (int sp = 0; sp < splits; ++sp) {
        float4 v[NBN];
#pragma unroll
        for (int j = 0; j < NBN; ++j) v[j] = src[sp * split_stride + j * 64];
#pragma unroll
        for (int i = 0; i < NBM; ++i) {
            if (i != I) continue;   // (the block index of the accumulators is a compile-time constant in the epilogue)
#pragma unroll
            for (int j = 0; j < NBN; ++j) {
                acc[i][j][0] += v[j].x;
                acc[i][j][1] += v[j].y;
                acc[i][j][2] += v[j].z;
                acc[i][j][3] += v[j].w;
            }
        }
    }
    const int n_wave = n0 + wave_n * (NBN * 16);
    uint32_t braw[NBN / 2];
    float bf[NBN];
    wide_bias_fetch<T, false, NBN>(bias, n_wave, l16, N, bias_vec_ok, braw);
    wide_bias_unpack<T, NBN>(braw, bf);
    const float ones[4] = {1.0f, 1.0f, 1.0f, 1.0f};  // (the split form takes no per-row factors)
#define KERNL_HALF_REDUCE_EPILOGUE(IB)                                                                                   \
    if (I == IB)                                                                                                         \
    wide_epilogue<T, ACT, IB, NBN, NBM>(acc, m0 + wave_m * (NBM * 16), n_wave, l16, g, out, act_in, M, N, out_rs, out_cs, \
                                        ai_rs, ai_cs, out_vec_ok, ai_vec_ok, bf, ones)
    KERNL_HALF_REDUCE_EPILOGUE(0);
    KERNL_HALF_REDUCE_EPILOGUE(1);
    KERNL_HALF_REDUCE_EPILOGUE(2);
    KERNL_HALF_REDUCE_EPILOGUE(3);
#undef KERNL_HALF_REDUCE_EPILOGUE
}

// ----------------------------------------------------------------------------------------------------
// Skinny kernel: at most 64 rows of x (decoding steps, pooled outputs).  The weight matrix is the only large operand
// and the job is to stream it once at HBM speed with every CU: a workgroup owns 16 output columns (gated: their 16
// gate and 16 value rows of the interleaved weight), its 4, 8 or 16 waves split K in interleaved 64-wide chunks (long
// rows get many waves: the loop is bound by memory latency, and what counts is how many bytes a CU has in flight), every lane
// fetches 32 contiguous bytes of its weight row per chunk (4 lanes cover a 128-byte line), and the fragments go from
// global memory straight into v_mfma_f32_16x16x32 — weights on the A side, the few x rows on the B side.  The lane
// of MFMA k-group g supplies k = 16 g + 8 s .. + 7 of the chunk in step s (s = 0, 1), on both sides, which is all
// the instruction needs.  The waves' partial sums meet in LDS.  x is re-read by every workgroup, from L2.
// ----------------------------------------------------------------------------------------------------
// W8: the weight is stored as one byte per element, fp8 e5m2 — the upper byte of the fp16 encoding (reference:
// `get_model_fp8`, experimental/llama-v2/kernel/fused_kernel_fp8.py:75-84, read back with `.to(tl.float8e5,
// bitcast=True).to(tl.float16)`, fused_kernel_ff.py:43-47).  A lane then fetches its 16 weights of a chunk as ONE
// 16-byte load and byte-permutes them into the two fp16 fragments; fp16 activations only.
// RMS: x is RMS-normalised on the way in (reference: `rms_matmul_rbe`, experimental/llama-v2/kernel/
// fused_kernel_proj_qkv.py:116-183): the x fragments are multiplied by the norm's weight (rounded to 16 bit, as there),
// every lane sums the squares of the x values that pass through it, and because the inverse root mean square is one
// scalar per row it is applied to the finished sums: out = rsqrt(mean(x^2) + eps) * ((x * g) @ w^T) + bias.
// Residual: out = act(...) + residual[m, n] when a residual pointer is given (the `hidden + projection(...)` of a
// decoder layer; no counterpart in the reference, whose model adds in eager PyTorch).
// ROPE: rotary position embedding applied to the output columns below `rope_cols`, in the half-split convention —
// inside every head of `2 * half` columns, column d pairs with d + half:
//     out[d] = y[d] cos[d] - y[d + half] sin[d],   out[d + half] = y[d + half] cos[d + half] + y[d] sin[d + half]
// (reference: the rotation inside `rms_matmul_rbe_qkv`, experimental/llama-v2/kernel/fused_kernel_proj_qkv.py:69-100
// and :186-247, there on interleaved pairs with angles computed in the kernel; here from the cos / sin tables the
// model computed, indexed by the row's batch entry and position).  A workgroup then owns the 16 columns d0 .. d0 + 15
// of a head AND their partners (NR = 2 blocks, `half` columns apart), so both members of a pair meet in one lane.
struct SkinnyExtra {
    const void *residual;   // [M, N] of T, or null
    int64_t res_rs, res_cs;
    const void *cos, *sin;  // rotation tables, element (b, s, d) at b * t_bs + s * t_ss + d
    int64_t t_bs, t_ss;
    int table_dtype;        // KERNL_F16 / KERNL_BF16 / KERNL_F32
    int half;               // half the head size
    int rope_cols;          // columns [0, rope_cols) are rotated
    int rows_per_batch;     // row m of x is position m % rows_per_batch of batch entry m / rows_per_batch
};

template <typename T, int MB, bool GATED, int WAVES, int NR, bool W8 = false, bool RMS = false, bool ROPE = false>
__global__ void __launch_bounds__(64 * WAVES)
linear_skinny_kernel(const T *__restrict__ X, const T *__restrict__ W, const T *__restrict__ bias, T *__restrict__ out,
                     T *__restrict__ act_in, int M, int N, int K, int64_t ldx, int64_t out_rs, int64_t out_cs,
                     int64_t ai_rs, int64_t ai_cs, int act, const T *__restrict__ rms_w, float eps, const SkinnyExtra ex) {
    static_assert(!ROPE || (NR == 2 && !GATED && !W8), "the rotating form pairs two plain 16-column blocks");
    typedef typename Vec8<T>::type vec8;
    constexpr int NA = GATED ? 2 : 1;        // weight fragments per 16 output columns: plain, or gate and value
    constexpr int NF = NA * NR;              // weight fragments per step (NR blocks of 16 output columns)
    constexpr int U = (MB <= 2 && NF <= 2 && !RMS) ? 4 : 2;  // chunks requested together
    static_assert(WAVES * NF * MB <= 64, "partial sums fit 64 KB of LDS");
    __shared__ __attribute__((aligned(16))) float red[WAVES][NF * MB][64][4];
    __shared__ float red_sq[RMS ? WAVES : 1][MB][16];

    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const int r = lane & 15, g = lane >> 4;
    // first output column of this workgroup (N counts output columns) and the distance between its column blocks
    const int blocks_per_half = ROPE ? ex.half / 16 : 1;
    const int n0 = ROPE ? ((int)blockIdx.x / blocks_per_half) * (2 * ex.half) + ((int)blockIdx.x % blocks_per_half) * 16
                        : (int)blockIdx.x * (16 * NR);
    const int rb_stride = ROPE ? ex.half : 16;
    // first interleaved row of the 16 output columns starting at nb (gated weights: 32 gate rows, 32 value rows, ...)
    auto gated_row = [](int nb) -> int { return (nb >> 5) * 64 + (nb & 31); };
    // rows of the weight this lane reads; columns beyond N repeat the last one and are never stored
    static_assert(!W8 || std::is_same<T, f16>::value, "one-byte weights are decoded to fp16");
    typedef typename std::conditional<W8, unsigned char, T>::type WT;  // what a weight element is stored as
    const WT *wbase = reinterpret_cast<const WT *>(W);
    const WT *wp[NF];
#pragma unroll
    for (int rb = 0; rb < NR; ++rb) {
        const int nb = n0 + rb_stride * rb;
        if (GATED) {
            const int row = gated_row(min(nb, N - 16)) + r;
            wp[rb * NA] = wbase + (int64_t)row * K + 16 * g;
            wp[rb * NA + NA - 1] = wbase + (int64_t)(row + 32) * K + 16 * g;
        } else {
            wp[rb * NA] = wbase + (int64_t)min(nb + r, N - 1) * K + 16 * g;
        }
    }
    const T *xp[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) xp[mb] = X + (int64_t)min(16 * mb + r, M - 1) * ldx + 16 * g;

    f32x4_acc acc[NF][MB];
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[f][mb] = f32x4_acc{0.0f, 0.0f, 0.0f, 0.0f};

    float sq[MB];  // sum of squares of the x values this lane has seen, per 16-row block (RMS)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) sq[mb] = 0.0f;
    // Bias and residual of the block this wave finishes first (unit `wave` of the epilogue), requested before the weight
    // stream: fetched where they are used they cost the wave one more memory round trip at the very end of a kernel whose
    // whole life is a few of them.
    float pre_bias[NA][4], pre_res[4];
    if constexpr (!ROPE) {
        const int rb = wave / MB, mb = wave % MB;
        const int nb = n0 + 16 * rb, m = 16 * mb + r;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int n = nb + 4 * g + e;
            const bool live = wave < NR * MB && m < M && n < N;
            const int brow = GATED ? gated_row(nb) + 4 * g + e : n;
            pre_bias[0][e] = (live && bias != nullptr) ? to_float(bias[brow]) : 0.0f;
            if (GATED) pre_bias[NA - 1][e] = (live && bias != nullptr) ? to_float(bias[brow + 32]) : 0.0f;
            pre_res[e] = (live && ex.residual != nullptr)
                             ? to_float(static_cast<const T *>(ex.residual)[(int64_t)m * ex.res_rs + (int64_t)n * ex.res_cs]) : 0.0f;
        }
    }
    const int nchunks = K / 64;
    const int rot = (int)((blockIdx.x * 13u) % (unsigned)nchunks);
    for (int c0 = wave; c0 < nchunks; c0 += WAVES * U) {
        vec8 wf[U][NF][2], xf[U][MB][2], gf[RMS ? U : 1][2];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            // chunks past the end are neither fetched nor multiplied (the test is uniform over the wave); only the
            // 16-wave form with 128 fragment registers in flight, which has none to spare for the branches, fetches
            // the last chunk again instead.  Workgroups walk the chunks from different starting points, so that they
            // do not all ask L2 for the same lines of x at once.
            constexpr bool kSkipTail = !(WAVES == 16 && U * (NF + MB) >= 16);
            if (kSkipTail && c0 + WAVES * u >= nchunks) continue;
            int cc = min(c0 + WAVES * u, nchunks - 1) + rot;
            cc = cc >= nchunks ? cc - nchunks : cc;
            const int k0 = cc * 64;
#pragma unroll
            for (int f = 0; f < NF; ++f) {
                if constexpr (W8) {
                    const u32x4 raw = *reinterpret_cast<const u32x4 *>(wp[f] + k0);
                    u32x4 lo, hi;  // bytes {0, b0, 0, b1} / {0, b2, 0, b3} of every word: fp16 pairs
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        lo[2 * j] = __builtin_amdgcn_perm(0u, raw[j], 0x010c000cu);
                        lo[2 * j + 1] = __builtin_amdgcn_perm(0u, raw[j], 0x030c020cu);
                        hi[2 * j] = __builtin_amdgcn_perm(0u, raw[2 + j], 0x010c000cu);
                        hi[2 * j + 1] = __builtin_amdgcn_perm(0u, raw[2 + j], 0x030c020cu);
                    }
                    wf[u][f][0] = __builtin_bit_cast(vec8, lo);
                    wf[u][f][1] = __builtin_bit_cast(vec8, hi);
                } else {
                    wf[u][f][0] = *reinterpret_cast<const vec8 *>(wp[f] + k0);
                    wf[u][f][1] = *reinterpret_cast<const vec8 *>(wp[f] + k0 + 8);
                }
            }
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                xf[u][mb][0] = *reinterpret_cast<const vec8 *>(xp[mb] + k0);
                xf[u][mb][1] = *reinterpret_cast<const vec8 *>(xp[mb] + k0 + 8);
            }
            if constexpr (RMS) {
                gf[u][0] = *reinterpret_cast<const vec8 *>(rms_w + k0 + 16 * g);
                gf[u][1] = *reinterpret_cast<const vec8 *>(rms_w + k0 + 16 * g + 8);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (c0 + WAVES * u < nchunks) {
                if constexpr (RMS) {
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
#pragma unroll
                            for (int e = 0; e < 8; ++e) {
                                const float xv = to_float(xf[u][mb][h][e]);
                                sq[mb] = fmaf(xv, xv, sq[mb]);
                            }
                            xf[u][mb][h] = xf[u][mb][h] * gf[u][h];
                        }
                }
#pragma unroll
                for (int f = 0; f < NF; ++f)
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb) {
                        acc[f][mb] = mfma16(wf[u][f][0], xf[u][mb][0], acc[f][mb]);
                        acc[f][mb] = mfma16(wf[u][f][1], xf[u][mb][1], acc[f][mb]);
                    }
            }
        }
    }

#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[wave][f * MB + mb][lane][e] = acc[f][mb][e];
    if constexpr (RMS) {
        // a row's squares are spread over the 4 lanes r, r + 16, r + 32, r + 48 of every wave
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            float t = sq[mb];
            t += __shfl_xor(t, 16, 64);
            t += __shfl_xor(t, 32, 64);
            if (g == 0) red_sq[wave][mb][r] = t;
        }
    }
    __syncthreads();

    // the waves share the NR x MB blocks of 16 columns x 16 rows: element e of a lane is output column nb + 4 g + e
    // of x row 16 mb + r
    if constexpr (ROPE) {
        // a wave takes both column blocks of a 16-row block: element e of a lane is column n0 + 4 g + e and its partner
        for (int mb = wave; mb < MB; mb += WAVES) {
            const int m = 16 * mb + r;
            float rstd = 1.0f;
            if constexpr (RMS) {
                float t = 0.0f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) t += red_sq[w][mb][r];
                rstd = 1.0f / sqrtf(t / (float)K + eps);
            }
            const int64_t trow = (int64_t)(min(m, M - 1) / ex.rows_per_batch) * ex.t_bs + (int64_t)(min(m, M - 1) % ex.rows_per_batch) * ex.t_ss;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int n = n0 + 4 * g + e;   // lower member of the pair; the upper one is `half` columns further
                float v[2];
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    float t4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int w = 0; w < WAVES; ++w) t4[w & 3] += red[w][a * MB + mb][lane][e];
                    v[a] = ((t4[0] + t4[1]) + (t4[2] + t4[3])) * rstd;
                }
                if (m >= M || n >= N) continue;
                if (bias != nullptr) {
                    v[0] += to_float(bias[n]);
                    v[1] += to_float(bias[n + ex.half]);
                }
                float y0 = v[0], y1 = v[1];
                if (n < ex.rope_cols) {
                    const int d = n % (2 * ex.half);
                    const float c0 = table_value(ex.cos, ex.table_dtype, trow + d), s0 = table_value(ex.sin, ex.table_dtype, trow + d);
                    const float c1 = table_value(ex.cos, ex.table_dtype, trow + d + ex.half);
                    const float s1 = table_value(ex.sin, ex.table_dtype, trow + d + ex.half);
                    y0 = v[0] * c0 - v[1] * s0;
                    y1 = v[1] * c1 + v[0] * s1;
                }
                if (ex.residual != nullptr) {
                    const T *res = static_cast<const T *>(ex.residual) + (int64_t)m * ex.res_rs;
                    y0 += to_float(res[(int64_t)n * ex.res_cs]);
                    y1 += to_float(res[(int64_t)(n + ex.half) * ex.res_cs]);
                }
                out[(int64_t)m * out_rs + (int64_t)n * out_cs] = from_float<T>(y0);
                out[(int64_t)m * out_rs + (int64_t)(n + ex.half) * out_cs] = from_float<T>(y1);
            }
        }
        return;
    }
    for (int unit = wave; unit < NR * MB; unit += WAVES) {
        const int rb = unit / MB, mb = unit % MB;
        const int nb = n0 + 16 * rb;
        const int m = 16 * mb + r;
        float rstd = 1.0f;
        if constexpr (RMS) {
            float t = 0.0f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) t += red_sq[w][mb][r];
            rstd = 1.0f / sqrtf(t / (float)K + eps);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int n = nb + 4 * g + e;
            float v[NA];
#pragma unroll
            for (int a = 0; a < NA; ++a) {
                float t4[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // fixed summation order: the result does not depend on timing
#pragma unroll
                for (int w = 0; w < WAVES; ++w) t4[w & 3] += red[w][(rb * NA + a) * MB + mb][lane][e];
                v[a] = ((t4[0] + t4[1]) + (t4[2] + t4[3])) * rstd;
            }
            if (m >= M || n >= N) continue;
            const bool first = unit == wave;  // what this block needs from memory is here already
            if (first) {
                v[0] += pre_bias[0][e];
                if (GATED) v[NA - 1] += pre_bias[NA - 1][e];
            } else if (bias != nullptr) {
                const int brow = GATED ? gated_row(nb) + 4 * g + e : n;
                v[0] += to_float(bias[brow]);
                if (GATED) v[NA - 1] += to_float(bias[brow + 32]);
            }
            if (!GATED && act_in != nullptr) act_in[(int64_t)m * ai_rs + (int64_t)n * ai_cs] = from_float<T>(v[0]);
            float y = apply_act16(v[0], act);
            if (GATED) y *= v[NA - 1];
            if (first) y += pre_res[e];
            else if (ex.residual != nullptr)
                y += to_float(static_cast<const T *>(ex.residual)[(int64_t)m * ex.res_rs + (int64_t)n * ex.res_cs]);
            out[(int64_t)m * out_rs + (int64_t)n * out_cs] = from_float<T>(y);
        }
    }
}

// ----------------------------------------------------------------------------------------------------
// FMA kernel: any dtype, any strides.  64x64 output tile, 16x16 threads, 4x4 outputs per thread, fp32 LDS tiles.
// ----------------------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
linear_fma_kernel(const T *__restrict__ X, const T *__restrict__ W, const T *__restrict__ bias,
                  T *__restrict__ out, T *__restrict__ act_in, int M, int N, int K, int64_t x_rs, int64_t x_cs,
                  int64_t out_rs, int64_t out_cs, int64_t ai_rs, int64_t ai_cs, int act) {
    __shared__ float xs[16][64 + 1];
    __shared__ float ws[16][64 + 1];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += 16) {
        for (int e = threadIdx.x; e < 64 * 16; e += 256) {
            const int r = e >> 4, kk = e & 15;
            const int gm = m0 + r, gn = n0 + r, gk = k0 + kk;
            xs[kk][r] = (gm < M && gk < K) ? to_float(X[(int64_t)gm * x_rs + (int64_t)gk * x_cs]) : 0.0f;
            ws[kk][r] = (gn < N && gk < K) ? to_float(W[(int64_t)gn * K + gk]) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
        }
        __syncthreads();
    }
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n >= N) continue;
            float r = acc[i][j];
            if (bias != nullptr) r += to_float(bias[n]);
            if (act_in != nullptr) act_in[(int64_t)m * ai_rs + (int64_t)n * ai_cs] = from_float<T>(r);
            out[(int64_t)m * out_rs + (int64_t)n * out_cs] = from_float<T>(apply_act(r, act));
        }
    }
}

// ----------------------------------------------------------------------------------------------------
// host dispatch
// ----------------------------------------------------------------------------------------------------
struct LinearArgs {
    const void *x, *w, *bias;
    void *out, *act_in;
    int M, N, K;
    int64_t x_rs, x_cs, out_rs, out_cs, ai_rs, ai_cs;
    int act;
    hipStream_t st;
    const SkinnyExtra *extra = nullptr;  // residual / rotation of the few-row kernel (decoding steps)
    const float *row_scale = nullptr;    // fp32 [M] factors of the finished sums (wide kernels only)
    const void *residual = nullptr;      // [M, N] matrix added to the rounded results (wide kernels, plain epilogue, no activation)
    int64_t res_rs = 0, res_cs = 0;
};

template <typename T, int NBN>
static WideResidual wide_residual_of(const LinearArgs &a) {
    WideResidual r;
    r.ptr = a.residual;
    r.rs = a.res_rs;
    r.cs = a.res_cs;
    // 16-byte pieces at columns that are multiples of 8, or 12-byte pieces (4-byte aligned) at multiples of 6
    r.vec_ok = a.residual != nullptr && a.res_cs == 1 &&
               (NBN == 8 ? (a.res_rs % 8 == 0 && aligned16(a.residual)) : (a.res_rs % 2 == 0 && (reinterpret_cast<uintptr_t>(a.residual) & 3) == 0));
    return r;
}

template <typename T, typename Cfg, int ACT, bool W8 = false>
static void launch_mfma_act(const LinearArgs &a) {
    auto kern = linear_mfma_kernel<T, Cfg, ACT, W8>;
    static bool attr_done = false;  // benign race: the attribute call is idempotent
    if (!attr_done) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, Cfg::LDS_BYTES);
        attr_done = true;
    }
    const int tiles_m = (a.M + Cfg::BM - 1) / Cfg::BM, tiles_n = (a.N + Cfg::BN - 1) / Cfg::BN;
    const int per_xcd = (tiles_m * tiles_n + 7) / 8;
    const T *x = static_cast<const T *>(a.x);
    const T *w = static_cast<const T *>(a.w);
    const T *bias = static_cast<const T *>(a.bias);
    T *out = static_cast<T *>(a.out);
    T *act_in = static_cast<T *>(a.act_in);
    const int out_vec_ok = a.out_cs == 1 && a.out_rs % 8 == 0 && aligned16(out);
    const int ai_vec_ok = act_in != nullptr && a.ai_cs == 1 && a.ai_rs % 8 == 0 && aligned16(act_in);
    const int bias_vec_ok = bias != nullptr && aligned16(bias);
    hipLaunchKernelGGL(kern, dim3(per_xcd * 8), dim3(Cfg::THREADS), Cfg::LDS_BYTES, a.st, x, w, bias, out,
                       act_in, a.M, a.N, a.K, a.x_rs, a.out_rs, a.out_cs, a.ai_rs, a.ai_cs, tiles_m, tiles_n,
                       out_vec_ok, ai_vec_ok, bias_vec_ok);
}

template <typename T, typename Cfg>
static void launch_mfma_cfg(const LinearArgs &a) {
    switch (a.act) {
        case KERNL_ACT_RELU: launch_mfma_act<T, Cfg, KERNL_ACT_RELU>(a); break;
        case KERNL_ACT_TANH: launch_mfma_act<T, Cfg, KERNL_ACT_TANH>(a); break;
        case KERNL_ACT_GELU_ERF: launch_mfma_act<T, Cfg, KERNL_ACT_GELU_ERF>(a); break;
        case KERNL_ACT_GELU_TANH: launch_mfma_act<T, Cfg, KERNL_ACT_GELU_TANH>(a); break;
        case KERNL_ACT_SILU: launch_mfma_act<T, Cfg, KERNL_ACT_SILU>(a); break;
        default: launch_mfma_act<T, Cfg, KERNL_ACT_NONE>(a); break;
    }
}

// one-byte weights (fp16 activations)
template <typename Cfg>
static void launch_mfma_w8(const LinearArgs &a) {
    switch (a.act) {
        case KERNL_ACT_RELU: launch_mfma_act<f16, Cfg, KERNL_ACT_RELU, true>(a); break;
        case KERNL_ACT_TANH: launch_mfma_act<f16, Cfg, KERNL_ACT_TANH, true>(a); break;
        case KERNL_ACT_GELU_ERF: launch_mfma_act<f16, Cfg, KERNL_ACT_GELU_ERF, true>(a); break;
        case KERNL_ACT_GELU_TANH: launch_mfma_act<f16, Cfg, KERNL_ACT_GELU_TANH, true>(a); break;
        case KERNL_ACT_SILU: launch_mfma_act<f16, Cfg, KERNL_ACT_SILU, true>(a); break;
        default: launch_mfma_act<f16, Cfg, KERNL_ACT_NONE, true>(a); break;
    }
}

// gated epilogues: tiles whose waves span an even number of 32-column blocks
template <typename T, typename Cfg>
static void launch_mfma_glu(const LinearArgs &a) {
    switch (a.act & (kGluBit - 1)) {
        case KERNL_ACT_GELU_ERF: launch_mfma_act<T, Cfg, kGluBit | KERNL_ACT_GELU_ERF>(a); break;
        case KERNL_ACT_GELU_TANH: launch_mfma_act<T, Cfg, kGluBit | KERNL_ACT_GELU_TANH>(a); break;
        case KERNL_ACT_RELU: launch_mfma_act<T, Cfg, kGluBit | KERNL_ACT_RELU>(a); break;
        case KERNL_ACT_NONE: launch_mfma_act<T, Cfg, kGluBit | KERNL_ACT_NONE>(a); break;
        case KERNL_ACT_TANH: launch_mfma_act<T, Cfg, kGluBit | KERNL_ACT_TANH>(a); break;
        default: launch_mfma_act<T, Cfg, kGluBit | KERNL_ACT_SILU>(a); break;
    }
}

template <typename T, int ACT, int NBN = 8, bool W8 = false, bool SCALED = false, bool RES = false>
static void launch_wide_act(const LinearArgs &a) {
    auto kern = linear_wide_kernel<T, ACT, NBN, W8, SCALED, RES>;
    constexpr int LDS_BYTES = 2 * (256 + 256) * 128;  // two stages
    static bool attr_done = false;  // benign race: the attribute call is idempotent
    if (!attr_done) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        attr_done = true;
    }
    const int tiles_m = (a.M + 255) / 256, tiles_n = (a.N + 32 * NBN - 1) / (32 * NBN);
    const int per_xcd = (tiles_m * tiles_n + 7) / 8;
    const T *bias = static_cast<const T *>(a.bias);
    T *out = static_cast<T *>(a.out);
    T *act_in = static_cast<T *>(a.act_in);
    const int out_vec_ok = a.out_cs == 1 && a.out_rs % 8 == 0 && aligned16(out);
    const int ai_vec_ok = act_in != nullptr && a.ai_cs == 1 && a.ai_rs % 8 == 0 && aligned16(act_in);
    const int bias_vec_ok = bias != nullptr && aligned16(bias);
    // persistent: at most one workgroup per CU (32 per XCD), each walks its share of the XCD's tiles.  The kernel
    // needs every tile to start in LDS stage 0: with an odd number of k-tiles each workgroup gets a single tile.
    const int slots = (per_xcd < 32 || ((a.K + 63) / 64) % 2 != 0) ? per_xcd : 32;
    hipLaunchKernelGGL(kern, dim3(slots * 8), dim3(256), LDS_BYTES, a.st, static_cast<const T *>(a.x),
                       static_cast<const T *>(a.w), bias, out, act_in, a.M, a.N, a.K, a.x_rs, a.out_rs, a.out_cs, a.ai_rs,
                       a.ai_cs, tiles_m, tiles_n, out_vec_ok, ai_vec_ok, bias_vec_ok, a.row_scale, wide_residual_of<T, NBN>(a));
}

template <typename T, int ACT, int NBN, bool W8 = false, bool SCALED = false, bool RES = false>
static void launch_wide_half_act(const LinearArgs &a) {
    auto kern = linear_wide_half_kernel<T, ACT, NBN, W8, false, SCALED, RES>;
    constexpr int LDS_BYTES = 3 * 16384 + 3 * 32768;  // three stages
    static bool attr_done = false;  // benign race: the attribute call is idempotent
    if (!attr_done) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        attr_done = true;
    }
    const int tiles_m = (a.M + 127) / 128, tiles_n = (a.N + 32 * NBN - 1) / (32 * NBN);
    const int per_xcd = (tiles_m * tiles_n + 7) / 8;
    const T *bias = static_cast<const T *>(a.bias);
    T *out = static_cast<T *>(a.out);
    T *act_in = static_cast<T *>(a.act_in);
    const int out_vec_ok = a.out_cs == 1 && a.out_rs % 8 == 0 && aligned16(out);
    const int ai_vec_ok = act_in != nullptr && a.ai_cs == 1 && a.ai_rs % 8 == 0 && aligned16(act_in);
    const int bias_vec_ok = bias != nullptr && aligned16(bias);
    hipLaunchKernelGGL(kern, dim3(per_xcd * 8), dim3(256), LDS_BYTES, a.st, static_cast<const T *>(a.x),
                       static_cast<const T *>(a.w), bias, out, act_in, a.M, a.N, a.K, a.x_rs, a.out_rs, a.out_cs, a.ai_rs,
                       a.ai_cs, tiles_m, tiles_n, out_vec_ok, ai_vec_ok, bias_vec_ok, static_cast<float *>(nullptr), 1, a.row_scale,
                       wide_residual_of<T, NBN>(a));
}

// Split form of the 128 x 192 kernel for row counts that leave most CUs without a tile (129 to about 700 rows against
// a few thousand columns): `splits` ranges of k-tiles per output tile, then the launch that adds them.
struct HalfSplitPlan {
    int tiles_m, tiles_n, splits;
    int64_t bytes;
};
static HalfSplitPlan half_split_plan(int64_t M, int64_t N, int64_t K) {
    HalfSplitPlan p;
    p.tiles_m = (int)((M + 127) / 128);
    p.tiles_n = (int)((N + 191) / 192);
    const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
    const int nk = (int)(K / 64);
    int64_t splits = 256 / tiles;           // one round of workgroups
    if (splits > nk / 16) splits = nk / 16; // ranges of at least 16 k-tiles: with K = 768 two ranges cost more (14 us) than one tile pass (11)
    if (splits > 4) splits = 4;             // partial tiles cost HBM traffic: rows x columns x 8 bytes per range
    if (splits < 1) splits = 1;
    // ranges of ceil(nk / splits) k-tiles: drop ranges that would be empty
    const int per = (nk + (int)splits - 1) / (int)splits;
    p.splits = (nk + per - 1) / per;
    p.bytes = p.splits > 1 ? (int64_t)p.splits * tiles * 128 * 192 * 4 : 0;
    return p;
}

template <typename T, int ACT>
static void launch_half_split_act(const LinearArgs &a, const HalfSplitPlan &p, float *part) {
    constexpr int NBN = 6;
    auto kern = linear_wide_half_kernel<T, KERNL_ACT_NONE, NBN, false, true>;
    constexpr int LDS_BYTES = 3 * 16384 + 3 * 32768;
    static bool attr_done = false;  // benign race: the attribute call is idempotent
    if (!attr_done) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        attr_done = true;
    }
    const int per_xcd = (p.tiles_m * p.tiles_n + 7) / 8;
    const T *bias = static_cast<const T *>(a.bias);
    T *out = static_cast<T *>(a.out);
    T *act_in = static_cast<T *>(a.act_in);
    const int out_vec_ok = a.out_cs == 1 && a.out_rs % 8 == 0 && aligned16(out);
    const int ai_vec_ok = act_in != nullptr && a.ai_cs == 1 && a.ai_rs % 8 == 0 && aligned16(act_in);
    const int bias_vec_ok = bias != nullptr && aligned16(bias);
    hipLaunchKernelGGL(kern, dim3(per_xcd * 8, p.splits), dim3(256), LDS_BYTES, a.st, static_cast<const T *>(a.x),
                       static_cast<const T *>(a.w), bias, out, act_in, a.M, a.N, a.K, a.x_rs, a.out_rs, a.out_cs, a.ai_rs,
                       a.ai_cs, p.tiles_m, p.tiles_n, out_vec_ok, ai_vec_ok, bias_vec_ok, part, p.splits, static_cast<const float *>(nullptr),
                       WideResidual());
    hipLaunchKernelGGL((linear_wide_half_reduce_kernel<T, ACT, NBN>), dim3(p.tiles_m * p.tiles_n, 4), dim3(256), 0, a.st,
                       part, bias, out, act_in, a.M, a.N, a.out_rs, a.out_cs, a.ai_rs, a.ai_cs, p.tiles_m, p.tiles_n,
                       out_vec_ok, ai_vec_ok, bias_vec_ok, p.splits);
}

template <typename T>
static void launch_half_split(const LinearArgs &a, const HalfSplitPlan &p, float *part) {
    switch (a.act) {
        case KERNL_ACT_RELU: launch_half_split_act<T, KERNL_ACT_RELU>(a, p, part); break;
        case KERNL_ACT_TANH: launch_half_split_act<T, KERNL_ACT_TANH>(a, p, part); break;
        case KERNL_ACT_GELU_ERF: launch_half_split_act<T, KERNL_ACT_GELU_ERF>(a, p, part); break;
        case KERNL_ACT_GELU_TANH: launch_half_split_act<T, KERNL_ACT_GELU_TANH>(a, p, part); break;
        case KERNL_ACT_SILU: launch_half_split_act<T, KERNL_ACT_SILU>(a, p, part); break;
        default: launch_half_split_act<T, KERNL_ACT_NONE>(a, p, part); break;
    }
}

template <typename T, int NBN>
static void launch_wide_half(const LinearArgs &a) {
    if (a.residual != nullptr) {   // (the entry point admits no activation and no per-row factors with a residual)
        launch_wide_half_act<T, KERNL_ACT_NONE, NBN, false, false, true>(a);
        return;
    }
    if (a.row_scale != nullptr) {  // (the entry point admits no activation with per-row factors here)
        launch_wide_half_act<T, KERNL_ACT_NONE, NBN, false, true>(a);
        return;
    }
    switch (a.act) {
        case KERNL_ACT_RELU: launch_wide_half_act<T, KERNL_ACT_RELU, NBN>(a); break;
        case KERNL_ACT_TANH: launch_wide_half_act<T, KERNL_ACT_TANH, NBN>(a); break;
        case KERNL_ACT_GELU_ERF: launch_wide_half_act<T, KERNL_ACT_GELU_ERF, NBN>(a); break;
        case KERNL_ACT_GELU_TANH: launch_wide_half_act<T, KERNL_ACT_GELU_TANH, NBN>(a); break;
        case KERNL_ACT_SILU: launch_wide_half_act<T, KERNL_ACT_SILU, NBN>(a); break;
        default: launch_wide_half_act<T, KERNL_ACT_NONE, NBN>(a); break;
    }
}

template <typename T>
static void launch_wide192(const LinearArgs &a) {
    if (a.residual != nullptr) {
        launch_wide_act<T, KERNL_ACT_NONE, 6, false, false, true>(a);
        return;
    }
    if (a.row_scale != nullptr) {
        launch_wide_act<T, KERNL_ACT_NONE, 6, false, true>(a);
        return;
    }
    switch (a.act) {
        case KERNL_ACT_RELU: launch_wide_act<T, KERNL_ACT_RELU, 6>(a); break;
        case KERNL_ACT_TANH: launch_wide_act<T, KERNL_ACT_TANH, 6>(a); break;
        case KERNL_ACT_GELU_ERF: launch_wide_act<T, KERNL_ACT_GELU_ERF, 6>(a); break;
        case KERNL_ACT_GELU_TANH: launch_wide_act<T, KERNL_ACT_GELU_TANH, 6>(a); break;
        case KERNL_ACT_SILU: launch_wide_act<T, KERNL_ACT_SILU, 6>(a); break;
        default: launch_wide_act<T, KERNL_ACT_NONE, 6>(a); break;
    }
}

template <typename T>
static void launch_wide(const LinearArgs &a) {
    if (a.residual != nullptr) {
        launch_wide_act<T, KERNL_ACT_NONE, 8, false, false, true>(a);
        return;
    }
    if (a.row_scale != nullptr) {  // (the entry point admits SiLU gates and plain sums with per-row factors)
        if (a.act & kGluBit) launch_wide_act<T, kGluBit | KERNL_ACT_SILU, 8, false, true>(a);
        else launch_wide_act<T, KERNL_ACT_NONE, 8, false, true>(a);
        return;
    }
    if (a.act & kGluBit) {
        switch (a.act & (kGluBit - 1)) {
            case KERNL_ACT_GELU_ERF: launch_wide_act<T, kGluBit | KERNL_ACT_GELU_ERF>(a); break;
            case KERNL_ACT_GELU_TANH: launch_wide_act<T, kGluBit | KERNL_ACT_GELU_TANH>(a); break;
            case KERNL_ACT_RELU: launch_wide_act<T, kGluBit | KERNL_ACT_RELU>(a); break;
            case KERNL_ACT_NONE: launch_wide_act<T, kGluBit | KERNL_ACT_NONE>(a); break;
            case KERNL_ACT_TANH: launch_wide_act<T, kGluBit | KERNL_ACT_TANH>(a); break;
            default: launch_wide_act<T, kGluBit | KERNL_ACT_SILU>(a); break;
        }
        return;
    }
    switch (a.act) {
        case KERNL_ACT_RELU: launch_wide_act<T, KERNL_ACT_RELU>(a); break;
        case KERNL_ACT_TANH: launch_wide_act<T, KERNL_ACT_TANH>(a); break;
        case KERNL_ACT_GELU_ERF: launch_wide_act<T, KERNL_ACT_GELU_ERF>(a); break;
        case KERNL_ACT_GELU_TANH: launch_wide_act<T, KERNL_ACT_GELU_TANH>(a); break;
        case KERNL_ACT_SILU: launch_wide_act<T, KERNL_ACT_SILU>(a); break;
        default: launch_wide_act<T, KERNL_ACT_NONE>(a); break;
    }
}

//                         BM   BN  BK  WAVES_M WAVES_N  MIN_BLOCKS
typedef LinearTile<256, 256, 64, 2, 4, 1> Tile256x256;
typedef LinearTile<256, 192, 64, 4, 2, 1> Tile256x192;
typedef LinearTile<128, 128, 64, 2, 2, 2> Tile128x128;
typedef LinearTile<256, 128, 32, 2, 2, 2> Tile256x128k32;  // 48 KB of LDS: two workgroups per CU

// Run-time proxy of a tile shape: tiles one CU has to work through, times the tile's area relative to 256x256, times
// a speed factor of the kernel that runs it (measured on the Llama-7B and BERT-base shapes: the wide kernel's k-loop is
// the fastest, and the longer K is the more the 8-wave kernels fall behind it).
static double tile_cost(int M, int N, int K, int bm, int bn, double base, double per_k) {
    const int64_t tiles = (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
    const int64_t per_cu = (tiles + 255) / 256;
    const double kf = (double)K / ((double)K + 1500.0);
    return (double)per_cu * ((double)bm * bn / 65536.0) * (base + per_k * kf);
}
// which: 1 = 256x256, 2 = 256x192, 3 = 128x128 (8-wave kernel), 5 = wide 256x256, 6 = wide 256x192, 7 = wide 128x256, 8 = wide 128x192
static int pick_tile(int M, int N, int K, bool gated, bool wide_only = false) {
    // (the wide kernels take any K the MFMA path takes, with a zero-filled last k-tile)
    int pick = 5;
    double best = tile_cost(M, N, K, 256, 256, 1.0, 0.0);
    const double c6 = gated ? 1e30 : tile_cost(M, N, K, 256, 192, 1.04, 0.0);
    if (c6 < best) { best = c6; pick = 6; }
    // half-height tiles: a quarter slower per output element at long K (more operand traffic per MFMA), and a
    // prologue per tile that weighs more the shorter K is; they win where 256-row tiles leave CUs idle
    const double c7 = gated ? 1e30 : tile_cost(M, N, K, 128, 256, 1.5, -0.35);
    if (c7 < best) { best = c7; pick = 7; }
    const double c8 = gated ? 1e30 : tile_cost(M, N, K, 128, 192, 1.65, -0.35);
    if (c8 < best) { best = c8; pick = 8; }
    // 256x192 gives a wave an odd number of column blocks: not usable for gate/value pairs
    // (wide_only: the caller needs an epilogue only the wide kernels have)
    const double c2 = gated || wide_only ? 1e30 : tile_cost(M, N, K, 256, 192, 1.2, 0.3);
    const double c3 = wide_only ? 1e30 : tile_cost(M, N, K, 128, 128, 1.9, 0.4);
    if (c2 < best) { best = c2; pick = 2; }
    if (c3 < best) { best = c3; pick = 3; }
    return pick;
}

// Which of the small-problem kernels (linear_small.hip) takes M x N x K, as the value of the tile hook that forces it
// (10 / 11 / 15: 32 x 64 / 64 x 64 / 64 x 128 tiles shared by the waves; 12 / 13 / 14: 16 x 32 / 32 x 32 / 64 x 32 tiles with
// the k-tiles dealt to the waves), or 0 when the problem is not their kind.  One round of workgroups is the condition for all of them.
//  - dealt k-tiles: weights of up to 8 M elements, 8 rows or more (fewer stream the weight faster), at most 256 tiles.
//    Graph replay, us, against what ran before: 16 x 768 x 3072 6.7 (9.0), 64 x 768 x 3072 8.0 (11.6), 128 x 768 x 3072
//    8.4 (14.3), 256 x 768 x 3072 9.8 (15.8), 128 x 768 x 768 5.1 (7.3), 64 x 2304 x 768 5.4 (7.6), 128 x 2048 x 2048 9.0
//    (15.2), 128 x 1024 x 8192 15.3 (25.3), 32 x 8192 x 1024 6.5 (10.1); 64 x 32 tiles where 32 x 32 need a second round:
//    512 x 768 x 3072 12.4 (18.3), 384 x 1024 x 4096 14.8 (18.7), 256 x 2048 x 2048 10.9 (17.1), 128 x 3072 x 768 7.1 (shared
//    32 x 64 tiles: 7.9);
//    4096 x 4096 and larger stay where they were.
//  - shared tiles: more than 64 rows and K < 1536 (from there on the stream-K / split-K kernels or the big tiles are
//    ahead): 128 x 2304 x 768 7.7 (11.7), 128 x 3072 x 768 8.3 (11.7), 512 x 768 x 768 7.6 (11.0), 512 x 1024 x 1024 8.6
//    (13.0), 128 x 4096 x 1024 10.0 (14.4); 64-row tiles: 256 x 3072 x 768 11.2 (11.8), 1024 x 1024 x 1024 12.2 (14.0).
//    With the tiles that share a weight tile on one XCD, one round of 64 x 64 tiles also wins over a long K where the
//    dealt tiles need two (1024 x 768 x 1536 10.8 against 18.5, 512 x 2048 x 2048 13.0 (19.2), 1024 x 768 x 3072 16.8
//    (18.9)), and one round of 64 x 128 tiles over a short K where 64 x 64 need two (512 x 3072 x 768 10.3 (12.3),
//    512 x 2304 x 768 10.1 (11.9), 2048 x 768 x 768 10.7 (12.2), 512 x 4096 x 1024 12.3 (14.7)).
static int small_problem_kind(int64_t M, int64_t N, int64_t K) {
    const int64_t cols32 = (N + 31) / 32, cols64 = (N + 63) / 64;
    const bool small_weight = N * K <= ((int64_t)1 << 23), short_k = M > 64 && K < 1536;
    if (small_weight && M >= 8 && M <= 16 && cols32 <= 256) return 12;
    if (small_weight && M > 16 && ((M + 31) / 32) * cols32 <= 256) return 13;
    if (small_weight && M > 16 && ((M + 63) / 64) * cols32 <= 256) return 14;
    if (short_k && ((M + 31) / 32) * cols64 <= 256) return 10;
    if (short_k && ((M + 63) / 64) * cols64 <= 256) return 11;
    // one round of 64 x 64 tiles over a long K where the dealt tiles would need a second one
    if (small_weight && M > 64 && ((M + 63) / 64) * cols64 <= 256) return 11;
    // short K, one round of 64 x 128 tiles where 64 x 64 would need two
    if (short_k && ((M + 63) / 64) * ((N + 127) / 128) <= 256) return 15;
    return 0;
}

extern int g_linear_force_tile;  // test / tuning hook (defined in linear.hip): 0 = heuristic, 1 = 256x256, 2 = 256x192, 3 = 128x128, 4 = 256x128 k32, 5 = wide 256x256, 6 = wide 256x192, 7 = wide 128x256, 8 = wide 128x192, 10 .. 15 = the small-problem kernels

template <typename T, bool GATED, int MB, int NR, bool W8, bool RMS = false, bool ROPE = false>
static void launch_skinny_blocks(const LinearArgs &a, const void *rms_w = nullptr, float eps = 0.0f,
                                 const SkinnyExtra *extra = nullptr) {
    const int n_out = GATED ? a.N / 2 : a.N;
    const dim3 grid((unsigned)((n_out + 16 * NR - 1) / (16 * NR)));  // the rotating form: N is a multiple of the head size
    SkinnyExtra ex = {};
    if (extra != nullptr) ex = *extra;
    else if (a.extra != nullptr) ex = *a.extra;
    const int act = a.act & (kGluBit - 1);
    // waves per workgroup: enough to have a whole block of weight rows in flight when K is long, never more than
    // there are chunks, and no more than the LDS for their partial sums allows
    const int nchunks = a.K / 64;
    // (the normalising form also keeps a few more loads per chunk in flight: half the waves for it)
    constexpr int kUnits = (GATED ? 2 : 1) * NR * MB * (RMS ? 2 : 1);
    constexpr int kMaxWaves = kUnits > 8 ? 4 : kUnits > 4 ? 8 : 16;
    // ... and few enough that the workgroups one CU gets (256 CUs) are resident together: a 1024-thread workgroup
    // fills half a CU, and 344 of them would leave a third of the chip idle
    const int per_cu = ((int)grid.x + 255) / 256;
    int waves = nchunks >= 64 ? 16 : nchunks >= 24 ? 8 : 4;
    if (per_cu >= 3) waves = 4;
    else if (per_cu == 2 && waves > 8) waves = 8;
#define KERNL_SKINNY(WV)                                                                                                \
    hipLaunchKernelGGL((linear_skinny_kernel<T, MB, GATED, WV, NR, W8, RMS, ROPE>), grid, dim3(64 * WV), 0, a.st,                \
                       static_cast<const T *>(a.x), static_cast<const T *>(a.w), static_cast<const T *>(a.bias),       \
                       static_cast<T *>(a.out), static_cast<T *>(a.act_in), a.M, n_out, a.K, a.x_rs, a.out_rs, a.out_cs, \
                       a.ai_rs, a.ai_cs, act, static_cast<const T *>(rms_w), eps, ex)
    if constexpr (kMaxWaves >= 16) {
        if (waves >= 16) { KERNL_SKINNY(16); return; }
    }
    if constexpr (kMaxWaves >= 8) {
        if (waves >= 8) { KERNL_SKINNY(8); return; }
    }
    KERNL_SKINNY(4);
#undef KERNL_SKINNY
}

template <typename T, bool GATED, bool W8 = false>
static void launch_skinny(const LinearArgs &a) {
    const int n_out = GATED ? a.N / 2 : a.N;
    const int mb = (a.M + 15) / 16;
    // every workgroup reads all of x (from L2), so more output columns per workgroup mean less of that traffic.
    // Gated and one-byte weights: with more than 16 rows of x and enough output columns to fill the chip twice over,
    // a workgroup takes 32 columns
    const bool two = n_out >= 8192 && mb >= 2;
    if constexpr (!W8 && !GATED) {
        // 16-bit plain weights, 8 rows of x or more (measured at 8..64 rows, 4096..32000 columns): as few 16-column
        // blocks per workgroup as put the whole grid on the chip at once, one workgroup per CU — 11008 columns in
        // blocks of 48 are 230 workgroups, where blocks of 32 leave 88 CUs with two workgroups and the rest with one;
        // grids that do not fit either way take 32 columns, 64 with more than 48 rows
        int nr = 1;
        if (a.M >= 8) {
            nr = (n_out + 16 * 256 - 1) / (16 * 256);
            if (nr > 4) nr = mb >= 4 ? 4 : 2;
        }
#define KERNL_SKINNY_NR(NRV)                                            \
    do {                                                                \
        if (mb <= 1) launch_skinny_blocks<T, GATED, 1, NRV, W8>(a);      \
        else if (mb <= 2) launch_skinny_blocks<T, GATED, 2, NRV, W8>(a); \
        else launch_skinny_blocks<T, GATED, 4, NRV, W8>(a);              \
    } while (0)
        if (nr == 1) KERNL_SKINNY_NR(1);
        else if (nr == 2) KERNL_SKINNY_NR(2);
        else if (nr == 3) KERNL_SKINNY_NR(3);
        else KERNL_SKINNY_NR(4);
#undef KERNL_SKINNY_NR
        return;
    }
    if constexpr (GATED && !W8) {
        // gated 16-bit weights, 8..32 rows of x: the same rule (measured: 11008 gate/value pairs against K = 4096 at
        // 32 rows 48 -> 34 us, 13824 against 5120 65 -> 56 us); more rows do not leave the LDS for 48 columns
        const int nr = (n_out + 16 * 256 - 1) / (16 * 256);
        if (a.M >= 8 && mb <= 2 && nr >= 3 && nr <= 4) {
            if (nr == 3) { if (mb <= 1) launch_skinny_blocks<T, GATED, 1, 3, W8>(a); else launch_skinny_blocks<T, GATED, 2, 3, W8>(a); }
            else { if (mb <= 1) launch_skinny_blocks<T, GATED, 1, 4, W8>(a); else launch_skinny_blocks<T, GATED, 2, 4, W8>(a); }
            return;
        }
    }
    if (mb <= 1) { if (two) launch_skinny_blocks<T, GATED, 1, 2, W8>(a); else launch_skinny_blocks<T, GATED, 1, 1, W8>(a); }
    else if (mb <= 2) { if (two) launch_skinny_blocks<T, GATED, 2, 2, W8>(a); else launch_skinny_blocks<T, GATED, 2, 1, W8>(a); }
    else { if (two) launch_skinny_blocks<T, GATED, 4, 2, W8>(a); else launch_skinny_blocks<T, GATED, 4, 1, W8>(a); }
}

// RMS-normalised input: 16 output columns per workgroup, 16-bit weights
template <typename T, bool GATED>
static void launch_skinny_rms(const LinearArgs &a, const void *rms_w, float eps) {
    const int mb = (a.M + 15) / 16;
    if (mb <= 1) launch_skinny_blocks<T, GATED, 1, 1, false, true>(a, rms_w, eps);
    else if (mb <= 2) launch_skinny_blocks<T, GATED, 2, 1, false, true>(a, rms_w, eps);
    else launch_skinny_blocks<T, GATED, 4, 1, false, true>(a, rms_w, eps);
}

// decoding-step projection with optional RMSNorm prologue, rotary epilogue and residual (plain 16-bit weights)
template <typename T>
static void launch_skinny_decode(const LinearArgs &a, const void *rms_w, float eps, const SkinnyExtra &ex) {
    const int mb = (a.M + 15) / 16;
    if (ex.half > 0) {  // rotating form: two column blocks per workgroup, always with the normalising prologue
        if (mb <= 1) launch_skinny_blocks<T, false, 1, 2, false, true, true>(a, rms_w, eps, &ex);
        else if (mb <= 2) launch_skinny_blocks<T, false, 2, 2, false, true, true>(a, rms_w, eps, &ex);
        else launch_skinny_blocks<T, false, 4, 2, false, true, true>(a, rms_w, eps, &ex);
    } else if (rms_w != nullptr) {
        if (mb <= 1) launch_skinny_blocks<T, false, 1, 1, false, true>(a, rms_w, eps, &ex);
        else if (mb <= 2) launch_skinny_blocks<T, false, 2, 1, false, true>(a, rms_w, eps, &ex);
        else launch_skinny_blocks<T, false, 4, 1, false, true>(a, rms_w, eps, &ex);
    } else {
        LinearArgs b = a;  // the plain kernel with its own grid rule; the residual travels in the arguments
        b.extra = &ex;
        launch_skinny<T, false>(b);
    }
}

}  // namespace kernl
