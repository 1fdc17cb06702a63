// LayerNorm / RMSNorm forward for gfx950, with an optional fused residual add.
//
// Memory-bound: the register-resident kernel reads every row from HBM exactly once (16-byte loads, one
// wave per row, the row stays in VGPRs between the statistics and the normalisation), reduces with DPP
// inside the wave, and writes 16-byte stores.  Semantics follow the reference kernel
// src/kernl/implementations/layer_norm.py:115-205: fp32 statistics, biased variance, rstd = 1/sqrt(var+eps),
// RMS branch keeps mean = 0 and uses mean(x^2).  The variance is the exact two-pass form Σ(x-mean)²/N on the
// register copy, which is at least as accurate as the reference's chunked Welford merge (:159-180).
#include "common.h"

namespace kernl {

template <typename T>
struct Row16 {  // one 16-byte chunk of a row
    static constexpr int kElems = 16 / sizeof(T);
    T v[kElems];
};

// A group of GROUP_WAVES waves (1 or the 4 of the block) per row; thread t of the group owns chunks t, t + G, ...
// (G = 64 GROUP_WAVES, CHUNKS of them at most).  A group walks rows with a fixed stride and fetches the next row
// before it reduces the current one, so that loads of one row overlap the arithmetic and the stores of another.
// HALF (single-wave groups only): a group is half a wave, so that a wave works on two rows at once — rows of 32·k
// chunks with odd k (768 fp16 values are 96 chunks) then keep every lane busy.
// FULL: the row is exactly CHUNKS chunks per thread of the group, so no chunk needs a bounds test, gamma / beta are
// converted to fp32 once per group instead of once per row, and a group whose row lies beyond M (the upper half of
// the last wave) computes on the last row again and skips the store — the per-element selects of the general form
// are gone.  BASELINE config 2 (768 fp16 values = 3 chunks per lane of a half wave) went from about 450 to about 250
// instructions per row pair: on such inputs the vector ALU work is of the order of the memory time.
template <typename T, int CHUNKS, bool RMS, bool HAS_RES, int GROUP_WAVES, bool HALF = false, bool FULL = false>
__global__ void __launch_bounds__(256)
layernorm_rows_kernel(const T *__restrict__ x, const T *__restrict__ res, const T *__restrict__ w,
                      const T *__restrict__ b, T *__restrict__ out, float *__restrict__ mean_out,
                      float *__restrict__ rstd_out, int M, int N, int64_t x_rs, int64_t res_rs,
                      int64_t out_rs, float eps, int stream_out) {
    constexpr int E = Row16<T>::kElems;
    static_assert(!HALF || GROUP_WAVES == 1, "half-wave groups are single-wave groups split in two");
    constexpr int G = HALF ? 32 : 64 * GROUP_WAVES;
    typedef Row16<T> chunk_t;
    __shared__ float red[2][4];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int t = HALF ? (lane & 31) : GROUP_WAVES == 1 ? lane : (int)threadIdx.x;  // index inside the group
    const int groups_per_block = HALF ? 8 : 4 / GROUP_WAVES;
    const int group = HALF ? 2 * wave + (lane >> 5) : GROUP_WAVES == 1 ? wave : 0;
    const int nchunks = N / E;
    const float inv_n = 1.0f / (float)N;

    // sum over the group: wave reduction, then (4-wave groups) a round trip through LDS
    auto group_sum = [&](float v, int slot) -> float {
        if (HALF) {
            float lo, hi;
            half_wave_sums(v, lo, hi);
            return lane < 32 ? lo : hi;
        }
        v = wave_sum(v);
        if (GROUP_WAVES == 1) return v;
        __syncthreads();  // the previous use of this slot has been read by everyone
        if (lane == 0) red[slot][wave] = v;
        __syncthreads();
        return (red[slot][0] + red[slot][1]) + (red[slot][2] + red[slot][3]);
    };

    // gamma / beta stay in registers (as 16-bit values; FULL: as fp32) for every row this group visits.
    chunk_t wv[CHUNKS], bv[CHUNKS];
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int ci = t + c * G;
        if (FULL || ci < nchunks) {
            wv[c] = *reinterpret_cast<const chunk_t *>(w + (int64_t)ci * E);
            if (b != nullptr) bv[c] = *reinterpret_cast<const chunk_t *>(b + (int64_t)ci * E);
        }
    }
    constexpr int CF = FULL ? CHUNKS : 1;
    float wf[CF][E], bf[CF][E];
    if (FULL) {
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
            for (int e = 0; e < E; ++e) {
                wf[c][e] = to_float(wv[c].v[e]);
                bf[c][e] = b != nullptr ? to_float(bv[c].v[e]) : 0.0f;
            }
    }

    const int row_step = gridDim.x * groups_per_block;
    int row = blockIdx.x * groups_per_block + group;
    chunk_t xn[CHUNKS], rn[HAS_RES ? CHUNKS : 1];
    auto fetch = [&](int r) {
        if (FULL) r = min(r, M - 1);  // a group beyond the last row reads the last row again (and stores nothing)
        const T *xr = x + (int64_t)r * x_rs;
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int ci = t + c * G;
            if (FULL || ci < nchunks) xn[c] = *reinterpret_cast<const chunk_t *>(xr + (int64_t)ci * E);
        }
        if (HAS_RES) {
            const T *rr = res + (int64_t)r * res_rs;
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c) {
                const int ci = t + c * G;
                if (FULL || ci < nchunks) rn[c] = *reinterpret_cast<const chunk_t *>(rr + (int64_t)ci * E);
            }
        }
    };
    if (FULL || row < M) fetch(row);

    // with half-wave groups the wave stays together while its lower half has a row; the upper half's last row may
    // lie beyond M, then it computes on zeros and stores nothing
    for (int lead = row - (HALF ? lane >> 5 : 0); lead < M; lead += row_step, row += row_step) {
        const bool live = !HALF || row < M;
        float v[CHUNKS][E];
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int ci = t + c * G;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                float a = 0.0f;
                if (FULL || (ci < nchunks && live)) {
                    a = to_float(xn[c].v[e]);
                    if (HAS_RES) a += to_float(rn[c].v[e]);
                }
                v[c][e] = a;
            }
        }
        if (FULL ? lead + row_step < M : row + row_step < M) fetch(row + row_step);

        float mean = 0.0f, var;
        if (RMS) {
            float ss = 0.0f;
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
                for (int e = 0; e < E; ++e) ss += v[c][e] * v[c][e];
            var = group_sum(ss, 0) * inv_n;
        } else {
            float s = 0.0f;
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
                for (int e = 0; e < E; ++e) s += v[c][e];
            mean = group_sum(s, 0) * inv_n;
            float ss = 0.0f;
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c) {
                const int ci = t + c * G;
                if (FULL || ci < nchunks) {
#pragma unroll
                    for (int e = 0; e < E; ++e) {
                        const float d = v[c][e] - mean;
                        ss += d * d;
                    }
                }
            }
            var = group_sum(ss, 1) * inv_n;
        }
        const float rstd = 1.0f / sqrtf(var + eps);
        if (t == 0 && live) {
            if (mean_out != nullptr) mean_out[row] = mean;
            if (rstd_out != nullptr) rstd_out[row] = rstd;
        }

        T *orow = out + (int64_t)row * out_rs;
        const float shift = -mean * rstd;  // (v - mean) * rstd = v * rstd + shift
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int ci = t + c * G;
            if (FULL ? live : (ci < nchunks && live)) {
                chunk_t o;
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    float y;
                    if (FULL) {
                        y = fmaf(fmaf(v[c][e], rstd, shift), wf[c][e], bf[c][e]);
                    } else {
                        y = (v[c][e] - mean) * rstd * to_float(wv[c].v[e]);
                        if (b != nullptr) y += to_float(bv[c].v[e]);
                    }
                    o.v[e] = from_float<T>(y);
                }
                // Outputs too large to stay cached until their consumer runs are written with streaming stores
                // (measured +15 % bandwidth here); smaller ones with plain stores, because the GEMM that follows
                // in a model then finds them in L2 / MALL (measured: streaming stores cost BERT-base 1 % end to end).
                if (stream_out)
                    __builtin_nontemporal_store(__builtin_bit_cast(u32x4, o), reinterpret_cast<u32x4 *>(orow + (int64_t)ci * E));
                else
                    *reinterpret_cast<chunk_t *>(orow + (int64_t)ci * E) = o;
            }
        }
    }
}

// Any strides, any N: one 256-thread block per row, three passes over the (cache-resident) row.
template <typename T, bool RMS, bool HAS_RES>
__global__ void __launch_bounds__(256)
layernorm_strided_kernel(const T *__restrict__ x, const T *__restrict__ res, const T *__restrict__ w,
                         const T *__restrict__ b, T *__restrict__ out, float *__restrict__ mean_out,
                         float *__restrict__ rstd_out, int M, int N, int64_t x_rs, int64_t x_cs,
                         int64_t res_rs, int64_t res_cs, int64_t out_rs, int64_t out_cs, float eps) {
    __shared__ float red[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float inv_n = 1.0f / (float)N;
    for (int row = blockIdx.x; row < M; row += gridDim.x) {
        const T *xr = x + (int64_t)row * x_rs;
        const T *rr = HAS_RES ? res + (int64_t)row * res_rs : nullptr;
        auto load = [&](int i) -> float {
            float a = to_float(xr[(int64_t)i * x_cs]);
            if (HAS_RES) a += to_float(rr[(int64_t)i * res_cs]);
            return a;
        };
        auto block_sum = [&](float s) -> float {
            s = wave_sum(s);
            __syncthreads();
            if (lane == 0) red[wave] = s;
            __syncthreads();
            return (red[0] + red[1]) + (red[2] + red[3]);
        };
        float mean = 0.0f;
        if (!RMS) {
            float s = 0.0f;
            for (int i = threadIdx.x; i < N; i += blockDim.x) s += load(i);
            mean = block_sum(s) * inv_n;
        }
        float ss = 0.0f;
        for (int i = threadIdx.x; i < N; i += blockDim.x) {
            const float d = load(i) - mean;
            ss += d * d;
        }
        const float var = block_sum(ss) * inv_n;
        const float rstd = 1.0f / sqrtf(var + eps);
        if (threadIdx.x == 0) {
            if (mean_out != nullptr) mean_out[row] = mean;
            if (rstd_out != nullptr) rstd_out[row] = rstd;
        }
        T *orow = out + (int64_t)row * out_rs;
        for (int i = threadIdx.x; i < N; i += blockDim.x) {
            float y = (load(i) - mean) * rstd * to_float(w[i]);
            if (b != nullptr) y += to_float(b[i]);
            orow[(int64_t)i * out_cs] = from_float<T>(y);
        }
    }
}

template <typename T, int CHUNKS, int GROUP_WAVES, bool HALF = false, bool FULL = false>
static void launch_rows(bool rms, bool has_res, dim3 grid, hipStream_t st, const T *x, const T *res,
                        const T *w, const T *b, T *out, float *mean, float *rstd, int M, int N, int64_t x_rs,
                        int64_t res_rs, int64_t out_rs, float eps) {
    // rows that fill every lane's chunks exactly take the form without bounds tests (single-wave groups of up to 4
    // chunks: gamma and beta are kept as fp32 there)
    if constexpr (!FULL && GROUP_WAVES == 1 && CHUNKS <= 4) {
        if (N == CHUNKS * (HALF ? 32 : 64) * (int)(16 / sizeof(T))) {
            launch_rows<T, CHUNKS, GROUP_WAVES, HALF, true>(rms, has_res, grid, st, x, res, w, b, out, mean, rstd, M, N, x_rs,
                                                            res_rs, out_rs, eps);
            return;
        }
    }
#define KERNL_LN_LAUNCH(R, H)                                                                                       \
    hipLaunchKernelGGL((layernorm_rows_kernel<T, CHUNKS, R, H, GROUP_WAVES, HALF, FULL>), grid, dim3(256), 0, st, x, res, w, b, \
                       out, mean, rstd, M, N, x_rs, res_rs, out_rs, eps, stream_out)
    const int stream_out = (int64_t)M * N * (int64_t)sizeof(T) > (128ll << 20);
    if (rms) {
        if (has_res) KERNL_LN_LAUNCH(true, true);
        else KERNL_LN_LAUNCH(true, false);
    } else {
        if (has_res) KERNL_LN_LAUNCH(false, true);
        else KERNL_LN_LAUNCH(false, false);
    }
#undef KERNL_LN_LAUNCH
}

template <typename T>
static int layernorm_dispatch(const void *x_, const void *res_, const void *w_, const void *b_, void *out_,
                              float *mean, float *rstd, int64_t M, int64_t N, int64_t x_rs, int64_t x_cs,
                              int64_t res_rs, int64_t res_cs, int64_t out_rs, int64_t out_cs, float eps,
                              bool rms, hipStream_t st) {
    const T *x = static_cast<const T *>(x_);
    const T *res = static_cast<const T *>(res_);
    const T *w = static_cast<const T *>(w_);
    const T *b = static_cast<const T *>(b_);
    T *out = static_cast<T *>(out_);
    const bool has_res = res != nullptr;
    constexpr int E = 16 / sizeof(T);
    const int64_t row_chunks = N / E;
    const bool vec_ok = (N % E == 0) && x_cs == 1 && out_cs == 1 && (!has_res || res_cs == 1) &&
                        (x_rs % E == 0) && (out_rs % E == 0) && (!has_res || res_rs % E == 0) &&
                        aligned16(x) && aligned16(out) && aligned16(w) && (b == nullptr || aligned16(b)) &&
                        (!has_res || aligned16(res)) && row_chunks <= 64 * 16;
    if (vec_ok) {
        // Rows of up to 1024 chunks stay in registers.  Long rows on few-row inputs are spread over the 4 waves of a
        // block (more loads in flight per row); otherwise a wave per row, 4 rows per block.  The grid is capped at
        // 8 waves per SIMD (4 where a wave takes two rows) so that every group walks several rows and gamma/beta loads
        // amortise.
        const bool block_per_row = row_chunks > 128 && M < 16384;
        // Two rows per wave, 32 lanes each, where that leaves fewer lanes idle than a wave per row (rows of up to 32
        // or of 65..96 chunks).
        const bool half_wave = !block_per_row && (row_chunks <= 32 || (row_chunks > 64 && row_chunks <= 96));
        const int64_t grid_cap = half_wave ? 1024 : 2048;
        const int64_t blocks_needed = block_per_row ? M : half_wave ? (M + 7) / 8 : (M + 3) / 4;
        const int grid = (int)(blocks_needed < grid_cap ? blocks_needed : grid_cap);
        const int chunks = (int)((row_chunks + (block_per_row ? 255 : 63)) / (block_per_row ? 256 : 64));
#define KERNL_LN_CASE(C, GW)                                                                                   \
    launch_rows<T, C, GW>(rms, has_res, dim3(grid), st, x, res, w, b, out, mean, rstd, (int)M, (int)N, x_rs, \
                          res_rs, out_rs, eps)
        if (half_wave) {
            if (row_chunks <= 32)
                launch_rows<T, 1, 1, true>(rms, has_res, dim3(grid), st, x, res, w, b, out, mean, rstd, (int)M, (int)N,
                                           x_rs, res_rs, out_rs, eps);
            else
                launch_rows<T, 3, 1, true>(rms, has_res, dim3(grid), st, x, res, w, b, out, mean, rstd, (int)M, (int)N,
                                           x_rs, res_rs, out_rs, eps);
        } else if (block_per_row) {
            if (chunks <= 1) KERNL_LN_CASE(1, 4);
            else if (chunks <= 2) KERNL_LN_CASE(2, 4);
            else KERNL_LN_CASE(4, 4);
        } else {
            if (chunks <= 1) KERNL_LN_CASE(1, 1);
            else if (chunks <= 2) KERNL_LN_CASE(2, 1);
            else if (chunks <= 4) KERNL_LN_CASE(4, 1);
            else if (chunks <= 8) KERNL_LN_CASE(8, 1);
            else KERNL_LN_CASE(16, 1);
        }
#undef KERNL_LN_CASE
    } else {
        const int grid = (int)(M < 65535 ? M : 65535);
#define KERNL_LN_LAUNCH(R, H)                                                                             \
    hipLaunchKernelGGL((layernorm_strided_kernel<T, R, H>), dim3(grid), dim3(256), 0, st, x, res, w, b, \
                       out, mean, rstd, (int)M, (int)N, x_rs, x_cs, res_rs, res_cs, out_rs, out_cs, eps)
        if (rms) {
            if (has_res) KERNL_LN_LAUNCH(true, true);
            else KERNL_LN_LAUNCH(true, false);
        } else {
            if (has_res) KERNL_LN_LAUNCH(false, true);
            else KERNL_LN_LAUNCH(false, false);
        }
#undef KERNL_LN_LAUNCH
    }
    return check_launch("layernorm");
}

// sum = a + b rounded to T (b may be NULL: then nothing is written), rstd[row] = 1 / sqrt(mean(sum^2) + eps) of the ROUNDED
// sum — what an RMSNorm applied to the stored tensor would compute.  One wave per row, 16-byte chunks.
template <typename T>
__global__ void __launch_bounds__(256) add_rms_stats_kernel(const T *__restrict__ a, const T *__restrict__ b, T *__restrict__ sum,
                                                            float *__restrict__ rstd, int M, int N, int64_t a_rs, int64_t b_rs,
                                                            int64_t sum_rs, float eps) {
    typedef typename Vec8<T>::type vec8;
    const int lane = threadIdx.x & 63, row = (int)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;
    const vec8 *ap = reinterpret_cast<const vec8 *>(a + (int64_t)row * a_rs);
    const vec8 *bp = b != nullptr ? reinterpret_cast<const vec8 *>(b + (int64_t)row * b_rs) : nullptr;
    vec8 *sp = b != nullptr ? reinterpret_cast<vec8 *>(sum + (int64_t)row * sum_rs) : nullptr;
    float sq = 0.0f;
    const int chunks = N / 8;
    auto take = [&](int c, vec8 v, vec8 w) __attribute__((always_inline)) {
        if (bp != nullptr) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = from_float<T>(to_float(v[e]) + to_float(w[e]));
            sp[c] = v;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float f = to_float(v[e]);
            sq = fmaf(f, f, sq);
        }
    };
    // four chunks of either operand in flight per lane (a 4096-wide row is two such rounds)
    int c = lane;
    for (; c + 192 < chunks; c += 256) {
        vec8 v[4], w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = ap[c + 64 * i];
        if (bp != nullptr) {
#pragma unroll
            for (int i = 0; i < 4; ++i) w[i] = bp[c + 64 * i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) take(c + 64 * i, v[i], w[i]);
    }
    for (; c < chunks; c += 64) take(c, ap[c], bp != nullptr ? bp[c] : vec8{});
    sq = wave_sum(sq);
    if (lane == 0) rstd[row] = rsqrtf(sq / (float)N + eps);
}

// Embedding lookups summed and normalised: out[m] = LayerNorm(round(round(t0[i0[m]] + t1[i1[m]]) + t2[i2[m]])) — the
// rows are added in the tensors' dtype, one addition after the other, as the eager model adds them.  One wave per output
// row, a lane keeps up to 4 chunks of 8 values (N <= 2048); an index outside its table is clamped into it.
struct EmbedTable {
    const void *table;   // [rows, N] contiguous, or null
    const int64_t *ids;  // entry (b, s) at b * ids_bs + s * ids_ss
    int64_t ids_bs, ids_ss, rows;
};
template <typename T>
__global__ void __launch_bounds__(256) embedding_layernorm_kernel(EmbedTable t0, EmbedTable t1, EmbedTable t2,
                                                                  const T *__restrict__ w, const T *__restrict__ b,
                                                                  T *__restrict__ out, int M, int S, int N, float eps) {
    typedef typename Vec8<T>::type vec8;
    const int lane = threadIdx.x & 63, row = (int)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= M) return;
    const int bi = row / S, si = row % S;
    auto row_of = [&](const EmbedTable &t) __attribute__((always_inline)) -> const vec8 * {
        int64_t id = t.ids[bi * t.ids_bs + si * t.ids_ss];
        id = id < 0 ? 0 : (id >= t.rows ? t.rows - 1 : id);
        return reinterpret_cast<const vec8 *>(static_cast<const T *>(t.table) + id * N);
    };
    const vec8 *r0 = row_of(t0);
    const vec8 *r1 = t1.table != nullptr ? row_of(t1) : nullptr;
    const vec8 *r2 = t2.table != nullptr ? row_of(t2) : nullptr;
    const int chunks = N / 8;
    float v[4][8];
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        const bool in = c < chunks;
        vec8 a = in ? r0[c] : vec8{};
        if (r1 != nullptr && in) {
            const vec8 o = r1[c];
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] = from_float<T>(to_float(a[e]) + to_float(o[e]));
        }
        if (r2 != nullptr && in) {
            const vec8 o = r2[c];
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] = from_float<T>(to_float(a[e]) + to_float(o[e]));
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            v[i][e] = to_float(a[e]);
            sum += v[i][e];
        }
    }
    const float mean = wave_sum(sum) / (float)N;
    float sq = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (lane + 64 * i < chunks) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float d = v[i][e] - mean;
                sq = fmaf(d, d, sq);
            }
        }
    }
    const float rstd = rsqrtf(wave_sum(sq) / (float)N + eps);
    vec8 *op = reinterpret_cast<vec8 *>(out + (int64_t)row * N);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int c = lane + 64 * i;
        if (c < chunks) {
            const vec8 g = reinterpret_cast<const vec8 *>(w)[c];
            const vec8 be = b != nullptr ? reinterpret_cast<const vec8 *>(b)[c] : vec8{};
            vec8 o;
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = from_float<T>(fmaf((v[i][e] - mean) * rstd, to_float(g[e]), b != nullptr ? to_float(be[e]) : 0.0f));
            op[c] = o;
        }
    }
}

static int layernorm_entry(const void *x, const void *res, const void *w, const void *b, void *out,
                           float *mean, float *rstd, int64_t M, int64_t N, int64_t x_rs, int64_t x_cs,
                           int64_t res_rs, int64_t res_cs, int64_t out_rs, int64_t out_cs, float eps,
                           int is_rms, int dtype, void *stream) {
    if (x == nullptr || w == nullptr || out == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "layernorm: x, w and out must not be NULL");
    if (M < 0 || N <= 0) return set_error(KERNL_ERR_INVALID_ARG, "layernorm: bad sizes M=%lld N=%lld",
                                          (long long)M, (long long)N);
    if (M > INT32_MAX || N > INT32_MAX)
        return set_error(KERNL_ERR_UNSUPPORTED, "layernorm: M and N must fit in 31 bits");
    if (M == 0) return KERNL_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case KERNL_F16:
            return layernorm_dispatch<f16>(x, res, w, b, out, mean, rstd, M, N, x_rs, x_cs, res_rs, res_cs,
                                           out_rs, out_cs, eps, is_rms != 0, st);
        case KERNL_BF16:
            return layernorm_dispatch<bf16>(x, res, w, b, out, mean, rstd, M, N, x_rs, x_cs, res_rs, res_cs,
                                            out_rs, out_cs, eps, is_rms != 0, st);
        case KERNL_F32:
            return layernorm_dispatch<float>(x, res, w, b, out, mean, rstd, M, N, x_rs, x_cs, res_rs,
                                             res_cs, out_rs, out_cs, eps, is_rms != 0, st);
        default:
            return set_error(KERNL_ERR_UNSUPPORTED, "layernorm: unknown dtype %d", dtype);
    }
}

}  // namespace kernl

extern "C" int kernl_layernorm_fwd(const void *x, const void *w, const void *bias, void *out, float *mean,
                                   float *rstd, int64_t M, int64_t N, int64_t x_row_stride,
                                   int64_t x_col_stride, int64_t out_row_stride, int64_t out_col_stride,
                                   float eps, int is_rms, int dtype, void *stream) {
    return kernl::layernorm_entry(x, nullptr, w, bias, out, mean, rstd, M, N, x_row_stride, x_col_stride,
                                  0, 0, out_row_stride, out_col_stride, eps, is_rms, dtype, stream);
}

extern "C" int kernl_add_layernorm_fwd(const void *x, const void *residual, const void *w, const void *bias,
                                       void *out, float *mean, float *rstd, int64_t M, int64_t N,
                                       int64_t x_row_stride, int64_t x_col_stride, int64_t res_row_stride,
                                       int64_t res_col_stride, int64_t out_row_stride,
                                       int64_t out_col_stride, float eps, int is_rms, int dtype,
                                       void *stream) {
    if (residual == nullptr)
        return kernl::set_error(KERNL_ERR_INVALID_ARG, "add_layernorm: residual must not be NULL");
    return kernl::layernorm_entry(x, residual, w, bias, out, mean, rstd, M, N, x_row_stride, x_col_stride,
                                  res_row_stride, res_col_stride, out_row_stride, out_col_stride, eps,
                                  is_rms, dtype, stream);
}

extern "C" int kernl_add_rms_stats_fwd(const void *a, const void *b, void *sum, float *rstd, int64_t M, int64_t N,
                                       int64_t a_row_stride, int64_t b_row_stride, int64_t sum_row_stride, float eps,
                                       int dtype, void *stream) {
    using namespace kernl;
    if (a == nullptr || rstd == nullptr) return set_error(KERNL_ERR_INVALID_ARG, "add_rms_stats: a and rstd must not be NULL");
    if (b != nullptr && sum == nullptr) return set_error(KERNL_ERR_INVALID_ARG, "add_rms_stats: b given without sum");
    if (M < 0 || N <= 0) return set_error(KERNL_ERR_INVALID_ARG, "add_rms_stats: bad sizes M=%lld N=%lld", (long long)M, (long long)N);
    if (dtype != KERNL_F16 && dtype != KERNL_BF16)
        return set_error(KERNL_ERR_UNSUPPORTED, "add_rms_stats: only f16 and bf16 are supported, got dtype %d", dtype);
    if (N % 8 != 0 || N > (1 << 20) || M > INT32_MAX - 4 || !aligned16(a) || a_row_stride % 8 != 0 ||
        (b != nullptr && (!aligned16(b) || !aligned16(sum) || b_row_stride % 8 != 0 || sum_row_stride % 8 != 0)))
        return set_error(KERNL_ERR_UNSUPPORTED, "add_rms_stats: rows must be contiguous, 16-byte aligned and a multiple of 8 "
                         "elements long");
    if (M == 0) return KERNL_OK;
    const dim3 grid((unsigned)((M + 3) / 4)), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == KERNL_F16)
        hipLaunchKernelGGL((add_rms_stats_kernel<f16>), grid, block, 0, st, static_cast<const f16 *>(a), static_cast<const f16 *>(b),
                           static_cast<f16 *>(sum), rstd, (int)M, (int)N, a_row_stride, b_row_stride, sum_row_stride, eps);
    else
        hipLaunchKernelGGL((add_rms_stats_kernel<bf16>), grid, block, 0, st, static_cast<const bf16 *>(a), static_cast<const bf16 *>(b),
                           static_cast<bf16 *>(sum), rstd, (int)M, (int)N, a_row_stride, b_row_stride, sum_row_stride, eps);
    return check_launch("add_rms_stats");
}

extern "C" int kernl_embedding_layernorm_fwd(const void *table0, const int64_t *ids0, int64_t ids0_batch_stride,
                                             int64_t ids0_seq_stride, int64_t rows0, const void *table1, const int64_t *ids1,
                                             int64_t ids1_batch_stride, int64_t ids1_seq_stride, int64_t rows1,
                                             const void *table2, const int64_t *ids2, int64_t ids2_batch_stride,
                                             int64_t ids2_seq_stride, int64_t rows2, const void *w, const void *bias, void *out,
                                             int64_t batch, int64_t seq, int64_t N, float eps, int dtype, void *stream) {
    using namespace kernl;
    if (table0 == nullptr || ids0 == nullptr || w == nullptr || out == nullptr || (table1 != nullptr && ids1 == nullptr) ||
        (table2 != nullptr && ids2 == nullptr))
        return set_error(KERNL_ERR_INVALID_ARG, "embedding + layernorm: table0, its ids, w and out must not be NULL, and every table needs ids");
    if (table1 == nullptr && table2 != nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "embedding + layernorm: tables are given in order (table2 without table1)");
    if (batch < 0 || seq < 0 || N <= 0 || rows0 <= 0 || (table1 != nullptr && rows1 <= 0) || (table2 != nullptr && rows2 <= 0))
        return set_error(KERNL_ERR_INVALID_ARG, "embedding + layernorm: bad sizes batch=%lld seq=%lld N=%lld", (long long)batch,
                         (long long)seq, (long long)N);
    if (dtype != KERNL_F16 && dtype != KERNL_BF16)
        return set_error(KERNL_ERR_UNSUPPORTED, "embedding + layernorm: only f16 and bf16 are supported, got dtype %d", dtype);
    if (N % 8 != 0 || N > 2048 || batch * seq > INT32_MAX || !aligned16(table0) || !aligned16(out) || !aligned16(w) ||
        (bias != nullptr && !aligned16(bias)) || (table1 != nullptr && !aligned16(table1)) || (table2 != nullptr && !aligned16(table2)))
        return set_error(KERNL_ERR_UNSUPPORTED, "embedding + layernorm: N must be a multiple of 8 and at most 2048, tables, w, bias "
                         "and out 16-byte aligned and contiguous");
    if (batch == 0 || seq == 0) return KERNL_OK;
    const EmbedTable t0 = {table0, ids0, ids0_batch_stride, ids0_seq_stride, rows0};
    const EmbedTable t1 = {table1, ids1, ids1_batch_stride, ids1_seq_stride, rows1};
    const EmbedTable t2 = {table2, ids2, ids2_batch_stride, ids2_seq_stride, rows2};
    const int M = (int)(batch * seq);
    const dim3 grid((unsigned)((M + 3) / 4)), block(256);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == KERNL_F16)
        hipLaunchKernelGGL((embedding_layernorm_kernel<f16>), grid, block, 0, st, t0, t1, t2, static_cast<const f16 *>(w),
                           static_cast<const f16 *>(bias), static_cast<f16 *>(out), M, (int)seq, (int)N, eps);
    else
        hipLaunchKernelGGL((embedding_layernorm_kernel<bf16>), grid, block, 0, st, t0, t1, t2, static_cast<const bf16 *>(w),
                           static_cast<const bf16 *>(bias), static_cast<bf16 *>(out), M, (int)seq, (int)N, eps);
    return check_launch("embedding + layernorm");
}
