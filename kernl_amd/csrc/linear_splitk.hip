// Linear layer for a FEW rows of x (at most 128: batched decoding steps, pooled outputs), as a stream-K product.
//
//     out[M,N] = act(x[M,K] · w[N,K]ᵀ + bias[N]) (+ residual[M,N])
// and the forms a batched decoding step of a Llama-style layer needs around it, as the one-to-64-row kernel of
// linear.hip has them (`linear_skinny_kernel`): RMSNorm of x on the way in, the gated linear unit on interleaved
// weights, rotary embedding of the leading columns, residual — all but the norm's scaling of x in the epilogue.
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
static constexpr int kFewRowTile = 16 * kFewRowWaves;      // weight rows (output columns) per tile
static constexpr int kFewRowMaxGrid = 256;                 // one workgroup per CU

enum FewRowMode { kFewRowPlain = 0, kFewRowGated = 1, kFewRowRope = 2 };

struct FewRowArgs {
    const void *x, *w, *bias, *residual, *rms_w, *cos, *sin;
    void *out;
    float *part;      // partial tiles: slot s at s * tile elements
    float *sqpart;    // sums of squares of the x rows, per workgroup that touched tile 0: [grid][128]
    int M, N, K;      // N: rows of the weight (gated: twice the output width)
    int64_t ldx, out_rs, out_cs, res_rs, res_cs, t_bs, t_ss;
    int act, tiles, nch, run, direct;
    float eps;
    int table_dtype, half, rope_cols, rows_per_batch;
};

struct FewRowPlan {
    int tiles;        // column tiles
    int nch;          // chunks of 64 k per tile
    int run;          // units per workgroup
    int grid;         // workgroups
    bool direct;      // every run is exactly one tile: no partial sums
    int64_t partial_bytes, sq_bytes;
};

static constexpr int kFewRowMaxRows = 128;
static inline int fewrow_row_blocks(int64_t M) { return M <= 16 ? 1 : M <= 32 ? 2 : M <= 64 ? 4 : 8; }

// N: rows of the weight.  `paired`: the epilogue combines two columns of a tile (gate and value, or the two members of
// a rotation pair), which only the second kernel does.
static FewRowPlan fewrow_plan(int64_t M, int64_t N, int64_t K, bool paired) {
    FewRowPlan p;
    p.nch = (int)(K / 64);
    p.tiles = (int)((N + kFewRowTile - 1) / kFewRowTile);
    const int64_t total = (int64_t)p.tiles * p.nch;
    int64_t run = (total + kFewRowMaxGrid - 1) / kFewRowMaxGrid;
    if (run < 4) run = 4;
    // whole tiles per workgroup where that costs at most a fifth of the CUs: no partial sums, one launch
    if (!paired && p.tiles <= kFewRowMaxGrid && p.tiles * 5 >= kFewRowMaxGrid * 4) run = p.nch;
    p.run = (int)run;
    p.grid = (int)((total + run - 1) / run);
    p.direct = !paired && p.run == p.nch;
    p.partial_bytes = p.direct ? 0 : (int64_t)(p.grid + p.tiles) * kFewRowTile * 16 * fewrow_row_blocks(M) * 4;
    p.sq_bytes = p.direct ? 0 : (int64_t)p.grid * kFewRowMaxRows * 4;
    return p;
}

// Bias, activation, residual and store for elements e = 0..3 of `v`: output columns n .. n + 3 of x row m.
template <typename T>
__device__ __forceinline__ void fewrow_store(const float (&v)[4], int m, int n, T *__restrict__ out, int n_out,
                                             int64_t out_rs, int64_t out_cs, const T *__restrict__ residual,
                                             int64_t res_rs, int64_t res_cs) {
    float y[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        y[e] = v[e];
        if (residual != nullptr && n + e < n_out) y[e] += to_float(residual[(int64_t)m * res_rs + (int64_t)(n + e) * res_cs]);
    }
    if (out_cs == 1 && (out_rs & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0 && n + 3 < n_out) {
        uint2 p;
        p.x = pack2<T>(y[0], y[1]);
        p.y = pack2<T>(y[2], y[3]);
        *reinterpret_cast<uint2 *>(out + (int64_t)m * out_rs + n) = p;
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (n + e < n_out) out[(int64_t)m * out_rs + (int64_t)(n + e) * out_cs] = from_float<T>(y[e]);
    }
}

// Plain epilogue of one 16 x 16 block of one lane: elements e = 0..3 of `acc` are output columns n .. n + 3 of x row m;
// rstd is the row's inverse root mean square (1 without the norm).
template <typename T>
__device__ __forceinline__ void fewrow_epilogue(const f32x4_acc &acc, float rstd, int m, int n, const FewRowArgs &a) {
    if (n >= a.N || m >= a.M) return;
    const T *bias = static_cast<const T *>(a.bias);
    float y[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float b = bias != nullptr ? to_float(bias[min(n + e, a.N - 1)]) : 0.0f;
        y[e] = apply_act16(acc[e] * rstd + b, a.act);
    }
    fewrow_store<T>(y, m, n, static_cast<T *>(a.out), a.N, a.out_rs, a.out_cs, static_cast<const T *>(a.residual), a.res_rs,
                    a.res_cs);
}

// W8: the weight is stored as one byte per element, fp8 e5m2 — the upper byte of the fp16 encoding (as in the other
// linear kernels' W8 forms): a lane's 16 weights of a unit are one 16-byte load, byte-permuted into its two fragments.
template <typename T, int MB, int WAVES, int GC, int RING, bool RMS, bool W8 = false>
__global__ void __launch_bounds__(64 * WAVES) linear_fewrow_kernel(const FewRowArgs a) {
    typedef typename Vec8<T>::type vec8;
    static_assert(RING % (2 * GC) == 0, "a round of RING units is a whole number of stage pairs");
    constexpr int THREADS = 64 * WAVES;
    typedef FewRowStageMap<MB, GC, THREADS> StageMap;   // index_math.h: shared with the host-side replay
    constexpr int MP = StageMap::MP;                    // rows of x, padded to whole MFMA blocks
    constexpr int CHUNK_BYTES = StageMap::CHUNK_BYTES;  // one staged chunk of x
    constexpr int XP = StageMap::XP;                    // 16-byte pieces of a group of x per thread
    constexpr int RPT = MP * 8 > THREADS ? MP * 8 / THREADS : 1;   // rows of x a thread stages pieces of
    static_assert(2 * GC * CHUNK_BYTES >= RPT * THREADS * 4, "the stages double as the buffer of the row sums");
    __shared__ __attribute__((aligned(16))) unsigned char xs[2][GC * CHUNK_BYTES];
    __shared__ float rstd_s[MP];

    static_assert(!W8 || std::is_same<T, f16>::value, "one-byte weights are decoded to fp16");
    typedef typename std::conditional<W8, unsigned char, T>::type WT;   // what a weight element is stored as
    const T *X = static_cast<const T *>(a.x);
    const WT *W = static_cast<const WT *>(a.w);
    const int M = a.M, N = a.N, K = a.K, tiles = a.tiles, run = a.run, direct = a.direct;
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
    vec8 wf[W8 ? 1 : RING][2];
    u32x4 wraw[W8 ? RING : 1];
    int rq_left = n_units - 1;                  // units the cursor may still advance by
    int rq_tile = first_tile, rq_chunk = first_chunk;
    auto weight_row = [&](int tile) __attribute__((always_inline)) -> const WT * {
        return W + (int64_t)min(tile * (16 * WAVES) + 16 * wave + r, N - 1) * K + 16 * g;
    };
    const WT *wrow = weight_row(rq_tile);
    auto request_w = [&](int slot) __attribute__((always_inline)) {
        const WT *src = wrow + (int64_t)rq_chunk * 64;
        if constexpr (W8) {
            wraw[slot] = *reinterpret_cast<const u32x4 *>(src);
        } else {
            wf[slot][0] = *reinterpret_cast<const vec8 *>(src);
            wf[slot][1] = *reinterpret_cast<const vec8 *>(src + 8);
        }
        if (rq_left > 0) {      // uniform; address arithmetic only
            --rq_left;
            if (++rq_chunk == nch) {
                rq_chunk = 0;
                wrow = weight_row(++rq_tile);
            }
        }
    };

    // ---- x: piece i of a thread is 16-byte piece (q & 7) of row (q >> 3) % MP of the group's unit q / (8 MP),
    // q = tid + THREADS i — row slot i % RPT of the thread (one row, or two with 128 rows of x).  Rows beyond M repeat
    // the last row; units past the end of the
    // run repeat its last unit.  RMS: the norm's weight travels with x, a piece is multiplied by it (one rounding to
    // 16 bits, as in the reference) on its way into LDS, and the thread adds up the squares of the unscaled values of
    // the units that count: those of tile 0, whose runs cover every chunk of K exactly once (with whole tiles per
    // workgroup: all of its own).
    vec8 xr[XP], gr[RMS ? XP : 1];
    const T *xrow[XP];
    int xunit[XP], xdst[XP];
    float sq[RPT];
#pragma unroll
    for (int t = 0; t < RPT; ++t) sq[t] = 0.0f;
#pragma unroll
    for (int i = 0; i < XP; ++i) {
        xrow[i] = X + (int64_t)min(StageMap::piece_row(tid, i), M - 1) * a.ldx + StageMap::piece_index(tid) * 8;
        xunit[i] = __builtin_amdgcn_readfirstlane(StageMap::piece_unit(tid, i));   // a wave's 64 pieces belong to one unit
        xdst[i] = StageMap::piece_dst(tid, i);
    }
    const T *grow = static_cast<const T *>(a.rms_w) + (tid & 7) * 8;
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
            if constexpr (RMS) gr[i] = *reinterpret_cast<const vec8 *>(grow + (int64_t)c * 64);
        }
        xg_unit += GC;
        xg_chunk += GC;
        xg_chunk = xg_chunk >= nch ? xg_chunk - nch : xg_chunk;
    };
    // stages the group requested last (its first unit is xg_unit - GC)
    auto stage_x = [&](int stage) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < XP; ++i) {
            if constexpr (RMS) {
                const int u = xg_unit - GC + xunit[i];
                if (u < n_units && (direct || u_begin + u < nch)) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float xv = to_float(xr[i][e]);
                        sq[i % RPT] = fmaf(xv, xv, sq[i % RPT]);
                    }
                }
                xr[i] = xr[i] * gr[i];
            }
            *reinterpret_cast<vec8 *>(xs[stage] + xdst[i]) = xr[i];
        }
    };
    int xoff[MB][2];   // this lane's operand fragments inside a staged chunk
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int s = 0; s < 2; ++s) xoff[mb][s] = StageMap::frag_offset(mb, r, g, s);

    f32x4_acc acc[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb] = f32x4_acc{0.0f, 0.0f, 0.0f, 0.0f};

    // ---- consumer: unit i of the run is chunk `c_chunk` of tile `c_tile`
    int c_tile = first_tile, c_chunk = first_chunk;
    // Partial tile of this workgroup for tile `tile`: slot blockIdx + tile.  The stores are issued from assembly: a
    // store the compiler knows of, inside a branch of the loop, makes it wait for EVERY outstanding load at the next
    // use of a fragment (loads and stores share one counter that it then treats as unordered).
    auto flush_partial = [&](int tile) __attribute__((always_inline)) {
        float4 *dst = reinterpret_cast<float4 *>(a.part) + (((int64_t)blockIdx.x + tile) * (WAVES * MB) + wave * MB) * 64 + lane;
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
            vec8 w0, w1;
            if constexpr (W8) {
                const u32x4 raw = wraw[slot];
                u32x4 lo, hi;  // bytes {0, b0, 0, b1} / {0, b2, 0, b3} of every word: fp16 pairs
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    lo[2 * jj] = __builtin_amdgcn_perm(0u, raw[jj], 0x010c000cu);
                    lo[2 * jj + 1] = __builtin_amdgcn_perm(0u, raw[jj], 0x030c020cu);
                    hi[2 * jj] = __builtin_amdgcn_perm(0u, raw[2 + jj], 0x010c000cu);
                    hi[2 * jj + 1] = __builtin_amdgcn_perm(0u, raw[2 + jj], 0x030c020cu);
                }
                w0 = __builtin_bit_cast(vec8, lo);
                w1 = __builtin_bit_cast(vec8, hi);
            } else {
                w0 = wf[slot][0];
                w1 = wf[slot][1];
            }
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) {
                const vec8 x0 = *reinterpret_cast<const vec8 *>(chunk + xoff[mb][0]);
                const vec8 x1 = *reinterpret_cast<const vec8 *>(chunk + xoff[mb][1]);
                acc[mb] = mfma16(w0, x0, acc[mb]);
                acc[mb] = mfma16(w1, x1, acc[mb]);
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
    // ... and the last round, which requests no weights
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

    if constexpr (RMS) {
        // a row's squares are spread over the pieces q = (row + MP k) * 8 + p, p = 0..7 (q = tid + THREADS slot)
        __syncthreads();                        // every wave is done with the stages
        float *sqbuf = reinterpret_cast<float *>(&xs[0][0]);
#pragma unroll
        for (int t = 0; t < RPT; ++t) sqbuf[t * THREADS + tid] = sq[t];
        __syncthreads();
        if (tid < MP) {
            float t = 0.0f;
#pragma unroll
            for (int k = 0; k < RPT * THREADS / (8 * MP); ++k)
#pragma unroll
                for (int pp = 0; pp < 8; ++pp) t += sqbuf[(tid + MP * k) * 8 + pp];
            if (direct) rstd_s[tid] = 1.0f / sqrtf(t / (float)K + a.eps);
            else if (u_begin < nch) a.sqpart[(int64_t)blockIdx.x * kFewRowMaxRows + tid] = t;
        }
        if (direct) __syncthreads();
    }
    if (!direct) return;
    // a run of exactly one tile: element e of a lane is output column n + e of x row 16 mb + r
    const int n = first_tile * (16 * WAVES) + 16 * wave + 4 * g;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) fewrow_epilogue<T>(acc[mb], RMS ? rstd_s[16 * mb + r] : 1.0f, 16 * mb + r, n, a);
}

// Adds the partial tiles of every tile in workgroup order and runs the epilogue.  One thread per 16-byte element of a
// tile (the same lane-to-element map as above).  Tile t holds units [t nch, (t + 1) nch), i.e. it was touched by
// workgroups (t nch) / run .. ((t + 1) nch - 1) / run, and workgroup w left its share in slot w + t.
//   gated   the weight's rows alternate in blocks of 32 between gate and value (waves 0, 1, 4, 5 hold gates, the waves
//           two further on the values of the same outputs): out = act(gate + bias) * (value + bias), half as wide
//   rope    inside a head of 2 * half columns, column d pairs with d + half (`half / 16` waves further on); the pair is
//           rotated by the row's table entries when it lies below rope_cols; the tile width is a multiple of the head size
template <typename T, int MB, int WAVES, int MODE>
__global__ void __launch_bounds__(256) linear_fewrow_reduce_kernel(const FewRowArgs a) {
    constexpr int TILE_ELEMS = WAVES * MB * 64;                      // 16-byte elements of one partial tile
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)a.tiles * TILE_ELEMS) return;
    const int tile = (int)(idx / TILE_ELEMS), e0 = (int)(idx - (int64_t)tile * TILE_ELEMS);
    const int lane = e0 & 63, mb = (e0 >> 6) % MB, wave = (e0 >> 6) / MB;
    const int pair_waves = MODE == kFewRowGated ? 2 : MODE == kFewRowRope ? a.half / 16 : 0;
    if (MODE == kFewRowGated && (wave & 2)) return;                  // value blocks: their gate's thread takes them
    if (MODE == kFewRowRope && ((16 * wave) % (2 * a.half)) >= a.half) return;
    const int m = 16 * mb + (lane & 15);
    const int n = tile * (16 * WAVES) + 16 * wave + 4 * (lane >> 4);  // row of the weight (first of four)
    if (m >= a.M || n >= a.N) return;
    const int nch = a.nch, run = a.run;
    const int w_first = (tile * nch) / run, w_last = ((tile + 1) * nch - 1) / run;   // units fit 31 bits
    const int n_slots = w_last - w_first + 1;
    const float4 *theirs = reinterpret_cast<const float4 *>(a.part) + ((int64_t)w_first + tile) * TILE_ELEMS + e0;
    // Every load of this thread is requested before the first one is used: the kernel is a chain of memory round trips
    // otherwise (partial tiles, the norm's row sums, tables), and it is all latency.
    const float4 *partner = theirs + pair_waves * MB * 64;
    f32x4_acc acc = {0.0f, 0.0f, 0.0f, 0.0f}, other = {0.0f, 0.0f, 0.0f, 0.0f};
    float4 pv[4], qv[4];
    const int first = min(n_slots, 4);
#pragma unroll
    for (int u = 0; u < 4; ++u) {   // (slots past the last one fetch it again: no branch around a load)
        const int64_t slot = (int64_t)min(u, n_slots - 1) * TILE_ELEMS;
        pv[u] = theirs[slot];
        if (MODE != kFewRowPlain) qv[u] = partner[slot];
    }
    float sq_sum = 0.0f;
    if (a.rms_w != nullptr) {
        const int w_sq_last = (nch - 1) / run;
        for (int w = 0; w <= w_sq_last; ++w) sq_sum += a.sqpart[(int64_t)w * kFewRowMaxRows + m];
    }
    const bool rotate = MODE == kFewRowRope && n < a.rope_cols;   // rope_cols is a multiple of the head size, n of 4
    float tc[2][4], ts[2][4];   // cos / sin of the four columns and of their partners
    if (MODE == kFewRowRope && rotate) {
        const int d = n % (2 * a.half);
        const int64_t trow = (int64_t)(m / a.rows_per_batch) * a.t_bs + (int64_t)(m % a.rows_per_batch) * a.t_ss + d;
        const bool vec = ((a.t_bs | a.t_ss) & 3) == 0 && ((reinterpret_cast<uintptr_t>(a.cos) | reinterpret_cast<uintptr_t>(a.sin)) & 15) == 0;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int64_t off = trow + h * a.half;
            if (vec && a.table_dtype == KERNL_F32) {
                const float4 c = *reinterpret_cast<const float4 *>(static_cast<const float *>(a.cos) + off);
                const float4 sn = *reinterpret_cast<const float4 *>(static_cast<const float *>(a.sin) + off);
                tc[h][0] = c.x; tc[h][1] = c.y; tc[h][2] = c.z; tc[h][3] = c.w;
                ts[h][0] = sn.x; ts[h][1] = sn.y; ts[h][2] = sn.z; ts[h][3] = sn.w;
            } else if (vec && a.table_dtype == KERNL_F16) {
                const f16x4 c = *reinterpret_cast<const f16x4 *>(static_cast<const f16 *>(a.cos) + off);
                const f16x4 sn = *reinterpret_cast<const f16x4 *>(static_cast<const f16 *>(a.sin) + off);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    tc[h][e] = (float)c[e];
                    ts[h][e] = (float)sn[e];
                }
            } else if (vec && a.table_dtype == KERNL_BF16) {
                const bf16x4 c = *reinterpret_cast<const bf16x4 *>(static_cast<const bf16 *>(a.cos) + off);
                const bf16x4 sn = *reinterpret_cast<const bf16x4 *>(static_cast<const bf16 *>(a.sin) + off);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    tc[h][e] = (float)c[e];
                    ts[h][e] = (float)sn[e];
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    tc[h][e] = table_value(a.cos, a.table_dtype, off + e);
                    ts[h][e] = table_value(a.sin, a.table_dtype, off + e);
                }
            }
        }
    }
    // add in workgroup order: the slots requested above, then any further ones four at a time
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        if (u < first) {
            acc[0] += pv[u].x; acc[1] += pv[u].y; acc[2] += pv[u].z; acc[3] += pv[u].w;
            if (MODE != kFewRowPlain) {
                other[0] += qv[u].x; other[1] += qv[u].y; other[2] += qv[u].z; other[3] += qv[u].w;
            }
        }
    }
    for (int s = 4; s < n_slots; ++s) {
        const float4 v = theirs[(int64_t)s * TILE_ELEMS];
        acc[0] += v.x; acc[1] += v.y; acc[2] += v.z; acc[3] += v.w;
        if (MODE != kFewRowPlain) {
            const float4 o = partner[(int64_t)s * TILE_ELEMS];
            other[0] += o.x; other[1] += o.y; other[2] += o.z; other[3] += o.w;
        }
    }
    const float rstd = a.rms_w != nullptr ? 1.0f / sqrtf(sq_sum / (float)a.K + a.eps) : 1.0f;
    if (MODE == kFewRowPlain) {
        fewrow_epilogue<T>(acc, rstd, m, n, a);
        return;
    }
    const T *bias = static_cast<const T *>(a.bias);
    T *out = static_cast<T *>(a.out);
    const T *residual = static_cast<const T *>(a.residual);
    if (MODE == kFewRowGated) {
        // weight rows n .. n + 3 are gates of output columns (n / 64) * 32 + n % 32 ..; their values sit 32 rows on
        const int n_out = (n >> 6) * 32 + (n & 31);
        float y[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float bg = bias != nullptr ? to_float(bias[min(n + e, a.N - 1)]) : 0.0f;
            const float bv = bias != nullptr ? to_float(bias[min(n + e + 32, a.N - 1)]) : 0.0f;
            y[e] = apply_act16(acc[e] * rstd + bg, a.act) * (other[e] * rstd + bv);
        }
        fewrow_store<T>(y, m, n_out, out, a.N / 2, a.out_rs, a.out_cs, residual, a.res_rs, a.res_cs);
        return;
    }
    // rope: columns n .. n + 3 and their partners `half` further on
    float lo[4], hi[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float v0 = acc[e] * rstd, v1 = other[e] * rstd;
        if (bias != nullptr) {
            v0 += to_float(bias[min(n + e, a.N - 1)]);
            v1 += to_float(bias[min(n + e + a.half, a.N - 1)]);
        }
        lo[e] = rotate ? v0 * tc[0][e] - v1 * ts[0][e] : v0;
        hi[e] = rotate ? v1 * tc[1][e] + v0 * ts[1][e] : v1;
    }
    fewrow_store<T>(lo, m, n, out, a.N, a.out_rs, a.out_cs, residual, a.res_rs, a.res_cs);
    fewrow_store<T>(hi, m, n + a.half, out, a.N, a.out_rs, a.out_cs, residual, a.res_rs, a.res_cs);
}

template <typename T, bool W8 = false>
static void launch_fewrow(FewRowArgs a, const FewRowPlan &p, int mode, hipStream_t st) {
    const int mb = fewrow_row_blocks(a.M);
    const dim3 grid((unsigned)p.grid), block(64 * kFewRowWaves);
    const dim3 rgrid((unsigned)(((int64_t)p.tiles * kFewRowWaves * mb * 64 + 255) / 256));
    const bool rms = a.rms_w != nullptr;
    // x groups of 2 units and a ring of 4 measured best (by 0.5 to 1.4 us against 4 and 8); 16 rows of x are too few
    // pieces for 512 threads to stage 2 units at a time
#define KERNL_FEWROW_MAIN(MBV, RMSV)                                                                                   \
    hipLaunchKernelGGL((linear_fewrow_kernel<T, MBV, kFewRowWaves, (MBV == 1 ? 4 : 2), (MBV == 1 ? 8 : 4), RMSV, W8>), \
                       grid, block, 0, st, a)
#define KERNL_FEWROW_REDUCE(MBV, MODEV)                                                                                \
    hipLaunchKernelGGL((linear_fewrow_reduce_kernel<T, MBV, kFewRowWaves, MODEV>), rgrid, dim3(256), 0, st, a)
#define KERNL_FEWROW(MBV)                                                                                              \
    do {                                                                                                               \
        if (rms) KERNL_FEWROW_MAIN(MBV, true);                                                                         \
        else KERNL_FEWROW_MAIN(MBV, false);                                                                            \
        if (!p.direct) {                                                                                               \
            if (mode == kFewRowGated) KERNL_FEWROW_REDUCE(MBV, kFewRowGated);                                          \
            else if (mode == kFewRowRope) KERNL_FEWROW_REDUCE(MBV, kFewRowRope);                                       \
            else KERNL_FEWROW_REDUCE(MBV, kFewRowPlain);                                                               \
        }                                                                                                              \
    } while (0)
    if (mb == 1) KERNL_FEWROW(1);
    else if (mb == 2) KERNL_FEWROW(2);
    else if (mb == 4) KERNL_FEWROW(4);
    else KERNL_FEWROW(8);
#undef KERNL_FEWROW
#undef KERNL_FEWROW_REDUCE
#undef KERNL_FEWROW_MAIN
}

}  // namespace kernl

extern "C" int64_t kernl_linear_fewrow_workspace_bytes(int64_t M, int64_t N, int64_t K, int gated, int rotated) {
    using namespace kernl;
    if (M <= 0 || M > kFewRowMaxRows || N <= 0 || K < 256 || K % 64 != 0) return 0;
    const FewRowPlan p = fewrow_plan(M, gated ? 2 * N : N, K, gated || rotated);
    return p.partial_bytes + p.sq_bytes;
}

namespace kernl {
static int fewrow_entry(const void *x, const void *rms_weight, float eps, const void *w, const void *bias,
                        const void *residual, void *out, void *workspace, int64_t workspace_bytes, int64_t M, int64_t N,
                        int64_t K, const int64_t x_strides[2], const int64_t out_strides[2],
                        const int64_t residual_strides[2], const void *cos, const void *sin, int64_t head_dim,
                        int64_t rope_cols, int64_t rows_per_batch, const int64_t table_strides[3], int table_dtype,
                        int activation, int gated, int dtype, void *stream, bool w8) {
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
    if (M > kFewRowMaxRows || K % 64 != 0 || K < 256 || N > (1 << 29) || K > INT32_MAX)
        return set_error(KERNL_ERR_UNSUPPORTED, "few-row linear: at most 128 rows of x and K a multiple of 64, at least 256 "
                         "(M=%lld K=%lld)", (long long)M, (long long)K);
    if (x_strides[1] != 1 || x_strides[0] % 8 != 0 || !aligned16(x) || !aligned16(w) ||
        (rms_weight != nullptr && !aligned16(rms_weight)))
        return set_error(KERNL_ERR_UNSUPPORTED, "few-row linear: x needs unit feature stride and 16-byte aligned rows, the "
                         "weights 16-byte aligned bases");
    if (workspace != nullptr && (reinterpret_cast<uintptr_t>(workspace) & 15) != 0)
        return set_error(KERNL_ERR_UNSUPPORTED, "few-row linear: the workspace must be 16-byte aligned");
    const bool rope = cos != nullptr || sin != nullptr;
    if (gated && (rope || N % 32 != 0))
        return set_error(KERNL_ERR_UNSUPPORTED, "few-row linear: the gated form takes no rotation and needs an output width "
                         "that is a multiple of 32 (the interleaving block), got %lld", (long long)N);
    FewRowArgs a = {};
    if (rope) {
        if (cos == nullptr || sin == nullptr || table_strides == nullptr)
            return set_error(KERNL_ERR_INVALID_ARG, "few-row linear: rotation needs cos, sin and their strides");
        if (table_dtype != KERNL_F16 && table_dtype != KERNL_BF16 && table_dtype != KERNL_F32)
            return set_error(KERNL_ERR_UNSUPPORTED, "few-row linear: unknown table dtype %d", table_dtype);
        if ((head_dim != 32 && head_dim != 64 && head_dim != 128) || N % head_dim != 0 || rope_cols < 0 || rope_cols > N ||
            rope_cols % head_dim != 0 || rows_per_batch <= 0 || table_strides[2] != 1 || activation != KERNL_ACT_NONE)
            return set_error(KERNL_ERR_UNSUPPORTED, "few-row linear: rotation needs a head size of 32, 64 or 128 that divides "
                             "N and rope_cols, tables with unit feature stride, rows_per_batch > 0 and no activation");
        a.cos = cos; a.sin = sin;
        a.t_bs = table_strides[0]; a.t_ss = table_strides[1];
        a.table_dtype = table_dtype;
        a.half = (int)(head_dim / 2);
        a.rope_cols = (int)rope_cols;
        a.rows_per_batch = (int)rows_per_batch;
    }
    if (M == 0) return KERNL_OK;
    const int64_t n_rows = gated ? 2 * N : N;   // rows of the weight
    if (((n_rows + kFewRowTile - 1) / kFewRowTile) * (K / 64) >= (int64_t)1 << 30)
        return set_error(KERNL_ERR_UNSUPPORTED, "few-row linear: N * K too large");
    const FewRowPlan p = fewrow_plan(M, n_rows, K, gated || rope);
    const int64_t need = p.partial_bytes + p.sq_bytes;
    if (need > 0 && (workspace == nullptr || workspace_bytes < need))
        return set_error(KERNL_ERR_INVALID_ARG, "few-row linear: the workspace must hold %lld bytes "
                         "(kernl_linear_fewrow_workspace_bytes), got %lld", (long long)need,
                         (long long)(workspace == nullptr ? 0 : workspace_bytes));
    a.x = x; a.w = w; a.bias = bias; a.residual = residual; a.rms_w = rms_weight; a.out = out;
    a.part = static_cast<float *>(workspace);
    a.sqpart = workspace != nullptr ? reinterpret_cast<float *>(static_cast<char *>(workspace) + p.partial_bytes) : nullptr;
    a.M = (int)M; a.N = (int)n_rows; a.K = (int)K;
    a.ldx = x_strides[0]; a.out_rs = out_strides[0]; a.out_cs = out_strides[1];
    a.res_rs = residual ? residual_strides[0] : 0; a.res_cs = residual ? residual_strides[1] : 0;
    a.act = activation; a.tiles = p.tiles; a.nch = p.nch; a.run = p.run; a.direct = p.direct ? 1 : 0;
    a.eps = eps;
    const int mode = gated ? kFewRowGated : rope ? kFewRowRope : kFewRowPlain;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (w8) launch_fewrow<f16, true>(a, p, mode, st);
    else if (dtype == KERNL_F16) launch_fewrow<f16>(a, p, mode, st);
    else launch_fewrow<bf16>(a, p, mode, st);
    return check_launch("linear (few rows, stream-K)");
}
}  // namespace kernl

extern "C" int kernl_linear_fewrow_fwd(const void *x, const void *rms_weight, float eps, const void *w, const void *bias,
                                       const void *residual, void *out, void *workspace, int64_t workspace_bytes,
                                       int64_t M, int64_t N, int64_t K, const int64_t x_strides[2],
                                       const int64_t out_strides[2], const int64_t residual_strides[2], const void *cos,
                                       const void *sin, int64_t head_dim, int64_t rope_cols, int64_t rows_per_batch,
                                       const int64_t table_strides[3], int table_dtype, int activation, int gated,
                                       int dtype, void *stream) {
    return kernl::fewrow_entry(x, rms_weight, eps, w, bias, residual, out, workspace, workspace_bytes, M, N, K, x_strides,
                               out_strides, residual_strides, cos, sin, head_dim, rope_cols, rows_per_batch, table_strides,
                               table_dtype, activation, gated, dtype, stream, false);
}

extern "C" int kernl_linear_fewrow_w8_fwd(const void *x, const void *rms_weight, float eps, const void *w8,
                                          const void *bias, const void *residual, void *out, void *workspace,
                                          int64_t workspace_bytes, int64_t M, int64_t N, int64_t K,
                                          const int64_t x_strides[2], const int64_t out_strides[2],
                                          const int64_t residual_strides[2], const void *cos, const void *sin,
                                          int64_t head_dim, int64_t rope_cols, int64_t rows_per_batch,
                                          const int64_t table_strides[3], int table_dtype, int activation, int gated,
                                          int dtype, void *stream) {
    if (dtype != KERNL_F16)
        return kernl::set_error(KERNL_ERR_UNSUPPORTED, "few-row linear (fp8 weight): activations must be f16, got dtype %d", dtype);
    return kernl::fewrow_entry(x, rms_weight, eps, w8, bias, residual, out, workspace, workspace_bytes, M, N, K, x_strides,
                               out_strides, residual_strides, cos, sin, head_dim, rope_cols, rows_per_batch, table_strides,
                               table_dtype, activation, gated, dtype, stream, true);
}
