// Flash-attention forward for gfx950:  out = softmax(q·kᵀ·scale + causal + mask) · v.
//
// Semantics follow the reference kernel src/kernl/implementations/attention.py:122-435: scores and both
// accumulators in fp32, additive mask with -inf entries clamped to a finite minimum, top-left aligned causal
// masking, online softmax over key tiles, P rounded to the input dtype before P·V.  The softmax is kept
// un-normalised until the end (one division per output element instead of the reference's per-tile
// renormalisation, attention.py:399-417) — the same value up to fp32 rounding.
//
// MFMA path.  A workgroup of 4 waves owns 128 query rows of one (batch, head); each wave owns 32 of them.
// Key/value tiles of 64 keys go HBM -> LDS directly (buffer loads with the LDS flag, double buffered, one barrier
// per tile):
//   K tile [64 keys][D]   row-major, 16-byte chunks XOR-swizzled;
//   V tile [64 keys][D]   row-major, 64-byte windows XOR-swizzled; P·V contracts over keys and an MFMA lane needs 8
//                         consecutive values of the contraction index, which the transposing LDS read
//                         (ds_read_b64_tr_b16) delivers from this layout.
// Scores are computed TRANSPOSED: Sᵀ = K·Qᵀ with K on the MFMA "A" side, so a lane ends up with the scores of
// ONE query row (lane % 32) against 32 keys.  Row max and row sum are then lane-local loops plus a single
// exchange with lane ^ 32, and the fp32 score registers, once exponentiated and packed to 16 bit, already are
// the MFMA "B" operand of Oᵀ = Vᵀ·Pᵀ — P never touches LDS.  Vᵀ rows are fed through rowperm16, so each lane
// finishes with 16 consecutive output features of its query row and writes them as two 16-byte stores.
#include "attention_common.h"

namespace kernl {

// ----------------------------------------------------------------------------------------------------
// Streaming MFMA kernel: 64-key tiles staged by buffer loads that write LDS directly (no register staging, no
// transposition pass): K swizzled as above, V row-major with its 64-byte windows swizzled, read back through the
// transposing LDS load.  A wave issues one instruction every few cycles whatever its kind, so the loop is kept
// free of bookkeeping: key tiles that need no masking at all ("clean") run first through a branch-free body that
// is unrolled over the two LDS stages; the others (ragged last tile, masked, causal diagonal) follow in a general
// body.  The order of key tiles does not matter to the online softmax.
// ----------------------------------------------------------------------------------------------------
// KV8: keys and values are stored as one byte per element (fp8 e5m2, the upper byte of the fp16 encoding).  Their
// tiles cannot be written to LDS by the load itself then: a thread fetches the 8 bytes of each of its 16-byte LDS
// chunks into registers while the current tile is processed, widens them and stores them before the barrier that
// publishes the stage.  Everything that reads LDS is the 16-bit kernel.
// WSPLIT (small grids: a few (batch, head) pairs, a few hundred keys or more): a workgroup owns 32 query rows instead of
// 128 and its four waves split the KEY tiles of those rows — wave w takes tiles w, w + 4, ... through a double buffer of
// its own, no barrier in the loop — and merge their (reference, row sum, accumulator) triples through LDS at the end.
// Four times the workgroups, a quarter of the serial tile chain per wave.  Head size 64, no mask or a per-key mask,
// non-causal, at most 64 key tiles; 8 stages of dynamic LDS.
template <typename T, int D, int WPE, int MASK_MODE, bool CAUSAL, bool KV8 = false, bool WSPLIT = false>
__global__ void __launch_bounds__(256, WPE) attention_stream_kernel(const AttnParams p) {
    static_assert(!WSPLIT || (D == 64 && !CAUSAL && !KV8 && MASK_MODE != MASK_MATRIX), "key tiles split over the waves: plain forms only");
    typedef typename Vec8<T>::type vec8;
    typedef __attribute__((address_space(3))) void lds_void;
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef short s16x8 __attribute__((ext_vector_type(8)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    typedef AttnTileMap<D> TileMap;                       // staging and fragment addresses of a K / V stage
    constexpr int BM = WSPLIT ? 32 : 128, BN = 64;
    constexpr int KROW = D * 2, VP = D * 2;               // LDS row bytes of the K tile [key][D] and V tile [key][D]
    constexpr int K_BYTES = BN * KROW, V_BYTES = BN * VP;
    constexpr int STAGE = K_BYTES + V_BYTES + BN * 4;     // + per-key additive term (fp32)
    constexpr int NBS = BN / 32, DB = D / 32, KS = D / 16;
    constexpr int DC = D / 8;                             // 16-byte chunks per K/V row
    constexpr int KI = BN * DC / (WSPLIT ? 64 : 256);     // 1 KB loads per wave for each of K and V
    constexpr int DMA_STRIDE = WSPLIT ? 1024 : 4096;      // LDS distance between a wave's consecutive loads of a tile

    // head size 64 stages matrix masks through LDS: every wave keeps the 32 rows x 64 keys it needs of the current
    // key tile (8 KB as fp32) in a region of its own
    constexpr bool MASK_VIA_LDS = (MASK_MODE == MASK_MATRIX && D == 64);
    constexpr int MASK_WAVE_BYTES = 32 * BN * 4;
    constexpr int MASK_LDS = MASK_VIA_LDS ? 4 * MASK_WAVE_BYTES : 0;

    __shared__ __attribute__((aligned(16))) unsigned char static_smem[WSPLIT ? 16 : 2 * STAGE + MASK_LDS];
    extern __shared__ __attribute__((aligned(16))) unsigned char dynamic_smem[];  // WSPLIT: 4 waves x 2 stages
    unsigned char *const smem = WSPLIT ? dynamic_smem : static_smem;

    // Workgroup ids are dealt round-robin to the 8 XCDs.  Normally the query tiles of one (batch, head) share an XCD
    // and with it the L2 that holds their keys and values; with a matrix mask that is broadcast over heads the
    // workgroups of one batch entry — all heads — share it, so that the mask, the larger operand, is fetched once.
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    int b, h, qt;
    if (WSPLIT) {
        // small grids: workgroups are dealt to the XCDs one by one (the keys and values of a head are small, every XCD
        // may fetch them), so that a grid of up to 256 workgroups is one round whatever the number of heads
        const int bh = (int)blockIdx.x / p.nq_tiles;
        qt = (int)blockIdx.x % p.nq_tiles;
        b = bh / p.H;
        h = bh % p.H;
    } else if (MASK_MODE == MASK_MATRIX && p.xcd_by_batch) {
        const int per_batch = p.H * p.nq_tiles;
        b = (slot / per_batch) * 8 + xcd;
        h = (slot % per_batch) / p.nq_tiles;
        qt = slot % p.nq_tiles;
        if (b >= p.B) return;
    } else {
        const int bh = (slot / p.nq_tiles) * 8 + xcd;
        qt = slot % p.nq_tiles;
        if (bh >= p.B * p.H) return;
        b = bh / p.H;
        h = bh % p.H;
    }
    if (CAUSAL) qt = p.nq_tiles - 1 - qt;  // longest rows first

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 31, lh = lane >> 5;
    const int q0 = qt * BM;
    const int m_wave0 = WSPLIT ? q0 : q0 + wave * 32;
    const int wave_lds = WSPLIT ? wave * (2 * STAGE) : 0;  // WSPLIT: the wave's private pair of stages
    const int ktid = WSPLIT ? lane : tid;                  // the thread's index among those that stage a tile together
    const int my_m = m_wave0 + lr;
    const int M = p.M, N = p.N;

    const T *qp = static_cast<const T *>(p.q) + b * p.qs[0] + h * p.qs[1];
    constexpr int KVB = KV8 ? 1 : 2;  // bytes per key / value element in memory
    const char *kp = static_cast<const char *>(p.k) + (b * p.ks[0] + h * p.ks[1]) * KVB;
    const char *vp = static_cast<const char *>(p.v) + (b * p.vs[0] + h * p.vs[1]) * KVB;
    T *op = static_cast<T *>(p.o) + b * p.os[0] + h * p.os[1];
    const int64_t mask_base = (MASK_MODE != MASK_NONE) ? b * p.ms[0] + h * p.ms[1] : 0;

    // ---- Q fragments (MFMA "B" side: lane holds its query row, 8 consecutive features per k-step)
    vec8 qf[KS];
    {
        const T *qrow = qp + (int64_t)min(my_m, M - 1) * p.qs[2] + lh * 8;
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const vec8 *>(qrow + s * 16);
    }
    // Q is multiplied by scale * log2(e) once, here (one more rounding of Q to 16 bits), so that the MFMA result is
    // the score in the base-2 domain and the tile loop spends no instruction on scaling.
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[s][e] = from_float<T>(to_float(qf[s][e]) * p.scale_log2);

    // ---- staging: the i-th load of a wave fills the 1 KB of 16-byte chunks [256 i + 64 wave, +64) of a tile;
    // every lane fetches the chunk of global memory that belongs at its LDS position under the tile's swizzle
    // (V: the 64-byte window of a row is XORed with low key bits so that a transposing read of 4 consecutive keys
    // x 32 features touches every bank once).  Rows past the last key lie beyond the extent of the buffer
    // resource and arrive as zeros.
    uint32_t kdma[KI], vdma[KI];
#pragma unroll
    for (int i = 0; i < KI; ++i) {
        const int qd = ktid + (WSPLIT ? 64 : 256) * i;
        const int row = TileMap::stage_row(qd);
        kdma[i] = (uint32_t)(((int64_t)row * p.ks[2] + TileMap::k_stage_chunk(qd) * 8) * KVB);
        vdma[i] = (uint32_t)(((int64_t)row * p.vs[2] + TileMap::v_stage_chunk(qd) * 8) * KVB);
    }
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void *)smem;
    const uint32_t dma_base = lds_base + (WSPLIT ? wave_lds : wave * 1024);
    const uint64_t kaddr = (uint64_t)(uintptr_t)kp, vaddr = (uint64_t)(uintptr_t)vp;
    const u32x4 krsrc = {(uint32_t)kaddr, (uint32_t)(kaddr >> 32) & 0xFFFFu,
                         (uint32_t)((((int64_t)N - 1) * p.ks[2] + D) * KVB), 0x00020000u};
    const u32x4 vrsrc = {(uint32_t)vaddr, (uint32_t)(vaddr >> 32) & 0xFFFFu,
                         (uint32_t)((((int64_t)N - 1) * p.vs[2] + D) * KVB), 0x00020000u};
    const int k_tile_bytes = (int)((int64_t)BN * p.ks[2] * KVB), v_tile_bytes = (int)((int64_t)BN * p.vs[2] * KVB);
    // one-byte keys and values: ordinary buffer loads into registers (the compiler tracks them), committed to LDS later
    const __amdgpu_buffer_rsrc_t krsrc8 = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char *>(kp), 0, KV8 ? (int)((((int64_t)N - 1) * p.ks[2] + D) * KVB) : 0, 0x00020000);
    const __amdgpu_buffer_rsrc_t vrsrc8 = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char *>(vp), 0, KV8 ? (int)((((int64_t)N - 1) * p.vs[2] + D) * KVB) : 0, 0x00020000);
    u32x2 kraw[KV8 ? KI : 1], vraw[KV8 ? KI : 1];
    // Inline assembly on purpose: the compiler, seeing LDS written by a load, would make every later LDS read
    // wait for the vector-memory counter, i.e. for the prefetch itself.  The explicit wait before the barrier
    // that publishes the stage is the one that matters.
    auto uniform = [](uint32_t x) __attribute__((always_inline)) -> uint32_t { return (uint32_t)__builtin_amdgcn_readfirstlane((int)x); };
    auto dma = [&](int tile, int stage) __attribute__((always_inline)) {
        if constexpr (KV8) {
#pragma unroll
            for (int i = 0; i < KI; ++i) {
                kraw[i] = __builtin_amdgcn_raw_buffer_load_b64(krsrc8, kdma[i], tile * k_tile_bytes, 0);
                vraw[i] = __builtin_amdgcn_raw_buffer_load_b64(vrsrc8, vdma[i], tile * v_tile_bytes, 0);
            }
            return;
        }
        // every operand below is wave-uniform; saying so explicitly keeps them in scalar registers whatever the
        // control flow around the call looks like to the compiler
        const uint32_t k_soff = uniform((uint32_t)(tile * k_tile_bytes)), v_soff = uniform((uint32_t)(tile * v_tile_bytes));
        const uint32_t sb = uniform(dma_base + stage * STAGE);
        const u32x4 kr = {uniform(krsrc[0]), uniform(krsrc[1]), uniform(krsrc[2]), uniform(krsrc[3])};
        const u32x4 vr = {uniform(vrsrc[0]), uniform(vrsrc[1]), uniform(vrsrc[2]), uniform(vrsrc[3])};
#pragma unroll
        for (int i = 0; i < KI; ++i)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :: "s"(sb + i * DMA_STRIDE), "v"(kdma[i]), "s"(kr), "s"(k_soff) : "memory", "m0");
#pragma unroll
        for (int i = 0; i < KI; ++i)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :: "s"(sb + K_BYTES + i * DMA_STRIDE), "v"(vdma[i]), "s"(vr), "s"(v_soff) : "memory", "m0");
    };
    // one-byte keys and values: the fetched bytes, widened (byte b of a dword becomes the 16-bit value b << 8), go to
    // the LDS positions the direct loads of the 16-bit kernel would have written
    auto kv8_commit = [&](int stage) __attribute__((always_inline)) {
        if constexpr (KV8) {
            unsigned char *sbase = smem + stage * STAGE + tid * 16;
#pragma unroll
            for (int i = 0; i < KI; ++i) {
                const u32x4 kw = {__builtin_amdgcn_perm(0u, kraw[i][0], 0x010c000cu), __builtin_amdgcn_perm(0u, kraw[i][0], 0x030c020cu),
                                  __builtin_amdgcn_perm(0u, kraw[i][1], 0x010c000cu), __builtin_amdgcn_perm(0u, kraw[i][1], 0x030c020cu)};
                const u32x4 vw = {__builtin_amdgcn_perm(0u, vraw[i][0], 0x010c000cu), __builtin_amdgcn_perm(0u, vraw[i][0], 0x030c020cu),
                                  __builtin_amdgcn_perm(0u, vraw[i][1], 0x010c000cu), __builtin_amdgcn_perm(0u, vraw[i][1], 0x030c020cu)};
                *reinterpret_cast<u32x4 *>(sbase + i * 4096) = kw;
                *reinterpret_cast<u32x4 *>(sbase + K_BYTES + i * 4096) = vw;
            }
        }
    };
    // per-key additive term of a general tile (mask value in the log2 domain, -inf past the last key); thread tid
    // < 64 owns key tid of the tile
    auto key_bias = [&](int tile) __attribute__((always_inline)) -> float {
        const int n = tile * BN + ktid;
        float bv = 0.0f;
        if (MASK_MODE == MASK_VECTOR)
            bv = scale_mask(load_mask_value(p.mask, p.mask_dtype, mask_base + min(n, N - 1) * p.ms[3]), p.clamp);
        if (n >= N) bv = -INFINITY;
        return bv;
    };

    // ---- key tiles: [0, n_clean) of the processing order need no masking, [n_clean, nt) take the general body
    const int n_end = CAUSAL ? min(N, q0 + BM + p.causal_off) : N;
    const int nt_all = (n_end + BN - 1) / BN;
    // (causal with a per-key mask: tiles that reach beyond the diagonal of the workgroup's first row are never clean)
    constexpr bool MAY_LIST = (MASK_MODE == MASK_VECTOR);
    const int first_diag_key = CAUSAL ? q0 + p.causal_off : 0x7fffffff;  // keys above it are hidden from some row
    const bool use_list = WSPLIT || (MAY_LIST && nt_all <= 64);  // (the host hands WSPLIT at most 64 tiles)
    int nt = nt_all, n_clean = 0;
    if (MASK_MODE == MASK_NONE) n_clean = CAUSAL ? min(N / BN, (q0 + p.causal_off + 1) / BN) : N / BN;
    // the first tile is fetched before the mask has been looked at: tile 0 almost always comes first
    // (WSPLIT: wave w's tiles are w, w + 4, ...)
    const int t_first = WSPLIT ? wave : 0;
    if (t_first < nt_all) dma(t_first, 0);
    // With a per-key mask every wave classifies all key tiles by itself (the mask row is a few KB, and this way no
    // barrier or LDS table is needed): bit t of clean_bits = tile t is all zero and full, of gen_bits = it needs
    // the general body; tiles in neither set are so negative everywhere that they contribute exactly 0 and are
    // dropped.  Both sets are wave-uniform scalars; tiles are taken from them lowest index first.
    uint64_t clean_bits = 0, gen_bits = 0;
    constexpr bool SHARED = !WSPLIT;
    __shared__ uint64_t tile_sets[4][2];
    if (use_list && MASK_MODE == MASK_VECTOR) {
        // lane l looks at key 64 t + l of tile t; 32-bit offsets (the host checks that a mask row fits them)
        auto classify = [&](auto *mrow) __attribute__((always_inline)) {
            const int ms3 = (int)p.ms[3];
            const int lane_off = lane * ms3, tile_step_off = BN * ms3;
            for (int t0 = 0; t0 < nt_all; t0 += 8) {
                float mv[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    mv[j] = 0.0f;
                    if (t0 + j < nt_all && (t0 + j) * BN + lane < N) mv[j] = (float)mrow[lane_off + (t0 + j) * tile_step_off];
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int t = t0 + j;
                    if (t < nt_all) {
                        const bool valid = t * BN + lane < N;
                        const float sm = scale_mask(mv[j], p.clamp);
                        const bool any_nonzero = __ballot(valid && (sm != 0.0f)) != 0;
                        const bool any_normal = __ballot(valid && (sm > kDeadMask)) != 0;
                        if (any_normal || CAUSAL) {  // (causal: a row may see dead keys only — they are visited)
                            if (any_nonzero || t * BN + BN > N || t * BN + BN - 1 > first_diag_key) gen_bits |= 1ull << t;
                            else clean_bits |= 1ull << t;
                        }
                    }
                }
            }
        };
        // Contiguous, 16-byte aligned mask rows take a shorter route: a lane loads 4 consecutive keys, so 16 lanes
        // cover a tile and one load covers 4 tiles; lanes 0..3 then each judge one of those tiles from the two
        // wave-wide ballots.
        auto classify4 = [&](auto *mrow) __attribute__((always_inline)) {
            typedef typename std::remove_cv<typename std::remove_pointer<decltype(mrow)>::type>::type MT;
            const __amdgpu_buffer_rsrc_t mrsrc =
                __builtin_amdgcn_make_buffer_rsrc(const_cast<MT *>(mrow), 0, N * (int)sizeof(MT), 0x00020000);
            // two loads (512 keys) in flight per step: the loop is a chain of memory round trips otherwise
            auto fetch = [&](int j, float (&mv)[4]) __attribute__((always_inline)) {
                const int e0 = (64 * j + lane) * 4;  // (beyond the row the buffer returns zeros; `valid` below ignores them)
                if constexpr (sizeof(MT) == 4) {
                    const f32x4 raw = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(mrsrc, e0 * 4, 0, 0));
#pragma unroll
                    for (int r = 0; r < 4; ++r) mv[r] = raw[r];
                } else {
                    typedef MT mt4 __attribute__((ext_vector_type(4)));
                    const mt4 raw = __builtin_bit_cast(mt4, __builtin_amdgcn_raw_buffer_load_b64(mrsrc, e0 * 2, 0, 0));
#pragma unroll
                    for (int r = 0; r < 4; ++r) mv[r] = (float)raw[r];
                }
            };
            auto judge = [&](int j, const float (&mv)[4]) __attribute__((always_inline)) {
                const int e0 = (64 * j + lane) * 4;
                bool nz = false, nm = false;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float sm = scale_mask(mv[r], p.clamp);
                    const bool valid = e0 + r < N;
                    nz |= valid && (sm != 0.0f);
                    nm |= valid && (sm > kDeadMask);
                }
                const uint64_t bz = __ballot(nz), bn = __ballot(nm);
                const int k = lane & 3, t = 4 * j + k;
                const bool any_nz = ((bz >> (16 * k)) & 0xFFFFull) != 0, any_nm = ((bn >> (16 * k)) & 0xFFFFull) != 0;
                const bool mine = lane < 4 && t < nt_all && (any_nm || CAUSAL);  // (causal: a row may see dead keys only — they are visited)
                const bool general = any_nz || t * BN + BN > N || t * BN + BN - 1 > first_diag_key;
                clean_bits |= (__ballot(mine && !general) & 0xFull) << (4 * j);
                gen_bits |= (__ballot(mine && general) & 0xFull) << (4 * j);
            };
            // SHARED: the four waves of a workgroup want the same two sets, so wave w judges the loads j = w, w + 4, ...
            // only and the sets are put together through LDS below (WSPLIT waves synchronise among themselves only:
            // each judges everything)
            constexpr int FIRST_STEP = SHARED ? 4 : 1;
            for (int j = SHARED ? wave : 0; j * 256 < N; j += 2 * FIRST_STEP) {
                float mv0[4], mv1[4];
                fetch(j, mv0);
                fetch(j + FIRST_STEP, mv1);
                judge(j, mv0);
                if ((j + FIRST_STEP) * 256 < N) judge(j + FIRST_STEP, mv1);
            }
        };
        const bool rows_vectorizable = p.ms[3] == 1;
        bool shared_sets = false;
        if (p.mask_dtype == KERNL_F32) {
            const float *mrow = static_cast<const float *>(p.mask) + mask_base;
            if (rows_vectorizable && aligned16(mrow)) classify4(mrow), shared_sets = SHARED;
            else classify(mrow);
        } else if (p.mask_dtype == KERNL_F16) {
            const f16 *mrow = static_cast<const f16 *>(p.mask) + mask_base;
            if (rows_vectorizable && aligned16(mrow)) classify4(mrow), shared_sets = SHARED;
            else classify(mrow);
        } else {
            const bf16 *mrow = static_cast<const bf16 *>(p.mask) + mask_base;
            if (rows_vectorizable && aligned16(mrow)) classify4(mrow), shared_sets = SHARED;
            else classify(mrow);
        }
        if constexpr (SHARED) {
            if (shared_sets) {  // (workgroup-uniform: the mask row's layout decides)
                if (lane == 0) {
                    tile_sets[wave][0] = clean_bits;
                    tile_sets[wave][1] = gen_bits;
                }
                __syncthreads();
                const uint64_t c = tile_sets[0][0] | tile_sets[1][0] | tile_sets[2][0] | tile_sets[3][0];
                const uint64_t g = tile_sets[0][1] | tile_sets[1][1] | tile_sets[2][1] | tile_sets[3][1];
                // (every lane read the same words: back into scalar registers, where the tile order is computed)
                clean_bits = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(c >> 32)) << 32) | (uint32_t)__builtin_amdgcn_readfirstlane((int)c);
                gen_bits = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(g >> 32)) << 32) | (uint32_t)__builtin_amdgcn_readfirstlane((int)g);
            }
        }
        // every key masked: keep all tiles, the result is the (finite) uniform average
        if ((clean_bits | gen_bits) == 0) gen_bits = (nt_all >= 64) ? ~0ull : ((1ull << nt_all) - 1ull);
        n_clean = __popcll(clean_bits);
        nt = n_clean + __popcll(gen_bits);
    }
    if constexpr (WSPLIT) {
        if (MASK_MODE == MASK_NONE) {  // the full tiles, then the ragged one
            const int full = N / BN;
            clean_bits = full >= 64 ? ~0ull : ((1ull << full) - 1ull);
            gen_bits = (N % BN) != 0 ? 1ull << full : 0ull;
        }
        const uint64_t mine = 0x1111111111111111ull << wave;  // tiles t with t % 4 == wave
        clean_bits &= mine;
        gen_bits &= mine;
        n_clean = __popcll(clean_bits);
        nt = n_clean + __popcll(gen_bits);
    }
    // next tile of the processing order; past the end it repeats `last` (a harmless extra prefetch)
    int order_pos = 0;
    auto next_tile = [&](int last) __attribute__((always_inline)) -> int {
        int t;
        if (use_list) {
            // (value selects on purpose: written as "clear the lowest bit of whichever set is not empty" the two sets end
            // up behind a selected address, i.e. in scratch memory)
            const bool from_clean = clean_bits != 0;
            const uint64_t set = from_clean ? clean_bits : gen_bits;
            const uint64_t rest = set & (set - 1);
            t = set != 0 ? __builtin_ctzll(set) : last;
            clean_bits = from_clean ? rest : clean_bits;
            gen_bits = from_clean ? gen_bits : rest;
        } else {
            t = min(order_pos, nt - 1);
        }
        ++order_pos;
        return __builtin_amdgcn_readfirstlane(t);
    };

    // ---- running state of this lane's query row
    // m_i is the exponent REFERENCE of the row (base-2 domain); its negative, replicated over a block of 16
    // registers, is the C operand of the first score MFMA of every block, so that the MFMA delivers
    // score - reference and the exponential needs no subtraction either.
    // (Head size 128 with a matrix mask has no registers left for that block: there the reference is subtracted
    // from every score by an instruction of its own.)
    constexpr bool REF_IN_MFMA = !(D == 128 && MASK_MODE == MASK_MATRIX);
    float m_i = 0.0f, m_masked = -INFINITY, l_i = 0.0f;
    bool fresh = true;
    f32x16 neg_m;
#pragma unroll
    for (int v = 0; v < 16; ++v) neg_m[v] = 0.0f;
    f32x16 o_acc[DB];
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) o_acc[d][v] = 0.0f;

    // LDS byte offsets of this lane's operand fragments.  K: row lr of a 32-key block, chunk 2 ks + lh.  V: in each
    // group of 16 lanes, lane i hands the transposing read the address of 4 consecutive features of key (i / 4)
    // and receives feature column i of the 4-key x 16-feature block, i.e. 4 consecutive keys of one feature; the
    // 16 lanes of a group are MFMA rows 16 (group % 2) + 0..15, whose features (through rowperm16) are four runs
    // of 4.
    int k_off[KS], vt_off[DB];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_off[ks] = TileMap::k_frag_offset(lr, lh, ks);
#pragma unroll
    for (int d = 0; d < DB; ++d) vt_off[d] = K_BYTES + TileMap::v_frag_offset(lane, d);
    const int64_t mask_row = mask_base + (int64_t)min(my_m, M - 1) * (MASK_MODE == MASK_MATRIX ? p.ms[2] : 0);
    // Matrix masks on the fast route: the 8 runs of 4 consecutive keys a lane needs from its mask row are
    // fetched one tile ahead, right after the previous tile's values have been consumed, into the same registers.
    constexpr bool MATRIX = (MASK_MODE == MASK_MATRIX);
    const bool m_fast = MATRIX && p.mask_fast != 0;
    const bool m_f32 = p.mask_dtype == KERNL_F32;
    const int m_esize = m_f32 ? 4 : 2;
    const __amdgpu_buffer_rsrc_t mrsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char *>(static_cast<const char *>(p.mask)) + (MATRIX ? mask_base * m_esize : 0), 0,
        MATRIX ? (int)((((int64_t)M - 1) * p.ms[2] + N) * m_esize) : 0, 0x00020000);
    const int m_voff = MATRIX ? (int)((int64_t)min(my_m, M - 1) * p.ms[2] + lh * 4) * m_esize : 0;
    const float clamp_eff = fmaxf(p.clamp, kClampFloor / kLog2eA);  // (-inf -> clamp) * log2(e) stays finite
    u32x4 mreg[MATRIX ? 2 * NBS * 2 : 1];
    // Routes 3 (fp32) and 4 (16-bit): the wave's 32 mask rows of a key tile travel HBM -> LDS by loads that write LDS
    // directly, 1 KB per instruction and fully coalesced (a row's 64 keys are 256 or 128 contiguous bytes), and from
    // there into the lane's registers.  LDS holds row r as 16-byte chunks at r * row_bytes + 16 * (c ^ f(r)), with
    // f(r) = r % 16 for fp32 rows (16 chunks) and (r / 2) % 8 for 16-bit rows (8 chunks): a lane reads its own row, so
    // the lanes of a read hit different banks.  Only the wave itself touches its region: program order and the
    // memory counters are all the synchronisation there is.
    const uint32_t mlds_base = lds_base + 2 * STAGE + wave * MASK_WAVE_BYTES;
    const uint64_t maddr = (uint64_t)(uintptr_t)(static_cast<const char *>(p.mask) + (MATRIX ? mask_base * m_esize : 0));
    const u32x4 mrsrc4 = {(uint32_t)maddr, (uint32_t)(maddr >> 32) & 0xFFFFu,
                          MATRIX ? (uint32_t)((((int64_t)M - 1) * p.ms[2] + N) * m_esize) : 0u, 0x00020000u};
    uint32_t mdma[MASK_VIA_LDS ? 8 : 1];
    if (MASK_VIA_LDS && p.mask_fast == 2) {
        const int row0 = q0 + wave * 32;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int r = m_f32 ? MaskTileMap<4>::stage_row(i, lane) : MaskTileMap<2>::stage_row(i & 3, lane);
            const int c = m_f32 ? MaskTileMap<4>::stage_chunk(i, lane) : MaskTileMap<2>::stage_chunk(i & 3, lane);
            // rows past the last query read the last row again (their results are never stored)
            mdma[i] = (uint32_t)(((int64_t)min(row0 + r, M - 1) * p.ms[2]) * m_esize + c * 16);
        }
    }
    auto mask_dma = [&](int tile) __attribute__((always_inline)) {
        const u32x4 mru = {uniform(mrsrc4[0]), uniform(mrsrc4[1]), uniform(mrsrc4[2]), uniform(mrsrc4[3])};
        const uint32_t soff = uniform((uint32_t)(tile * BN * m_esize));
        const uint32_t mb = uniform(mlds_base);
        if (m_f32) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                             :: "s"(mb + i * 1024), "v"(mdma[i]), "s"(mru), "s"(soff) : "memory", "m0");
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                             :: "s"(mb + i * 1024), "v"(mdma[i]), "s"(mru), "s"(soff) : "memory", "m0");
        }
    };
    // LDS -> registers, then (the region being free again) the request for the tile after
    auto mask_take = [&](auto route_c, int tile_after) __attribute__((always_inline)) {
        constexpr int ROUTE = decltype(route_c)::value;
        const unsigned char *mb = smem + 2 * STAGE + wave * MASK_WAVE_BYTES;
        if (ROUTE == 3) {
#pragma unroll
            for (int i = 0; i < NBS * 4; ++i)
                mreg[i] = *reinterpret_cast<const u32x4 *>(mb + MaskTileMap<4>::read_offset(lr, lh, i));
        } else {
#pragma unroll
            for (int i = 0; i < NBS * 4; ++i) {
                const u32x2 two = *reinterpret_cast<const u32x2 *>(mb + MaskTileMap<2>::read_offset(lr, lh, i));
                mreg[i >> 1][2 * (i & 1)] = two[0];
                mreg[i >> 1][2 * (i & 1) + 1] = two[1];
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        mask_dma(tile_after);
    };
    auto mask_issue = [&](auto route_c, int tile) __attribute__((always_inline)) {
        constexpr int ROUTE = decltype(route_c)::value;
        if (ROUTE == 2) {
#pragma unroll
            for (int i = 0; i < NBS * 4; ++i)
                mreg[i] = __builtin_amdgcn_raw_buffer_load_b128(mrsrc, m_voff + ((i >> 2) * 32 + (i & 3) * 8) * 4, tile * BN * 4, 0);
        } else if (ROUTE == 1) {
#pragma unroll
            for (int i = 0; i < NBS * 4; ++i) {
                const u32x2 two = __builtin_amdgcn_raw_buffer_load_b64(mrsrc, m_voff + ((i >> 2) * 32 + (i & 3) * 8) * 2, tile * BN * 2, 0);
                mreg[i >> 1][2 * (i & 1)] = two[0];
                mreg[i >> 1][2 * (i & 1) + 1] = two[1];
            }
        }
    };

    const uint64_t clean_bits0 = clean_bits, gen_bits0 = gen_bits;  // for a second pass over the tiles
    __shared__ int redo_flag;
    int t_cur = 0, t_nxt = 0;
    if (nt > 0) {
        t_cur = next_tile(0);
        t_nxt = next_tile(t_cur);
    }
    // one key tile: prefetch the next one into the other stage, scores, online softmax, P·V, publish
    // ROUTE: how a matrix mask is read (0 = element by element, 1 = prefetched 16-bit vectors, 2 = prefetched fp32
    // vectors); a compile-time choice so that the tile body carries no branches for it
    // EDGE: the tile may hold keys past the last one or beyond the causal diagonal of some row of the workgroup
    // publishes a stage: to the workgroup, or — WSPLIT, where a stage belongs to one wave, whose LDS operations execute in
    // program order — only to the compiler
    auto stage_sync = [&]() __attribute__((always_inline)) {
        if constexpr (WSPLIT) __builtin_amdgcn_wave_barrier();
        else __syncthreads();
    };
    // opt (wave-uniform, clean tiles only): no running maximum, see `clean_tiles` below
    auto tile_step = [&](auto general_c, auto stage_c, auto route_c, auto edge_c, auto opt_c) __attribute__((always_inline)) {
        constexpr bool GENERAL = decltype(general_c)::value;
        constexpr bool OPT = !GENERAL && REF_IN_MFMA && decltype(opt_c)::value;
        constexpr int ST = decltype(stage_c)::value;
        constexpr int ROUTE = decltype(route_c)::value;
        constexpr bool EDGE = decltype(edge_c)::value;
            const int tile = t_cur, tile_next = t_nxt;
        const int n0 = tile * BN;
        // With a prefetched matrix mask the compiler waits for ALL vector-memory loads before it touches the last
        // mask register (it does not know about the loads issued in assembly), so there the next tile is only
        // requested once the mask values have been consumed.
        constexpr bool LATE_DMA = GENERAL && (MASK_MODE == MASK_MATRIX) && ROUTE < 3;
        if (!LATE_DMA) dma(tile_next, ST ^ 1);
        float bias_next = 0.0f;
        if (GENERAL && ktid < BN) bias_next = key_bias(tile_next);

        const unsigned char *sb = smem + wave_lds + ST * STAGE;
        // a wave whose 32 rows all lie above a causal tile has nothing to compute in it
        if (!(GENERAL && CAUSAL && n0 > m_wave0 + 31 + p.causal_off)) {
            // ---- Sᵀ = K · Qᵀ, relative to the row's reference
            f32x16 s_acc[NBS];
            auto scores = [&]() __attribute__((always_inline)) {
                __builtin_amdgcn_s_setprio(2);
#pragma unroll
                for (int nb = 0; nb < NBS; ++nb) {
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        const vec8 kf = *reinterpret_cast<const vec8 *>(sb + nb * 32 * KROW + k_off[ks]);
                        s_acc[nb] = mfma32(kf, qf[ks], ks == 0 ? neg_m : s_acc[nb]);  // neg_m stays 0 without REF_IN_MFMA
                    }
                }
                __builtin_amdgcn_s_setprio(0);
            };
            scores();

            // ---- online softmax on this lane's row; key of s_acc[nb][v] is n0 + 32 nb + 8 (v/4) + 4 lh + (v%4)
            float mx = -INFINITY;
            if (GENERAL) {
                const float *colbias = reinterpret_cast<const float *>(sb + K_BYTES + V_BYTES);
                // EXACT: per-key term (-inf past the last key), -inf mask entries replaced by the clamp value, causal
                // cut.  The short form — prefetched matrix masks on tiles that are no edge — adds the mask value as it
                // is: an entry of -inf leaves a score of -inf and a probability of exactly 0, which is what the clamped
                // value gives too unless EVERY key of the row is masked; a row that ends the tile without a finite score
                // sends the wave through the exact form once more (the key tile is still in LDS).
                auto masked_scores = [&](auto exact_c) __attribute__((always_inline)) {
                    constexpr bool EXACT = decltype(exact_c)::value;
#pragma unroll
                    for (int nb = 0; nb < NBS; ++nb) {
#pragma unroll
                        for (int g = 0; g < 4; ++g) {
                            const int nl = nb * 32 + g * 8 + lh * 4;  // key index inside the tile
                            f32x4 cb = {0.0f, 0.0f, 0.0f, 0.0f};
                            if (EXACT) cb = *reinterpret_cast<const f32x4 *>(colbias + nl);
                            f32x4 mm = {0.0f, 0.0f, 0.0f, 0.0f};
                            if (MATRIX && ROUTE != 0) {
                                const int i = nb * 4 + g;
                                if (ROUTE == 2 || ROUTE == 3) {
                                    mm = __builtin_bit_cast(f32x4, mreg[i]);
                                } else {
                                    typedef T t4 __attribute__((ext_vector_type(4)));
                                    const u32x2 two = {mreg[i >> 1][2 * (i & 1)], mreg[i >> 1][2 * (i & 1) + 1]};
                                    const t4 h4 = __builtin_bit_cast(t4, two);
#pragma unroll
                                    for (int r = 0; r < 4; ++r) mm[r] = (float)h4[r];
                                }
                            }
#pragma unroll
                            for (int r = 0; r < 4; ++r) {
                                float sv = s_acc[nb][g * 4 + r];
                                if (EXACT) sv += cb[r];
                                if (!REF_IN_MFMA) sv -= m_i;
                                if (MATRIX) {
                                    if (ROUTE != 0) {
                                        sv = fmaf(EXACT ? fmaxf(mm[r], clamp_eff) : mm[r], kLog2eA, sv);
                                    } else {
                                        const int n = min(n0 + nl + r, N - 1);
                                        sv += scale_mask(load_mask_value(p.mask, p.mask_dtype, mask_row + n * p.ms[3]), p.clamp);
                                    }
                                }
                                if (EXACT && CAUSAL && (n0 + nl + r > my_m + p.causal_off)) sv = -INFINITY;
                                s_acc[nb][g * 4 + r] = sv;
                                mx = fmaxf(mx, sv);
                            }
                        }
                    }
                };
                if (MATRIX && ROUTE != 0 && !EDGE) {
                    masked_scores(BoolC<false>());
                    // (written so that a NaN score takes the exact form too)
                    if (__builtin_amdgcn_ballot_w64(!(halves32_max(mx) > -INFINITY)) != 0) {
                        scores();
                        mx = -INFINITY;
                        masked_scores(BoolC<true>());
                    }
                } else {
                    masked_scores(BoolC<true>());
                }
            } else if (!OPT) {
#pragma unroll
                for (int nb = 0; nb < NBS; ++nb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        if (!REF_IN_MFMA) s_acc[nb][v] -= m_i;
                        mx = fmaxf(mx, s_acc[nb][v]);
                    }
            }
            if (LATE_DMA) dma(tile_next, ST ^ 1);
            if constexpr (!OPT) {
            mx = halves32_max(mx);  // the other 16-key half of every 32-key block lives in lane ^ 32
            // The scores are relative to the reference m_i, which is not the running maximum: it only moves (and
            // the accumulator and row sum are rescaled) when a score exceeds it by more than 2^8, so probabilities
            // stay <= 256 — exact in fp32, well inside the 16-bit range — and after the first tiles the rescale
            // almost never runs.  The final O / l is independent of the reference.
            // A row is `fresh` until it has seen a tile with an ordinary score (both lanes of a row agree on that,
            // as they agree on mx); until then m_i stays 0.  Tiles whose scores all lie below kMaskedScore (mask
            // entries of -inf arrive as -1.7e38, half-precision "minus infinity" biases as -9e4) are accumulated
            // against a reference of their own, m_masked, subtracted explicitly here, so that a row without any
            // ordinary key still gets its softmax over the masked ones (the plain average of V for -inf masks, as in
            // the reference implementation).  The first ordinary tile discards that, and sets m_i to its maximum
            // wherever that lies: the reference in the MFMA never goes where fp32 scores relative to it would lose
            // their resolution.
            const bool ordinary = mx > kMaskedScore;
            if (__builtin_amdgcn_ballot_w64(mx > kRescaleThreshold || (fresh && mx > -INFINITY)) != 0) {
                float alpha, dsub;
                if (!fresh) {
                    dsub = fmaxf(mx, 0.0f);
                    alpha = __builtin_amdgcn_exp2f(-dsub);
                    m_i += dsub;
                } else if (ordinary) {
                    dsub = mx;
                    alpha = 0.0f;
                    m_i = mx;
                } else {
                    const float m_new = fmaxf(m_masked, mx);
                    alpha = (m_masked == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(m_masked - m_new);
                    dsub = (m_new == -INFINITY) ? 0.0f : m_new;
                    m_masked = m_new;
                }
                l_i *= alpha;
#pragma unroll
                for (int d = 0; d < DB; ++d)
#pragma unroll
                    for (int v = 0; v < 16; ++v) o_acc[d][v] *= alpha;
#pragma unroll
                for (int nb = 0; nb < NBS; ++nb)
#pragma unroll
                    for (int v = 0; v < 16; ++v) s_acc[nb][v] -= dsub;
#pragma unroll
                for (int v = 0; v < 16; ++v) neg_m[v] = REF_IN_MFMA ? -m_i : 0.0f;
            }
            fresh = fresh && !ordinary;
            }  // !OPT
#pragma unroll
            for (int nb = 0; nb < NBS; ++nb)
#pragma unroll
                for (int v = 0; v < 16; ++v) s_acc[nb][v] = __builtin_amdgcn_exp2f(s_acc[nb][v]);

            // ---- Oᵀ += Vᵀ · Pᵀ; the row sum is taken from the unrounded probabilities with plain additions (the
            // reference does the same, attention.py:399-417): v_dot2c_f32_f16 on the packed pairs, one instruction
            // less per pair, measured 16 cycles of the matrix pipe each when MFMAs are in flight
            float rs = 0.0f, rs2 = 0.0f;
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int ps = 0; ps < BN / 16; ++ps) {
                const int nb = ps >> 1, half8 = (ps & 1) * 8;
                u32x4 pk;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    pk[j] = pack2<T>(s_acc[nb][half8 + 2 * j], s_acc[nb][half8 + 2 * j + 1]);
                    rs += s_acc[nb][half8 + 2 * j];
                    rs2 += s_acc[nb][half8 + 2 * j + 1];
                }
                const vec8 pf = __builtin_bit_cast(vec8, pk);
#pragma unroll
                for (int d = 0; d < DB; ++d) {
                    const unsigned char *va = sb + 16 * ps * VP + vt_off[d];
                    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)va);
                    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(va + 8 * VP));
                    const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    o_acc[d] = mfma32(__builtin_bit_cast(vec8, both), pf, o_acc[d]);
                }
            }
            __builtin_amdgcn_s_setprio(0);
            l_i += rs + rs2;
        } else if (LATE_DMA) {
            dma(tile_next, ST ^ 1);
        }

        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's part of the next tile is in LDS
        kv8_commit(ST ^ 1);
        if (GENERAL && MATRIX) {
            if (ROUTE >= 3) mask_take(route_c, min(tile_next + 1, nt - 1));  // matrix masks walk the tiles in order
            else mask_issue(route_c, tile_next);
        }
        if (GENERAL && ktid < BN)
            *reinterpret_cast<float *>(smem + wave_lds + (ST ^ 1) * STAGE + K_BYTES + V_BYTES + ktid * 4) = bias_next;
        stage_sync();
        t_cur = t_nxt;
        t_nxt = next_tile(t_nxt);
    };

    if (nt > 0) {
        if (t_cur != t_first) dma(t_cur, 0);
        if (n_clean == 0 && ktid < BN)
            *reinterpret_cast<float *>(smem + wave_lds + K_BYTES + V_BYTES + ktid * 4) = key_bias(t_cur);
        kv8_commit(0);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // everything issued so far (Q fragments included) has landed
    stage_sync();

    // clean tiles in pairs over the two stages; an odd one leaves the general tiles starting in stage 1
    // Clean tiles: the first one in full (it takes the row's exponent reference to its maximum: every key of a clean tile
    // is ordinary), the others OPTIMISTICALLY — no running maximum, no rescale check, scores straight into the
    // exponential against the reference the row has — which saves a quarter of a clean tile's vector instructions.
    // Probabilities may then exceed the 2^8 the full step keeps them under; they are still exact enough as long as they
    // fit 16 bits (the relative precision of a half does not depend on its magnitude).  A row sum that reaches 60000 —
    // or is no longer a number — says that some probability may not have fitted: the workgroup (WSPLIT: the wave, which
    // stages its own tiles) then starts over with full steps.  That takes a score 16 octaves above everything in the
    // row's first tile; tests/test_attention.py::test_softmax_reference_moves_with_the_scores has such rows.
    auto clean_tiles = [&](auto opt) __attribute__((always_inline)) -> int {
        int i = 0;
        if (n_clean > 0) {
            tile_step(BoolC<false>(), IntC<0>(), IntC<0>(), BoolC<true>(), BoolC<false>());
            i = 1;
        }
        for (; i + 1 < n_clean; i += 2) {
            tile_step(BoolC<false>(), IntC<1>(), IntC<0>(), BoolC<true>(), opt);
            tile_step(BoolC<false>(), IntC<0>(), IntC<0>(), BoolC<true>(), opt);
        }
        if (i < n_clean) {
            tile_step(BoolC<false>(), IntC<1>(), IntC<0>(), BoolC<true>(), opt);
            ++i;
        }
        return i;
    };
    int idx = 0;
    constexpr bool CAN_OPT = REF_IN_MFMA && MASK_MODE != MASK_MATRIX;
    bool full_pass = true;
    if constexpr (CAN_OPT) {
        if (n_clean > 1) {
            full_pass = false;
            idx = clean_tiles(BoolC<true>());
            int again = __builtin_amdgcn_ballot_w64(!(l_i < 60000.0f)) != 0 ? 1 : 0;
            if constexpr (!WSPLIT) {
                // the four waves stage tiles together: they start over together
                if (tid == 0) redo_flag = 0;
                __syncthreads();
                if (again != 0 && lane == 0) redo_flag = 1;
                __syncthreads();
                again = redo_flag;
            }
            if (__builtin_amdgcn_readfirstlane(again) != 0) {
                full_pass = true;
                clean_bits = clean_bits0;
                gen_bits = gen_bits0;
                order_pos = 0;
                t_cur = next_tile(0);
                t_nxt = next_tile(t_cur);
                m_i = 0.0f;
                m_masked = -INFINITY;
                l_i = 0.0f;
                fresh = true;
#pragma unroll
                for (int v = 0; v < 16; ++v) neg_m[v] = 0.0f;
#pragma unroll
                for (int d = 0; d < DB; ++d)
#pragma unroll
                    for (int v = 0; v < 16; ++v) o_acc[d][v] = 0.0f;
                dma(t_cur, 0);  // (every wave has passed the barrier of the last step: nobody reads the stages any more)
                kv8_commit(0);
                __builtin_amdgcn_s_waitcnt(0x0F70);
                stage_sync();
            }
        }
    }
    if (full_pass) idx = clean_tiles(BoolC<false>());
    const bool odd_clean = (n_clean & 1) != 0;
    if (idx < nt) {
        if (n_clean > 0) {  // the additive terms of the first general tile
            if (ktid < BN)
                *reinterpret_cast<float *>(smem + wave_lds + (odd_clean ? STAGE : 0) + K_BYTES + V_BYTES + ktid * 4) = key_bias(t_cur);
            stage_sync();
        }
        auto general_tiles = [&](auto route_c) __attribute__((always_inline)) {
            constexpr int ROUTE = decltype(route_c)::value;
            if (MATRIX && ROUTE >= 3) {
                mask_dma(t_cur);
                __builtin_amdgcn_s_waitcnt(0x0F70);
                mask_take(route_c, t_nxt);
            } else if (MATRIX) {
                mask_issue(route_c, t_cur);
            }
            // Prefetched matrix masks: the leading tiles that lie entirely before the last key and before the causal
            // diagonal of the workgroup's first row take the short form of the masking code, in pairs over the two
            // stages like the clean tiles of the other mask modes (there are no clean tiles with a matrix mask).
            bool odd = odd_clean;
            if (MATRIX && ROUTE != 0 && (D == 64 || !CAUSAL)) {  // head size 128, causal: no registers to spare for a second tile body
                const int n_fast = min(nt, CAUSAL ? min(N / BN, (q0 + p.causal_off + 1) / BN) : N / BN);
                for (; idx + 1 < n_fast; idx += 2) {
                    tile_step(BoolC<true>(), IntC<0>(), route_c, BoolC<false>(), BoolC<false>());
                    tile_step(BoolC<true>(), IntC<1>(), route_c, BoolC<false>(), BoolC<false>());
                }
                if (idx < n_fast) {
                    tile_step(BoolC<true>(), IntC<0>(), route_c, BoolC<false>(), BoolC<false>());
                    ++idx;
                    odd = true;
                }
            }
            if (odd && idx < nt) {
                tile_step(BoolC<true>(), IntC<1>(), route_c, BoolC<true>(), BoolC<false>());
                ++idx;
            }
            for (; idx < nt; idx += 2) {
                tile_step(BoolC<true>(), IntC<0>(), route_c, BoolC<true>(), BoolC<false>());
                if (idx + 1 < nt) tile_step(BoolC<true>(), IntC<1>(), route_c, BoolC<true>(), BoolC<false>());
            }
            // the last step's request for another mask tile must have landed before the wave ends
            if (MATRIX && ROUTE >= 3) __builtin_amdgcn_s_waitcnt(0x0F70);
        };
        if (MASK_VIA_LDS && p.mask_fast == 2 && m_f32) general_tiles(IntC<3>());
        else if (MASK_VIA_LDS && p.mask_fast == 2) general_tiles(IntC<4>());
        else if (MATRIX && m_fast && m_f32) general_tiles(IntC<2>());
        else if (MATRIX && m_fast) general_tiles(IntC<1>());
        else general_tiles(IntC<0>());
    }

    if constexpr (WSPLIT) {
        // ---- the four waves hold partial results for the SAME 32 rows, each relative to a reference of its own: the
        // row's exponent reference if the wave has seen an ordinary score (class 2), the reference of its masked scores
        // if it has only seen those (class 1), nothing (class 0).  As inside a wave, ordinary keys discard masked ones.
        // Every wave leaves its triple in its own (now idle) stages; wave w then merges accumulator registers
        // 8 w .. 8 w + 7 of all four — 8 consecutive features of the row — and stores them.
        constexpr int XO = 32 * 64;  // floats of an accumulator image: [register][lane]
        float *mine = reinterpret_cast<float *>(smem + wave_lds);
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int v = 0; v < 16; ++v) mine[(d * 16 + v) * 64 + lane] = o_acc[d][v];
        mine[XO + lane] = fresh ? m_masked : m_i;
        mine[XO + 64 + lane] = halves32_sum(l_i);
        mine[XO + 128 + lane] = !fresh ? 2.0f : (m_masked > -INFINITY ? 1.0f : 0.0f);
        __syncthreads();
        float ref[4], sum[4], cls[4];
        float top = 0.0f;
#pragma unroll
        for (int z = 0; z < 4; ++z) {
            const float *part = reinterpret_cast<const float *>(smem + z * (2 * STAGE));
            ref[z] = part[XO + lane];
            sum[z] = part[XO + 64 + lane];
            cls[z] = part[XO + 128 + lane];
            top = fmaxf(top, cls[z]);
        }
        float m_all = -INFINITY;
#pragma unroll
        for (int z = 0; z < 4; ++z)
            if (cls[z] == top) m_all = fmaxf(m_all, ref[z]);
        float wgt[4], l_all = 0.0f;
#pragma unroll
        for (int z = 0; z < 4; ++z) {
            wgt[z] = (cls[z] == top && top > 0.0f) ? __builtin_amdgcn_exp2f(ref[z] - m_all) : 0.0f;
            l_all = fmaf(wgt[z], sum[z], l_all);
        }
        const float inv = 1.0f / l_all;
        float r[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float a = 0.0f;
#pragma unroll
            for (int z = 0; z < 4; ++z)
                a = fmaf(wgt[z], reinterpret_cast<const float *>(smem + z * (2 * STAGE))[(8 * wave + e) * 64 + lane], a);
            r[e] = a * inv;
        }
        if (my_m < M) {
            // registers 8 w .. 8 w + 7 = block d = w / 2, elements 8 (w % 2) ..: features 32 d + 16 lh + 8 (w % 2) .. + 7
            u32x4 pk;
#pragma unroll
            for (int j = 0; j < 4; ++j) pk[j] = pack2<T>(r[2 * j], r[2 * j + 1]);
            *reinterpret_cast<u32x4 *>(op + (int64_t)my_m * p.os[2] + (wave >> 1) * 32 + lh * 16 + (wave & 1) * 8) = pk;
        }
        return;
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
    const int n_end = causal ? min(p.N, m + 1 + p.causal_off) : p.N;
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
template <typename T, int D, int WPE>
static void launch_stream(const AttnParams &p, int mask_mode, bool causal, hipStream_t st) {
    const int bh_padded = (mask_mode == MASK_MATRIX && p.xcd_by_batch) ? ((p.B + 7) / 8) * 8 * p.H : ((p.B * p.H + 7) / 8) * 8;
    dim3 grid((unsigned)(bh_padded * p.nq_tiles)), block(256);
#define KERNL_ATTN_LAUNCH(MM, C) hipLaunchKernelGGL((attention_stream_kernel<T, D, WPE, MM, C>), grid, block, 0, st, p)
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

// small grids, head size 64: 32-row workgroups whose waves split the key tiles (the kernel's WSPLIT form)
template <typename T>
static void launch_stream_wsplit(AttnParams p, int mask_mode, hipStream_t st) {
    constexpr int LDS_BYTES = 8 * (2 * 64 * 128 + 64 * 4);  // 4 waves x 2 stages of a K tile, a V tile and 64 per-key terms
    p.nq_tiles = (p.M + 31) / 32;
    dim3 grid((unsigned)(p.B * p.H * p.nq_tiles)), block(256);
    auto k_none = attention_stream_kernel<T, 64, 1, MASK_NONE, false, false, true>;
    auto k_vec = attention_stream_kernel<T, 64, 1, MASK_VECTOR, false, false, true>;
    static bool attr_done = false;  // benign race: the attribute calls are idempotent
    if (!attr_done) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(k_none), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        (void)hipFuncSetAttribute(reinterpret_cast<const void *>(k_vec), hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        attr_done = true;
    }
    if (mask_mode == MASK_NONE) hipLaunchKernelGGL(k_none, grid, block, LDS_BYTES, st, p);
    else hipLaunchKernelGGL(k_vec, grid, block, LDS_BYTES, st, p);
}

// one-byte keys and values: fp16 queries, no mask or a per-key mask
template <int D>
static void launch_stream_kv8(const AttnParams &p, int mask_mode, bool causal, hipStream_t st) {
    const int bh_padded = ((p.B * p.H + 7) / 8) * 8;
    dim3 grid((unsigned)(bh_padded * p.nq_tiles)), block(256);
#define KERNL_ATTN_LAUNCH8(MM, C) hipLaunchKernelGGL((attention_stream_kernel<f16, D, 2, MM, C, true>), grid, block, 0, st, p)
    if (mask_mode == MASK_NONE) {
        if (causal) KERNL_ATTN_LAUNCH8(MASK_NONE, true);
        else KERNL_ATTN_LAUNCH8(MASK_NONE, false);
    } else {
        if (causal) KERNL_ATTN_LAUNCH8(MASK_VECTOR, true);
        else KERNL_ATTN_LAUNCH8(MASK_VECTOR, false);
    }
#undef KERNL_ATTN_LAUNCH8
}

int g_attention_force_scalar = 0;  // test hook: route everything through the scalar kernel
int g_attention_variant = 0;       // tuning hook: register budget (waves per SIMD) of the head-size-64 MFMA kernel

}  // namespace kernl

extern "C" void kernl_attention_force_scalar(int on) { kernl::g_attention_force_scalar = on; }
extern "C" void kernl_attention_set_variant(int which) { kernl::g_attention_variant = which; }

static int attention_entry(const void *q, const void *k, const void *v, void *out, const void *mask,
                           int64_t B, int64_t H, int64_t M, int64_t N, int64_t D,
                           const int64_t q_strides[4], const int64_t k_strides[4],
                           const int64_t v_strides[4], const int64_t o_strides[4],
                           const int64_t mask_sizes[4], const int64_t mask_strides[4], int mask_dtype,
                           float sm_scale, int is_causal, int64_t start_position, float mask_min_clamp, int dtype,
                           void *stream, bool kv8 = false) {
    using namespace kernl;
    if (start_position < 0 || start_position > (1 << 24))
        return set_error(KERNL_ERR_INVALID_ARG, "attention: start_position %lld out of range", (long long)start_position);
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
    p.mask_fast = 0;
    p.xcd_by_batch = 0;
    p.causal_off = is_causal != 0 ? (int)start_position : 0;
    if (mask_mode == MASK_MATRIX && (mask_dtype == KERNL_F32 || mask_dtype == dtype)) {
        const int64_t es = mask_dtype == KERNL_F32 ? 4 : 2;
        p.mask_fast = mask_strides[3] == 1 && p.ms[0] % 4 == 0 && p.ms[1] % 4 == 0 && p.ms[2] % 4 == 0 && p.ms[2] > 0 &&
                      aligned16(mask) && ((M - 1) * p.ms[2] + N + 128) * es < (1ll << 31);
        const int64_t chunk = 16 / es;  // elements per 16 bytes
        if (p.mask_fast && p.ms[0] % chunk == 0 && p.ms[1] % chunk == 0 && p.ms[2] % chunk == 0) p.mask_fast = 2;
        // broadcast over heads but not over the batch: the mask outweighs K and V, map workgroups by batch entry
        p.xcd_by_batch = p.ms[1] == 0 && p.ms[0] != 0 && H > 1;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool causal = is_causal != 0;

    auto rows_ok = [](const void *ptr, const int64_t s[4]) {
        return s[3] == 1 && s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0 && aligned16(ptr);
    };
    const bool mfma_ok = !g_attention_force_scalar && (D == 64 || D == 128) && sm_scale > 0.0f &&
                         rows_ok(q, q_strides) && rows_ok(k, k_strides) && rows_ok(v, v_strides) &&
                         rows_ok(out, o_strides) && (int64_t)((B + 7) / 8) * 8 * H * p.nq_tiles < (1ll << 31) &&
                         k_strides[2] > 0 && v_strides[2] > 0 &&  // one head's K / V extent must fit 31-bit byte offsets
                         (N + 128) * k_strides[2] < (1ll << 30) && (N + 128) * v_strides[2] < (1ll << 30) &&
                         (mask == nullptr || (mask_strides[3] >= 0 && (N + 128) * mask_strides[3] < (1ll << 30)));
    if (kv8) {
        // one-byte keys and values only exist on the MFMA kernel: no scalar route, no matrix masks
        if (dtype != KERNL_F16)
            return set_error(KERNL_ERR_UNSUPPORTED, "attention (fp8 keys/values): queries and output must be f16, got dtype %d", dtype);
        if (mask_mode == MASK_MATRIX)
            return set_error(KERNL_ERR_UNSUPPORTED, "attention (fp8 keys/values): only per-key masks are supported");
        if (!mfma_ok)
            return set_error(KERNL_ERR_UNSUPPORTED, "attention (fp8 keys/values): head size 64 or 128, unit feature strides, "
                             "strides that are multiples of 8 and 16-byte aligned bases are required");
        if (D == 64) launch_stream_kv8<64>(p, mask_mode, causal, st);
        else launch_stream_kv8<128>(p, mask_mode, causal, st);
        return check_launch("attention (mfma, fp8 keys/values)");
    }
    // Small grids (BERT-base at batch 1: 12 heads x 4 query tiles on 256 CUs, each walking all key tiles): 32-row
    // workgroups whose four waves split the key tiles, where that still is a single round of workgroups (one per CU:
    // 130 KB of LDS) and every wave gets a tile.  Measured over 4 .. 64 heads x 64 .. 1536 rows x 256 .. 2048 keys: ahead of
    // both other kernels wherever the grid is at most 256 workgroups ([1,12,512,64]: 9.8 -> 7.5 us, [1,16,512,2048]:
    // 28.0 -> 15.1), behind from the second round on.  (Hook: variant 5 takes this form wherever it applies, 3 and 4 never.)
    {
        const int64_t wgs32 = B * H * ((M + 31) / 32);
        const bool applies = mfma_ok && D == 64 && !causal && mask_mode != MASK_MATRIX && N <= 64 * 64;
        const bool pays = N >= 256 && wgs32 <= 224;  // (at 256 the pipelined kernel, which takes such grids next, draws level)
        if (applies && g_attention_variant != 3 && g_attention_variant != 4 && (pays || g_attention_variant == 5)) {
            if (dtype == KERNL_F16) launch_stream_wsplit<f16>(p, mask_mode, st);
            else launch_stream_wsplit<bf16>(p, mask_mode, st);
            return check_launch("attention (mfma, key tiles split over waves)");
        }
    }
    // the software-pipelined kernel takes long key sequences of what it covers (hook: variant 3 keeps everything on the
    // streaming kernel, variant 4 sends everything the pipelined kernel covers to it)
    if (mfma_ok && g_attention_variant != 3 &&
        launch_attention_pipe(p, (int)D, dtype, mask_mode, causal, g_attention_variant == 4, st))
        return check_launch("attention (pipelined mfma)");
    if (mfma_ok) {
        // head size 64 without a matrix mask fits the register budget of 3 waves per SIMD (168 VGPRs); the
        // matrix-mask body (mask values prefetched in registers) and head size 128 run at 2 waves per SIMD.
        int wpe = (D == 64 && mask_mode != MASK_MATRIX) ? 3 : 2;
        if (D == 64 && g_attention_variant == 1) wpe = 3;
        if (D == 64 && g_attention_variant == 2) wpe = 2;
        if (dtype == KERNL_F16) {
            if (D == 64 && wpe == 3) launch_stream<f16, 64, 3>(p, mask_mode, causal, st);
            else if (D == 64) launch_stream<f16, 64, 2>(p, mask_mode, causal, st);
            else launch_stream<f16, 128, 2>(p, mask_mode, causal, st);
        } else {
            if (D == 64 && wpe == 3) launch_stream<bf16, 64, 3>(p, mask_mode, causal, st);
            else if (D == 64) launch_stream<bf16, 64, 2>(p, mask_mode, causal, st);
            else launch_stream<bf16, 128, 2>(p, mask_mode, causal, st);
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

extern "C" int kernl_attention_fwd(const void *q, const void *k, const void *v, void *out, const void *mask,
                                   int64_t B, int64_t H, int64_t M, int64_t N, int64_t D,
                                   const int64_t q_strides[4], const int64_t k_strides[4],
                                   const int64_t v_strides[4], const int64_t o_strides[4],
                                   const int64_t mask_sizes[4], const int64_t mask_strides[4], int mask_dtype,
                                   float sm_scale, int is_causal, float mask_min_clamp, int dtype, void *stream) {
    return attention_entry(q, k, v, out, mask, B, H, M, N, D, q_strides, k_strides, v_strides, o_strides, mask_sizes,
                           mask_strides, mask_dtype, sm_scale, is_causal, 0, mask_min_clamp, dtype, stream);
}

extern "C" int kernl_attention_cached_fwd(const void *q, const void *k, const void *v, void *out, const void *mask,
                                          int64_t B, int64_t H, int64_t M, int64_t N, int64_t D,
                                          const int64_t q_strides[4], const int64_t k_strides[4],
                                          const int64_t v_strides[4], const int64_t o_strides[4],
                                          const int64_t mask_sizes[4], const int64_t mask_strides[4], int mask_dtype,
                                          float sm_scale, int64_t start_position, float mask_min_clamp, int dtype,
                                          void *stream) {
    return attention_entry(q, k, v, out, mask, B, H, M, N, D, q_strides, k_strides, v_strides, o_strides, mask_sizes,
                           mask_strides, mask_dtype, sm_scale, 1, start_position, mask_min_clamp, dtype, stream);
}

extern "C" int kernl_attention_kv8_fwd(const void *q, const void *k8, const void *v8, void *out, const void *mask,
                                       int64_t B, int64_t H, int64_t M, int64_t N, int64_t D,
                                       const int64_t q_strides[4], const int64_t k_strides[4],
                                       const int64_t v_strides[4], const int64_t o_strides[4],
                                       const int64_t mask_sizes[4], const int64_t mask_strides[4], int mask_dtype,
                                       float sm_scale, int is_causal, int64_t start_position, float mask_min_clamp,
                                       int dtype, void *stream) {
    return attention_entry(q, k8, v8, out, mask, B, H, M, N, D, q_strides, k_strides, v_strides, o_strides, mask_sizes,
                           mask_strides, mask_dtype, sm_scale, is_causal, is_causal ? start_position : 0, mask_min_clamp,
                           dtype, stream, true);
}
