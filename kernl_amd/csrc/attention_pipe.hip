// Flash-attention forward for gfx950, software-pipelined form:  out = softmax(q·kᵀ·scale + causal + mask) · v.
//
// Semantics as in attention.hip (reference kernel src/kernl/implementations/attention.py:122-435: fp32 scores and
// accumulators, additive mask with -inf clamped to a finite minimum, top-left aligned causal masking, online softmax
// over key tiles, P rounded to the input dtype before P·V).
//
// What is different from the streaming kernel of attention.hip is the instruction stream of a wave.  Measured on this
// chip, ONE wave that interleaves 1 MFMA (32x32x16) : 2 v_exp_f32 : 2 plain VALU instructions runs at the speed of
// its MFMAs alone (537 cycles for 16 + 32 + 32 against 521 for the MFMAs), while 4 plain instructions beside the 2
// exponentials cost 769, and a wave that first does its MFMAs and then its softmax runs at the sum of both.  So the
// loop is pipelined inside the wave over units of 32 keys (half a key tile): a unit computes, side by side and
// mutually independent,
//     the scores of the NEXT 32 keys                       (4 MFMAs, K tile from LDS),
//     the probabilities of THESE 32 keys from their scores  (16 v_exp_f32, 8 conversions to 16 bit, 8 row-sum steps),
//     the product P·V of the PREVIOUS 32 keys               (4 MFMAs, V tile from LDS),
// laid out by hand as one MFMA per slot with its share of the softmax work, pinned with scheduling barriers.
// To fit that budget the loop has NO row maximum and no rescaling: scores come out of the MFMA already relative
// to the row's exponent reference (its negative is the C operand), and the reference is the maximum of the row's
// first tile.  Probabilities of later tiles may exceed 1; as long as none exceeds the 16-bit range the final O / l is
// exact whatever the reference.  If one does, the accumulator holds infinities: the workgroup then redoes its rows
// with a plain loop that tracks the maximum (rare: a score must exceed the first tile's maximum by 16 in base-2 units).
// The row sum is two v_add_f32 per pair on the unrounded probabilities (as the reference sums them): v_dot2c_f32_f16
// on the packed pairs is one instruction less, but the dot unit shares the matrix pipe — 762 cycles per 16 MFMAs
// instead of 592.
//
// Data movement: K and V tiles go HBM -> LDS directly (buffer loads with the LDS flag) into rings of 4 slots each,
// requested two tiles ahead of their use; one workgroup barrier per tile.  Layouts and the transposed-score trick
// (Sᵀ = K·Qᵀ, a lane owns one query row; the packed probabilities already are the MFMA B operand of Oᵀ = Vᵀ·Pᵀ) are
// those of attention.hip.
//
// The grid is persistent (two workgroups per CU, each walking a fixed list of (batch, head, query tile) items): the
// next item's query rows, first K / V tiles and mask row are requested as soon as the ring is free — all of them
// into LDS (the query and mask rows into ring slots that are idle between two items) — and arrive while the finished
// item is normalised and stored.
//
// Where it is used: from 1024 keys on, where the pipelined stream is 4..16 % ahead of the streaming kernel.  Below that
// the fixed cost of an item weighs as much as its tile loop.  Cycle stamps at 512 keys (8 tiles, two workgroups per CU):
// about 18 000 cycles per item, of which the tile loop takes 9 700; the rest is the first tile's serial chain (2 800),
// the request of the next item (2 000 .. 3 000: some 180 scalar instructions of address arithmetic and 14 .. 22
// tile-sized loads, executed by all eight waves of the CU at once), the tile classification of a per-key mask (2 500),
// the store (1 200), the overflow vote (700) and waits.  Every wave runs such serial code at about ten cycles per
// instruction, so the count of instructions outside the loop is what is left to cut; running one item per workgroup
// under the hardware's own dispatch measures the same as the persistent grid (36.8 us either way at [32,12,512,64]).
#include "attention_common.h"

#ifndef KERNL_ATTN_PIPE_LOOKAHEAD
#define KERNL_ATTN_PIPE_LOOKAHEAD 4
#endif

namespace kernl {

template <typename T, int D, int MASK_MODE, bool CAUSAL>
__global__ void __launch_bounds__(256, D == 64 ? 2 : 1) attention_pipe_kernel(const AttnParams p) {
    typedef typename Vec8<T>::type vec8;
    typedef __attribute__((address_space(3))) void lds_void;
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    static_assert(D == 64 || D == 128, "head size 64 (two workgroups per CU) or 128 (one: the rings take 128 KB of LDS)");
    constexpr int BM = 128, BN = 64, NS = 4;
    typedef AttnTileMap<D> TileMap;                      // staging and fragment addresses of a K / V tile (index_math.h)
    constexpr int KROW = D * 2, VP = D * 2;              // LDS row bytes of the K tile [key][D] and V tile [key][D]
    constexpr int K_BYTES = BN * KROW, V_BYTES = BN * VP;
    constexpr int DB = D / 32, KS = D / 16;
    constexpr int DC = D / 8;                            // 16-byte chunks per K/V row
    constexpr int KI = BN * DC / 256;                    // 1 KB loads per wave for each of K and V
    constexpr int V_RING = NS * K_BYTES;
    constexpr int BIAS_OFF = NS * (K_BYTES + V_BYTES);
    constexpr bool VEC = (MASK_MODE == MASK_VECTOR);
    constexpr int BIAS_KEYS = VEC ? kPipeMaxMaskKeys : 0;
    constexpr int PER = VEC ? BIAS_KEYS / 256 : 1;       // keys of a mask row per thread
    static_assert(!(VEC && CAUSAL), "per-key masks with causal masking take the streaming kernel");
    static_assert(KI * 4096 == K_BYTES && K_BYTES == V_BYTES, "a tile is KI loads of 1 KB per wave");
    // What an item needs before its first tile is PREFETCHED INTO LDS, into ring slots that are idle between two items
    // (the next item's first tiles only take K slots 0..2 and V slots 0..1):
    //   query rows   V ring slots 2 and 3: wave w keeps its 32 rows at Q_STAGE + w * KS KB, lane l's fragment s at
    //                + s KB + 16 l — every lane reads back exactly what its own load wrote;
    //   mask row     K ring slot 3, one dword per key (16-bit masks: the value in the low half).  Rows of up to
    //                64 * PER keys are fetched by EVERY wave into a quarter of the slot of its own; longer rows once,
    //                shared out over the four waves.
    // Nothing the compiler knows as a register is pending between request and use (an earlier form kept these loads'
    // destination registers live across the previous item's epilogue; the register allocator was free to copy them
    // before the wait that made them valid, and one build did).
    constexpr int Q_STAGE = V_RING + 2 * V_BYTES, MASK_STAGE = 3 * K_BYTES;
    constexpr int WAVE_ROW_KEYS = 64 * PER;  // 512: longest mask row a single wave classifies by itself
    static_assert(KS * 1024 * 4 <= 2 * V_BYTES, "the four waves' query rows fit two V ring slots");
    static_assert(!VEC || (kPipeMaxMaskKeys * 4 <= K_BYTES && WAVE_ROW_KEYS * 4 * 4 <= K_BYTES), "a mask row fits K ring slot 3");
    typedef BoolC<true> Yes;
    typedef BoolC<false> No;

    // head size 64 fits the 64 KB a kernel may declare; head size 128 takes its 128 KB of rings as dynamic LDS
    constexpr int LDS_BYTES = BIAS_OFF + BIAS_KEYS * 4 + 96;
    __shared__ __attribute__((aligned(16))) unsigned char smem_fixed[D == 64 ? LDS_BYTES : 16];
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_dynamic[];
    unsigned char *const smem = D == 64 ? smem_fixed : smem_dynamic;
    float *bias_lds = reinterpret_cast<float *>(smem + BIAS_OFF);  // additive terms of the item's keys (see the classification)
    int *vote_lds = reinterpret_cast<int *>(smem + BIAS_OFF + BIAS_KEYS * 4 + 16);  // 4 ints: per-wave overflow votes

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 31, lh = lane >> 5;
    const int M = p.M, N = p.N;
    const bool wave_rows = VEC && N <= WAVE_ROW_KEYS;
    const int bias_wave = wave_rows ? wave * WAVE_ROW_KEYS : 0;  // short rows: every wave keeps the terms in a copy of its own
    auto uniform = [](uint32_t x) __attribute__((always_inline)) -> uint32_t { return (uint32_t)__builtin_amdgcn_readfirstlane((int)x); };

    // ---- the work of this workgroup.  The grid is persistent: 8 W workgroups, W per XCD (workgroup ids are dealt
    // round-robin to the XCDs by hardware).  XCD x owns the (batch, head) pairs bh = x, x + 8, ...; its items are
    // (pair, query tile) with the query tiles of a pair next to each other, so that the workgroups working on one
    // pair at the same time share its K and V through that XCD's L2.  Workgroup j of the XCD takes item j of every
    // round of W items, in alternating direction (the long and the short query tiles of causal attention pair up).
    const int xcd = blockIdx.x & 7, wg_j = blockIdx.x >> 3, wg_w = gridDim.x >> 3;
    const int bh_total = p.B * p.H;
    const int n_items = (xcd < bh_total) ? ((bh_total - xcd + 7) / 8) * p.nq_tiles : 0;
    auto item_of_round = [&](int r) __attribute__((always_inline)) -> int {
        const int idx = r * wg_w + ((r & 1) ? wg_w - 1 - wg_j : wg_j);
        return idx < n_items ? idx : -1;
    };
    int round = 0;
    int item = item_of_round(0);
    if (item < 0) return;

    // ---- staging (as in attention.hip): the i-th load of a wave fills the 1 KB of 16-byte chunks
    // [256 i + 64 wave, +64) of a tile; every lane fetches the chunk of global memory that belongs at its LDS
    // position under the tile's swizzle.  Rows past the last key lie beyond the buffer resource and arrive as zeros.
    uint32_t kdma[KI], vdma[KI];
#pragma unroll
    for (int i = 0; i < KI; ++i) {
        const int qd = tid + 256 * i;
        const int row = TileMap::stage_row(qd);
        kdma[i] = (uint32_t)(((int64_t)row * p.ks[2] + TileMap::k_stage_chunk(qd) * 8) * 2);
        vdma[i] = (uint32_t)(((int64_t)row * p.vs[2] + TileMap::v_stage_chunk(qd) * 8) * 2);
    }
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void *)smem;
    const uint32_t dma_base = lds_base + wave * 1024;
    const int k_tile_bytes = (int)((int64_t)BN * p.ks[2] * 2), v_tile_bytes = (int)((int64_t)BN * p.vs[2] * 2);
    const uint32_t k_extent = (uint32_t)((((int64_t)N - 1) * p.ks[2] + D) * 2), v_extent = (uint32_t)((((int64_t)N - 1) * p.vs[2] + D) * 2);
    // Inline assembly on purpose: the compiler, seeing LDS written by a load, would make every later LDS read wait
    // for the vector-memory counter, i.e. for the prefetches themselves.  The explicit counter waits before the
    // barrier of each step are the ones that matter.
    auto dma_tile = [&](uint64_t base_addr, uint32_t extent, const uint32_t (&lane_off)[KI], uint32_t soff_bytes, uint32_t lds_dst) __attribute__((always_inline)) {
        const u32x4 rsrc = {uniform((uint32_t)base_addr), uniform((uint32_t)(base_addr >> 32) & 0xFFFFu), uniform(extent), 0x00020000u};
        const uint32_t soff = uniform(soff_bytes), sb = uniform(lds_dst);
#pragma unroll
        for (int i = 0; i < KI; ++i)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :: "s"(sb + i * 4096), "v"(lane_off[i]), "s"(rsrc), "s"(soff) : "memory", "m0");
    };

    // LDS byte offsets of this lane's operand fragments (see attention.hip)
    int k_off[KS], vt_off[DB];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_off[ks] = TileMap::k_frag_offset(lr, lh, ks);
#pragma unroll
    for (int d = 0; d < DB; ++d) vt_off[d] = V_RING + TileMap::v_frag_offset(lane, d);
    auto k_frag = [&](int ring_slot, int half, int ks) __attribute__((always_inline)) -> vec8 {
        return *reinterpret_cast<const vec8 *>(smem + ring_slot * K_BYTES + half * 32 * KROW + k_off[ks]);
    };
    auto v_frag = [&](int ring_slot, int ps, int d) __attribute__((always_inline)) -> vec8 {
        const unsigned char *va = smem + ring_slot * V_BYTES + 16 * ps * VP + vt_off[d];
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)va);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(va + 8 * VP));
        return __builtin_bit_cast(vec8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };

    // ---- what an item needs before its first tile, requested as early as possible (for the first item here, for
    // every later one while the previous item finishes): the query rows, the first K and V tiles in natural order
    // (what a mask that pads on the right ends up with; another order re-requests them), the mask row.
    //   ring requests:  K(0), V(0), K(1), K(2), V(1)   — step t then requests K(t+3) and V(t+2)
    uint64_t kaddr = 0, vaddr = 0;  // of the item whose tiles are being requested
    // (batch, head, first query row, key tiles up to the causal bound) of the item being computed and of the requested one
    int cur_b = 0, cur_h = 0, cur_q0 = 0, cur_nt_all = 0, req_b = 0, req_h = 0, req_q0 = 0, req_nt_all = 0;
    auto set_kv = [&](int b, int h) __attribute__((always_inline)) {
        kaddr = (uint64_t)(uintptr_t)(static_cast<const T *>(p.k) + b * p.ks[0] + h * p.ks[1]);
        vaddr = (uint64_t)(uintptr_t)(static_cast<const T *>(p.v) + b * p.vs[0] + h * p.vs[1]);
    };
    auto dma_k = [&](int tile, int ring_slot) __attribute__((always_inline)) {
        dma_tile(kaddr, k_extent, kdma, (uint32_t)(tile * k_tile_bytes), dma_base + ring_slot * K_BYTES);
    };
    auto dma_v = [&](int tile, int ring_slot) __attribute__((always_inline)) {
        dma_tile(vaddr, v_extent, vdma, (uint32_t)(tile * v_tile_bytes), dma_base + V_RING + ring_slot * V_BYTES);
    };
    auto request_first_tiles = [&](int t0, int t1, int t2) __attribute__((always_inline)) {
        dma_k(t0, 0);
        dma_v(t0, 0);
        dma_k(t1, 1);
        dma_k(t2, 2);
        dma_v(t1, 1);
    };
    // Query rows and mask row of the requested item -> their LDS staging areas (direct-to-LDS loads from inline assembly,
    // like the tile loads: the compiler would make every barrier wait for loads it knows of, and these are meant to stay
    // in flight across the barriers of the previous item's epilogue).
    auto request_staged = [&]() __attribute__((always_inline)) {
        const int my_m = req_q0 + wave * 32 + lr;
        const uint64_t qaddr = (uint64_t)(uintptr_t)(static_cast<const T *>(p.q) + req_b * p.qs[0] + req_h * p.qs[1]);
        const u32x4 qrsrc = {uniform((uint32_t)qaddr), uniform((uint32_t)(qaddr >> 32) & 0xFFFFu),
                             uniform((uint32_t)((((int64_t)M - 1) * p.qs[2] + D) * 2)), 0x00020000u};
        const uint32_t qoff = (uint32_t)(((int64_t)min(my_m, M - 1) * p.qs[2] + lh * 8) * 2);
        const uint32_t qdst = uniform(lds_base + Q_STAGE + wave * (KS * 1024));
#pragma unroll
        for (int s = 0; s < KS; ++s)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :: "s"(qdst + s * 1024), "v"(qoff), "s"(qrsrc), "s"(32 * s) : "memory", "m0");
        if (VEC) {
            // one value per key; keys past the end read as 0 through the bounds of the buffer resource and are set
            // to -inf afterwards
            const int es = p.mask_dtype == KERNL_F32 ? 4 : 2;
            const uint64_t maddr = (uint64_t)(uintptr_t)(static_cast<const char *>(p.mask) + (req_b * p.ms[0] + req_h * p.ms[1]) * es);
            const u32x4 mrsrc = {uniform((uint32_t)maddr), uniform((uint32_t)(maddr >> 32) & 0xFFFFu),
                                 uniform((uint32_t)(((int64_t)(N - 1) * p.ms[3] + 1) * es)), 0x00020000u};
            const int step_bytes = (int)p.ms[3] * es;
            // load i of a wave covers 64 consecutive keys, lane l the key first + l, written to LDS as dword first + l
            const int first = wave_rows ? 0 : 64 * wave, step = wave_rows ? 64 : 256;
            const uint32_t mdst = uniform(lds_base + MASK_STAGE + (wave_rows ? wave * (WAVE_ROW_KEYS * 4) : 64 * 4 * wave));
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                if (first + step * i < N) {  // wave-uniform
                    if (p.mask_dtype == KERNL_F32)
                        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds"
                                     :: "s"(mdst + step * 4 * i), "v"((first + step * i + lane) * step_bytes), "s"(mrsrc) : "memory", "m0");
                    else
                        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_ushort %1, %2, 0 offen lds"
                                     :: "s"(mdst + step * 4 * i), "v"((first + step * i + lane) * step_bytes), "s"(mrsrc) : "memory", "m0");
                }
            }
        }
    };
    auto request_item = [&](int idx) __attribute__((always_inline)) {
        const int bh = 8 * (idx / p.nq_tiles) + xcd, qt = idx % p.nq_tiles;
        req_b = bh / p.H;
        req_h = bh % p.H;
        req_q0 = (CAUSAL ? p.nq_tiles - 1 - qt : qt) * BM;
        const int n_end = CAUSAL ? min(N, req_q0 + BM + p.causal_off) : N;
        req_nt_all = (n_end + BN - 1) / BN;
        set_kv(req_b, req_h);
        const int last = req_nt_all - 1;
        request_first_tiles(0, min(1, last), min(2, last));
        request_staged();
    };
    // one mask value as the classification sees it: the staged dword of key n decoded, scaled to the log2 domain with
    // -inf replaced by the clamp value, -inf past the last key
    auto staged_mask_value = [&](uint32_t raw, int n) __attribute__((always_inline)) -> float {
        float mv = __builtin_bit_cast(float, raw);
        if (p.mask_dtype != KERNL_F32) {
            const uint16_t bits = (uint16_t)raw;
            mv = p.mask_dtype == KERNL_F16 ? (float)__builtin_bit_cast(f16, bits) : (float)__builtin_bit_cast(bf16, bits);
        }
        return n < N ? scale_mask(mv, p.clamp) : -INFINITY;
    };
    request_item(item);
    auto lds_barrier = []() __attribute__((always_inline)) {  // LDS writes of this wave are done, then the workgroup barrier
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
        __builtin_amdgcn_s_barrier();
    };

    // ---- per item: tile order, running state
    uint32_t clean_bits = 0, gen_bits = 0;  // at most kPipeMaxMaskKeys / BN = 32 tiles; wave-uniform
    int first_tile = 0, nt = 0, n_clean = 0, order_pos = 1;
    // from the classes of all tiles (clean_bits, gen_bits; ord_bits = tiles holding a key whose term is 0): tile
    // counts and the first tile
    auto pick_first = [&](uint32_t ord_bits) __attribute__((always_inline)) {
        clean_bits = uniform(clean_bits);
        gen_bits = uniform(gen_bits);
        ord_bits = uniform(ord_bits);
        n_clean = __popc(clean_bits);
        nt = n_clean + __popc(gen_bits);
        if (n_clean == 0) {
            // no clean tile: the first tile must hold an ordinary key (it sets the exponent reference)
            uint32_t cand = gen_bits & ord_bits;
            if (cand == 0) cand = gen_bits;
            first_tile = __builtin_amdgcn_readfirstlane(__builtin_ctz(cand));
            gen_bits &= ~(1u << first_tile);
        } else {
            first_tile = __builtin_amdgcn_readfirstlane(__builtin_ctz(clean_bits));
            clean_bits &= clean_bits - 1;
        }
    };
    // The classes again, by one wave alone from the additive terms in LDS (the second pass over an item's tiles).
    auto classify_tiles = [&]() __attribute__((always_inline)) {
        const int npad = cur_nt_all * BN;
        uint32_t ord_bits = 0;
        clean_bits = 0;
        gen_bits = 0;
        for (int g = 0; g * 64 < npad; ++g) {
            const int n = g * 64 + lane;
            const float v = bias_lds[bias_wave + n];
            const bool valid = n < N;
            const bool any_nz = __ballot(valid && v != 0.0f) != 0, any_nm = __ballot(valid && v > kDeadMask) != 0,
                       any_ord = __ballot(valid && v == 0.0f) != 0;
            const bool full = g * 64 + 64 <= N;
            if (any_nm) {
                if (any_nz || !full) gen_bits |= 1u << g;
                else clean_bits |= 1u << g;
            }
            if (any_ord) ord_bits |= 1u << g;
        }
        pick_first(ord_bits);
    };
    auto next_tile = [&](int last) __attribute__((always_inline)) -> int {
        int t;
        if (VEC) {
            // branch-free on purpose (wave-uniform selects): clean tiles first, then general ones, then `last` again
            const uint32_t cb = clean_bits, gb = gen_bits;
            const uint32_t src = cb != 0 ? cb : gb;
            t = src != 0 ? (int)__builtin_ctz(src | 0x80000000u) : last;
            clean_bits = cb & (cb - 1);
            gen_bits = cb != 0 ? gb : (gb & (gb - 1));
        } else {
            t = min(order_pos, nt - 1);
        }
        ++order_pos;
        return __builtin_amdgcn_readfirstlane(t);
    };
    int tq[4];          // tiles at positions t .. t+3
    vec8 qf[KS];        // query fragments times scale * log2(e): the MFMA delivers base-2 scores
    float l_i, la, lb, ce0, ce1;
    f32x16 neg_m;
    f32x16 o_acc[DB];
    f32x16 Sa, Sb;      // scores of the lower / upper 32 keys of a tile
    u32x4 Pa[2], Pb[2]; // their packed probabilities
    int key_limit = 0;  // last key this lane's row may see (causal diagonal, end of the keys), minus the lane's own offset

    // masking of the scores of a general tile: pair e (0..7) of the lane's scores of the half `half`, in place
    auto mask_pair = [&](f32x16 &Sc, int e, int half, int n0) __attribute__((always_inline)) {
        const int v0 = 2 * e;
        const int c0 = 32 * half + 8 * (v0 / 4) + (v0 % 4);  // key of the first score of the pair, relative to n0 + 4 lh
        if (VEC) {
            const f32x2 cb = *reinterpret_cast<const f32x2 *>(bias_lds + bias_wave + n0 + c0 + lh * 4);
            Sc[v0] += cb[0];
            Sc[v0 + 1] += cb[1];
        } else {
            const int rel = key_limit - n0;
            if (c0 > rel) Sc[v0] = -INFINITY;
            if (c0 + 1 > rel) Sc[v0 + 1] = -INFINITY;
        }
    };

    // Operand fragments are read from LDS LA slots before the MFMA that consumes them, across unit and step
    // boundaries: F[m % LA] holds the fragment of slot m.
    // Slot m of a unit: even -> K fragment (ks = m / 2) of the unit's score half; odd -> V fragment (ps, d) of its P·V half.
    constexpr int LA = KERNL_ATTN_PIPE_LOOKAHEAD;
    constexpr int NSLOT = 2 * KS;     // MFMAs of a unit: KS for the scores of 32 keys, KS = 2 DB for P·V of 32 keys
    constexpr int SPP = NSLOT / 8;    // slots per pair of probabilities (a unit has 8 pairs)
    vec8 F[LA];
    auto slot_frag = [&](int m, int qk_slot, int qk_half, int pv_slot, int pv_half) __attribute__((always_inline)) -> vec8 {
        if ((m & 1) == 0) return k_frag(qk_slot, qk_half, m >> 1);
        return v_frag(pv_slot, 2 * pv_half + (m >> 1) / DB, (m >> 1) % DB);
    };

    // One unit of the pipeline: 8 slots, each with at most one MFMA, one pair of probabilities and the fragment read
    // for the slot LA later (of this unit or of the next one, whose ring slots and halves are the n* arguments).
    //   DO_QK  Snext = scores of 32 keys: K ring slot qk_slot, half qk_half           (MFMAs in the even slots)
    //   E      Pcur  = probabilities of the 32 keys whose scores are in Scur (half cur_half of the tile at n0)
    //   DO_PV  o_acc += V(ring slot pv_slot, half pv_half) · Pprev                     (MFMAs in the odd slots)
    // The softmax chain of a pair of scores is spread over two slots: the exponentials in the pair's own slot, the
    // row-sum additions and the conversion in the next one (of the next unit for the last pair: ce0 / ce1 carry it
    // over), in the order  MFMA, reads, exp, add, exp, add, cvt  — measured per 16 MFMAs of one wave: 592 cycles this
    // way, 762 or more with the row sum on v_dot2c_f32_f16 wherever it is placed (the dot unit shares the matrix
    // pipe), 1100 with the exponentials last in the slot.
#define KERNL_SB __builtin_amdgcn_sched_barrier(0)
    auto unit = [&](f32x16 &Scur, u32x4 (&Pcur)[2], f32x16 &Snext, u32x4 (&Pprev)[2], auto doqk_c, auto general_c, auto carry_c,
                    int qk_slot, int qk_half, int pv_slot, int pv_half, int nqk_slot, int nqk_half, int npv_slot, int npv_half,
                    int n0, int cur_half) __attribute__((always_inline)) {
        constexpr bool DO_QK = decltype(doqk_c)::value, GENERAL = decltype(general_c)::value, HAS_CARRY = decltype(carry_c)::value;
#pragma unroll
        for (int m = 0; m < NSLOT; ++m) {
            if ((m & 1) == 0) {
                if (DO_QK) Snext = mfma32(F[m % LA], qf[m >> 1], m == 0 ? neg_m : Snext);
            } else {
                o_acc[(m >> 1) % DB] = mfma32(F[m % LA], __builtin_bit_cast(vec8, Pprev[(m >> 1) / DB]), o_acc[(m >> 1) % DB]);
            }
            KERNL_SB;
            if (m + LA < NSLOT) F[m % LA] = slot_frag(m + LA, qk_slot, qk_half, pv_slot, pv_half);
            else F[m % LA] = slot_frag(m + LA - NSLOT, nqk_slot, nqk_half, npv_slot, npv_half);
            KERNL_SB;
            if (m % SPP == 0) {
                const int e = m / SPP;  // pair of probabilities handled in this slot
                if (GENERAL) mask_pair(Scur, e, cur_half, n0);
                const float e0 = __builtin_amdgcn_exp2f(Scur[2 * e]);
                KERNL_SB;
                if (e > 0 || HAS_CARRY) la += ce0;
                KERNL_SB;
                const float e1 = __builtin_amdgcn_exp2f(Scur[2 * e + 1]);
                KERNL_SB;
                if (e > 0 || HAS_CARRY) {
                    lb += ce1;
                    KERNL_SB;
                    const uint32_t pk = pack2<T>(ce0, ce1);
                    if (e == 0) Pprev[1][3] = pk;
                    else Pcur[(e - 1) / 4][(e - 1) % 4] = pk;
                }
                ce0 = e0;
                ce1 = e1;
                KERNL_SB;
            }
        }
    };

    // Step t >= 1 (ts = t % 4):  request K(t+3), V(t+2);
    //   unit A: scores of (t, upper half), probabilities of (t, lower half), P·V of (t-1, upper half);
    //   unit B: scores of (t+1, lower half) unless t is the last position, probabilities of (t, upper), P·V of (t, lower);
    // the unit after B is unit A of step t+1 (or, after the last position, the P·V of its upper half, whose fragments
    // sit in the odd slots just the same).
    auto step = [&](int ts, auto general_c, auto last_c) __attribute__((always_inline)) {
        constexpr bool LAST = decltype(last_c)::value;
        const int n0 = tq[0] * BN;
        if (!LAST) {
            dma_k(tq[3], (ts + 3) & 3);
            dma_v(tq[2], (ts + 2) & 3);
        }
        const int k1 = (ts + 1) & 3, v3 = (ts + 3) & 3;
        unit(Sa, Pa, Sb, Pb, Yes(), general_c, Yes(), ts, 1, v3, 1, k1, 0, ts, 0, n0, 0);
        if (LAST) unit(Sb, Pb, Sa, Pa, No(), general_c, Yes(), k1, 0, ts, 0, k1, 1, ts, 1, n0, 1);
        else unit(Sb, Pb, Sa, Pa, Yes(), general_c, Yes(), k1, 0, ts, 0, k1, 1, ts, 1, n0, 1);
        // this wave's part of K(t+2) and V(t+1) has landed (only this step's requests may still be in flight); after
        // the barrier everybody's has, and nobody reads the ring slots any more that the next step's requests overwrite
        if (!LAST) __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * KI));  // vmcnt(2 KI): all but the requests of this step
        else __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int j = 0; j < 3; ++j) tq[j] = tq[j + 1];
        tq[3] = next_tile(tq[3]);
    };

    for (;;) {
        // ================= the item's tile order =================
        cur_b = req_b;
        cur_h = req_h;
        cur_q0 = req_q0;
        cur_nt_all = req_nt_all;
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's share of everything requested for the item has landed
        // this wave's query rows (and, for short mask rows, its copy of the mask row) leave the staging areas before the
        // barrier: after it any wave may request tiles into those ring slots
        vec8 q_raw[KS];
        {
            const unsigned char *qs = smem + Q_STAGE + wave * (KS * 1024) + lane * 16;
#pragma unroll
            for (int s = 0; s < KS; ++s) q_raw[s] = *reinterpret_cast<const vec8 *>(qs + s * 1024);
        }
        uint32_t mraw[PER];
        if (VEC && wave_rows) {
            const uint32_t *ms = reinterpret_cast<const uint32_t *>(smem + MASK_STAGE) + wave * WAVE_ROW_KEYS + lane;
#pragma unroll
            for (int i = 0; i < PER; ++i) mraw[i] = ms[64 * i];
#pragma unroll
            for (int i = 0; i < PER; ++i) asm volatile("" : "+v"(mraw[i]));  // the reads are done with before the barrier
        }
#pragma unroll
        for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(q_raw[s]));
        // all four waves' parts of the first tiles (and of a shared mask row) have landed: every wave waited for
        // everything it had requested
        lds_barrier();
        nt = cur_nt_all;
        n_clean = 0;
        first_tile = 0;
        order_pos = 1;
        bool zero_q = false;
        // Per-key masks.  Additive terms of all keys (log2 domain, -inf past the last key), relative to the largest one:
        // softmax does not change when every key's term moves by the same amount, and this way some key is always
        // "ordinary" (term 0), so the exponent reference set by the first tile is an ordinary score.  When even the
        // largest term is a clamped -inf, fp32 scores would have absorbed q·k entirely: q is dropped, which gives the
        // plain average of V over those keys, as the reference does.
        // Tile classes from two ballots per tile (lane l looks at key 64 i + l of tile i): clean = full and all zero,
        // general = needs the masked body, neither = so negative everywhere that the tile contributes exactly 0.  Keys
        // past the end carry -inf: neither zero nor above the "contributes nothing" bound, so a tile that holds one
        // counts as non-zero — which is what a ragged tile must be — and a tile beyond the row sets no bit at all.
        if (VEC && wave_rows) {
            // every wave for itself, from registers: no exchange, no further barrier; the terms go to a copy of the
            // wave's own
            float mv[PER];
            float lmax = -INFINITY;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                mv[i] = staged_mask_value(mraw[i], lane + 64 * i);
                lmax = fmaxf(lmax, mv[i]);
            }
            const float bmax = wave_max(lmax);
            zero_q = bmax < kNegBig;
            uint32_t all_ord = 0;
            clean_bits = 0;
            gen_bits = 0;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                const float v = mv[i] - bmax;
                bias_lds[bias_wave + lane + 64 * i] = v;
                const uint64_t nz = __ballot(v != 0.0f), nm = __ballot(v > kDeadMask);
                const uint32_t bit = 1u << i;
                gen_bits |= (nm != 0 && nz != 0) ? bit : 0u;
                clean_bits |= (nm != 0 && nz == 0) ? bit : 0u;
                all_ord |= (nz != ~0ull) ? bit : 0u;
            }
            pick_first(all_ord);
        } else if (VEC) {
            // long rows: every wave walks the whole staged row twice (maximum, then terms and classes); tile i's terms
            // are written by wave i % 4, and a second barrier publishes them
            const uint32_t *ms = reinterpret_cast<const uint32_t *>(smem + MASK_STAGE) + lane;
            float lmax = -INFINITY;
            for (int i = 0; i < cur_nt_all; ++i) lmax = fmaxf(lmax, staged_mask_value(ms[64 * i], lane + 64 * i));
            const float bmax = wave_max(lmax);
            zero_q = bmax < kNegBig;
            uint32_t all_ord = 0;
            clean_bits = 0;
            gen_bits = 0;
            for (int i = 0; i < cur_nt_all; ++i) {
                const float v = staged_mask_value(ms[64 * i], lane + 64 * i) - bmax;
                if ((i & 3) == wave) bias_lds[lane + 64 * i] = v;
                const uint64_t nz = __ballot(v != 0.0f), nm = __ballot(v > kDeadMask);
                const uint32_t bit = 1u << i;
                gen_bits |= (nm != 0 && nz != 0) ? bit : 0u;
                clean_bits |= (nm != 0 && nz == 0) ? bit : 0u;
                all_ord |= (nz != ~0ull) ? bit : 0u;
            }
            pick_first(all_ord);
            lds_barrier();  // the terms are in LDS, and nobody reads the staged row any more
        } else {
            n_clean = CAUSAL ? min(N / BN, (cur_q0 + p.causal_off + 1) / BN) : N / BN;
            n_clean = min(n_clean, nt);
        }
        tq[0] = first_tile;
#pragma unroll
        for (int j = 1; j < 4; ++j) tq[j] = next_tile(tq[j - 1]);
        {
            const int last = cur_nt_all - 1;
            const bool natural = tq[0] == 0 && tq[1] == min(1, last) && tq[2] == min(2, last);
            if (!natural) {  // wave-uniform, and the same in every wave; nobody's natural-order request is still in flight
                request_first_tiles(tq[0], tq[1], tq[2]);
                __builtin_amdgcn_s_waitcnt(0x0F70);
                __builtin_amdgcn_s_barrier();
            }
        }
        key_limit = (CAUSAL ? min(N - 1, cur_q0 + wave * 32 + lr + p.causal_off) : N - 1) - lh * 4;
        if constexpr (std::is_same<T, f16>::value) {
            // q * c as two packed half-precision steps, q * c_hi + q * c_lo with c_hi = c rounded to 16 bits: 8 packed
            // instructions per 16 elements instead of unpack, multiply, repack (the second rounding is another half ulp)
            const f16 c_hi = (f16)p.scale_log2, c_lo = (f16)(p.scale_log2 - (float)c_hi);
            const f16 z_hi = zero_q ? (f16)0.0f : c_hi, z_lo = zero_q ? (f16)0.0f : c_lo;
            const f16x8 vhi = {z_hi, z_hi, z_hi, z_hi, z_hi, z_hi, z_hi, z_hi}, vlo = {z_lo, z_lo, z_lo, z_lo, z_lo, z_lo, z_lo, z_lo};
#pragma unroll
            for (int s = 0; s < KS; ++s) qf[s] = __builtin_elementwise_fma(q_raw[s], vlo, q_raw[s] * vhi);
        } else {
#pragma unroll
            for (int s = 0; s < KS; ++s)
#pragma unroll
                for (int e = 0; e < 8; ++e) qf[s][e] = from_float<T>(zero_q ? 0.0f : to_float(q_raw[s][e]) * p.scale_log2);
        }
        l_i = 0.0f;
        la = 0.0f;
        lb = 0.0f;
        ce0 = 0.0f;
        ce1 = 0.0f;
#pragma unroll
        for (int v = 0; v < 16; ++v) neg_m[v] = 0.0f;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int v = 0; v < 16; ++v) o_acc[d][v] = 0.0f;

        // ================= position 0: K(0) has landed -> scores (against a reference of 0), row maximum = the
        // row's reference, probabilities of the lower half; then the unit-B half of a step =================
        {
            vec8 fa[KS], fb[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                fa[ks] = k_frag(0, 0, ks);
                fb[ks] = k_frag(0, 1, ks);
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                Sa = mfma32(fa[ks], qf[ks], ks == 0 ? neg_m : Sa);
                Sb = mfma32(fb[ks], qf[ks], ks == 0 ? neg_m : Sb);
            }
            const int n0 = tq[0] * BN;
            if (n_clean == 0) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    mask_pair(Sa, e, 0, n0);
                    mask_pair(Sb, e, 1, n0);
                }
            }
            float mx = -INFINITY;
#pragma unroll
            for (int v = 0; v < 16; ++v) mx = fmaxf(mx, fmaxf(Sa[v], Sb[v]));
            mx = halves32_max(mx);  // the other half of every 32-key block lives in lane ^ 32
            if (mx == -INFINITY) mx = 0.0f;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                Sa[v] -= mx;
                Sb[v] -= mx;
                neg_m[v] = -mx;
            }
            float rs = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float e0 = __builtin_amdgcn_exp2f(Sa[2 * e]), e1 = __builtin_amdgcn_exp2f(Sa[2 * e + 1]);
                Pa[e / 4][e % 4] = pack2<T>(e0, e1);
                rs += e0 + e1;
            }
            l_i = rs;
            // K(1) and V(0) have landed too: every wave waited for all of the item's first requests before the barrier above
            // the first unit: scores of (1, lower half) if there is a position 1, probabilities of (0, upper), P·V of (0, lower)
#pragma unroll
            for (int m = 0; m < LA && m < NSLOT; ++m) F[m] = slot_frag(m, 1, 0, 0, 0);
            if (nt > 1) {
                dma_k(tq[3], 3);
                dma_v(tq[2], 2);
                unit(Sb, Pb, Sa, Pa, Yes(), No(), No(), 1, 0, 0, 0, 1, 1, 0, 1, n0, 1);
                __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * KI));  // vmcnt(2 KI): all but the requests of this step
            } else {
                unit(Sb, Pb, Sa, Pa, No(), No(), No(), 1, 0, 0, 0, 1, 1, 0, 1, n0, 1);
                __builtin_amdgcn_s_waitcnt(0x0F70);
            }
            __builtin_amdgcn_s_barrier();
#pragma unroll
            for (int j = 0; j < 3; ++j) tq[j] = tq[j + 1];
            tq[3] = next_tile(tq[3]);
        }
        // ================= positions 1 .. nt-1: clean ones (four at a time with compile-time ring slots, then one
        // at a time), general ones, and the last position without further scores =================
        int t = 1;
        if (nt > 1) {
            const int cend = min(n_clean, nt - 1);
            for (; t + 4 <= cend; t += 4) {
                step(1, No(), No());
                step(2, No(), No());
                step(3, No(), No());
                step(0, No(), No());
            }
            for (; t < cend; ++t) step(t & 3, No(), No());
            for (; t < nt - 1; ++t) step(t & 3, Yes(), No());
            if (t < n_clean) step(t & 3, No(), Yes());
            else step(t & 3, Yes(), Yes());
        }
        // ================= P·V of the upper half of the last position; the fragments of its first slots were read
        // by the last unit =================
        la += ce0;
        lb += ce1;
        Pb[1][3] = pack2<T>(ce0, ce1);
        l_i += la + lb;
        {
            const int ls = (nt - 1) & 3;
#pragma unroll
            for (int m = 1; m < NSLOT; m += 2) {
                const vec8 vf = (m < LA) ? F[m % LA] : slot_frag(m, ls, 1, ls, 1);
                o_acc[(m >> 1) % DB] = mfma32(vf, __builtin_bit_cast(vec8, Pb[(m >> 1) / DB]), o_acc[(m >> 1) % DB]);
            }
        }
        // ================= the ring is free: the next item's queries, first tiles and mask row are requested now
        // and arrive while this item's result is normalised and stored =================
        ++round;
        const int next_item = item_of_round(round);
        __builtin_amdgcn_s_barrier();  // every wave has read its last fragments
        if (next_item >= 0) request_item(next_item);

        // ---- did some probability leave the 16-bit range?  One vote per workgroup, because the tiles are loaded by
        // all four waves together.
        float l_tot = halves32_sum(l_i);
        {
            // a probability beyond the 16-bit range enters P·V as infinity: the row's accumulator then holds
            // infinities or NaNs (0 * x keeps them and maps every finite x to 0)
            // (the row sum, taken from the unrounded probabilities, is at least as large as the largest of them: rows
            // whose sum is within the 16-bit range need no look at the accumulator)
            int any_bad = 0;
            if (__builtin_amdgcn_ballot_w64(!(l_tot < 60000.0f)) != 0) {
                float chk = 0.0f;
#pragma unroll
                for (int d = 0; d < DB; ++d)
#pragma unroll
                    for (int v = 0; v < 16; ++v) chk = fmaf(o_acc[d][v], 0.0f, chk);
                const bool bad = !(l_tot < 3.0e38f) || !(chk == 0.0f);
                any_bad = __builtin_amdgcn_ballot_w64(bad) != 0 ? 1 : 0;
            }
            if (lane == 0) vote_lds[wave] = any_bad;
            lds_barrier();
            const int redo = vote_lds[0] | vote_lds[1] | vote_lds[2] | vote_lds[3];
            if (__builtin_amdgcn_readfirstlane(redo) != 0) {
                // Plain loop over the same tiles in the same order: one tile at a time through ring slot 3 (the
                // next item's first tiles sit in slots 0..2), running maximum as the reference, everything rescaled
                // when it moves.  Runs with the finished item's addresses, mask terms (still in LDS) and rows.
                // (the next item's staged rows are on their way into ring slot 3, which this loop uses: they must have
                // landed everywhere before the first tile is requested; they are requested again afterwards)
                __builtin_amdgcn_s_waitcnt(0x0F70);
                __syncthreads();
                set_kv(cur_b, cur_h);
                if (VEC) classify_tiles();
                order_pos = 1;
                float m_run = -INFINITY;
                l_i = 0.0f;
#pragma unroll
                for (int d = 0; d < DB; ++d)
#pragma unroll
                    for (int v = 0; v < 16; ++v) o_acc[d][v] = 0.0f;
#pragma unroll
                for (int v = 0; v < 16; ++v) neg_m[v] = 0.0f;
                int tile = first_tile;
                for (int pos = 0; pos < nt; ++pos) {
                    __syncthreads();
                    dma_k(tile, 3);
                    dma_v(tile, 3);
                    __builtin_amdgcn_s_waitcnt(0x0F70);
                    __syncthreads();
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        Sa = mfma32(k_frag(3, 0, ks), qf[ks], ks == 0 ? neg_m : Sa);
                        Sb = mfma32(k_frag(3, 1, ks), qf[ks], ks == 0 ? neg_m : Sb);
                    }
                    if (pos >= n_clean) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            mask_pair(Sa, e, 0, tile * BN);
                            mask_pair(Sb, e, 1, tile * BN);
                        }
                    }
                    float mx = -INFINITY;
#pragma unroll
                    for (int v = 0; v < 16; ++v) mx = fmaxf(mx, fmaxf(Sa[v], Sb[v]));
                    mx = halves32_max(mx);
                    const float m_new = fmaxf(m_run, mx);
                    const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
                    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);  // 0 while nothing has been seen
                    m_run = m_new;
                    float rs = 0.0f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float a0 = __builtin_amdgcn_exp2f(Sa[2 * e] - m_use), a1 = __builtin_amdgcn_exp2f(Sa[2 * e + 1] - m_use);
                        const float b0 = __builtin_amdgcn_exp2f(Sb[2 * e] - m_use), b1 = __builtin_amdgcn_exp2f(Sb[2 * e + 1] - m_use);
                        Pa[e / 4][e % 4] = pack2<T>(a0, a1);
                        Pb[e / 4][e % 4] = pack2<T>(b0, b1);
                        rs += (a0 + a1) + (b0 + b1);
                    }
                    l_i = l_i * alpha + rs;
#pragma unroll
                    for (int d = 0; d < DB; ++d)
#pragma unroll
                        for (int v = 0; v < 16; ++v) o_acc[d][v] *= alpha;
#pragma unroll
                    for (int i = 0; i < 2 * DB; ++i) {
                        o_acc[i % DB] = mfma32(v_frag(3, i / DB, i % DB), __builtin_bit_cast(vec8, Pa[i / DB]), o_acc[i % DB]);
                        o_acc[i % DB] = mfma32(v_frag(3, 2 + i / DB, i % DB), __builtin_bit_cast(vec8, Pb[i / DB]), o_acc[i % DB]);
                    }
                    tile = next_tile(tile);
                }
                l_tot = halves32_sum(l_i);
                if (next_item >= 0) {
                    // the plain loop went through ring slot 3 of K and of V, where the next item's mask row and half of
                    // its query rows were waiting: request them again
                    set_kv(req_b, req_h);
                    __syncthreads();
                    request_staged();
                }
            }
        }
        // ---- normalise and store: lane holds features 32 d + 16 lh + (0..15) of its row
        const float inv_l = 1.0f / l_tot;
        const int my_m = cur_q0 + wave * 32 + lr;
        if (my_m < M) {
            T *orow = static_cast<T *>(p.o) + cur_b * p.os[0] + cur_h * p.os[1] + (int64_t)my_m * p.os[2] + lh * 16;
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
        if (next_item < 0) break;
        item = next_item;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // no load may still be writing LDS when the workgroup ends
}

template <typename T, int D>
static void launch_pipe_t(const AttnParams &p, int mask_mode, bool causal, hipStream_t st) {
    // persistent grid: as many workgroups per CU as the LDS rings allow (two at head size 64, one at 128), 32 CUs per
    // XCD, fewer when the busiest XCD has fewer items
    constexpr int kPerCu = D == 64 ? 2 : 1;
    constexpr int kRingBytes = 4 * 2 * 64 * D * 2;
    const int heads_per_xcd = (p.B * p.H + 7) / 8;
    const int64_t items_per_xcd = (int64_t)heads_per_xcd * p.nq_tiles;
    const int per_xcd = (int)(items_per_xcd < 32 * kPerCu ? items_per_xcd : 32 * kPerCu);
    dim3 grid((unsigned)(8 * per_xcd)), block(256);
    const int lds_bytes = D == 64 ? 0 : kRingBytes + (mask_mode == MASK_VECTOR ? kPipeMaxMaskKeys * 4 : 0) + 96;
#define KERNL_PIPE_LAUNCH(MM, C)                                                                                        \
    do {                                                                                                               \
        auto kern = attention_pipe_kernel<T, D, MM, C>;                                                                \
        static bool attr_done = false; /* benign race: the attribute call is idempotent */                             \
        if (!attr_done) {                                                                                              \
            (void)hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                      kRingBytes + kPipeMaxMaskKeys * 4 + 96);                                         \
            attr_done = true;                                                                                          \
        }                                                                                                              \
        hipLaunchKernelGGL(kern, grid, block, lds_bytes, st, p);                                                        \
    } while (0)
    if (mask_mode == MASK_VECTOR) KERNL_PIPE_LAUNCH(MASK_VECTOR, false);
    else if (causal) KERNL_PIPE_LAUNCH(MASK_NONE, true);
    else KERNL_PIPE_LAUNCH(MASK_NONE, false);
#undef KERNL_PIPE_LAUNCH
}

// true if the problem was launched here; false: not covered, the caller takes the streaming kernel
bool launch_attention_pipe(const AttnParams &p, int D, int dtype, int mask_mode, bool causal, bool force, hipStream_t st) {
    if (D != 64 && D != 128) return false;
    if (mask_mode == MASK_MATRIX) return false;
    if (mask_mode == MASK_VECTOR && (causal || p.N > kPipeMaxMaskKeys)) return false;
    if (((int64_t)p.M + 128) * p.qs[2] >= (1ll << 30)) return false;  // the query rows are fetched through 32-bit byte offsets
    // From kPipeMinKeys keys on, and for SMALL grids (at most one 128-query item per CU) from 256 keys on: there the
    // streaming kernel has no other workgroup on the CU to fill a wave's dependent phases with, and this kernel's own
    // overlap is worth 10-16 % (head size 64, [1,64,512,64]: 10.6 -> 9.3 us, [1,32,512,768]: 13.0 -> 10.2; with 512 items 4 %,
    // beyond that it ties or loses, as at BASELINE config 1).
    const bool small_grid = D == 64 && !causal && p.N >= 256 && (int64_t)p.B * p.H * ((p.M + 127) / 128) <= 256;
    if (!force && p.N < kPipeMinKeys && !small_grid) return false;
    // Head size 128 runs one workgroup per CU here and is no faster per tile than the streaming kernel (both sit at the
    // chip's power limit); what it wins is BALANCE when a causal problem has few (batch, head) pairs: a persistent
    // workgroup pairs long and short query tiles, where the streaming kernel's grid is one round of unequal workgroups
    // (measured, [1,32,2048,128] causal: 50 against 60 us; 64 pairs: +3..6 %; 128 pairs or 40: slower).
    if (!force && D == 128 && !(causal && mask_mode == MASK_NONE && p.B * p.H <= 64 && (p.B * p.H) % 8 == 0)) return false;
    if (D == 64) {
        if (dtype == KERNL_F16) launch_pipe_t<f16, 64>(p, mask_mode, causal, st);
        else launch_pipe_t<bf16, 64>(p, mask_mode, causal, st);
    } else {
        if (dtype == KERNL_F16) launch_pipe_t<f16, 128>(p, mask_mode, causal, st);
        else launch_pipe_t<bf16, 128>(p, mask_mode, causal, st);
    }
    return true;
}

}  // namespace kernl
