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
// To fit the 2 + 2 budget the loop has NO row maximum and no rescaling: scores come out of the MFMA already relative
// to the row's exponent reference (its negative is the C operand), and the reference is the maximum of the row's
// first tile.  Probabilities of later tiles may exceed 1; as long as none exceeds the 16-bit range the final O / l is
// exact whatever the reference.  If one does, the row sum ends up infinite: the workgroup then redoes its rows with a
// plain loop that tracks the maximum (rare: a score must exceed the first tile's maximum by 16 in base-2 units).
//
// Data movement: K and V tiles go HBM -> LDS directly (buffer loads with the LDS flag) into rings of 4 slots each,
// requested two tiles ahead of their use; one workgroup barrier per tile.  Layouts and the transposed-score trick
// (Sᵀ = K·Qᵀ, a lane owns one query row; the packed probabilities already are the MFMA B operand of Oᵀ = Vᵀ·Pᵀ) are
// those of attention.hip.
#include "attention_common.h"

#ifndef KERNL_ATTN_PIPE_LOOKAHEAD
#define KERNL_ATTN_PIPE_LOOKAHEAD 4
#endif

namespace kernl {

#ifdef WHATIF_PIN_MFMA
__device__ __forceinline__ f32x16 pinned_mfma(f16x8 a, f16x8 b, f32x16 c) {
    f32x16 d;
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}
__device__ __forceinline__ f32x16 pinned_mfma(bf16x8 a, bf16x8 b, f32x16 c) {
    f32x16 d;
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}
#define UNIT_MFMA pinned_mfma
#else
#define UNIT_MFMA mfma32
#endif

template <typename T, int MASK_MODE, bool CAUSAL>
__global__ void __launch_bounds__(256, 2) attention_pipe_kernel(const AttnParams p) {
    typedef typename Vec8<T>::type vec8;
    typedef __attribute__((address_space(3))) void lds_void;
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    constexpr int D = 64, BM = 128, BN = 64, NS = 4;
    constexpr int KROW = D * 2, VP = D * 2;              // LDS row bytes of the K tile [key][D] and V tile [key][D]
    constexpr int K_BYTES = BN * KROW, V_BYTES = BN * VP;
    constexpr int DB = D / 32, KS = D / 16;
    constexpr int DC = D / 8;                            // 16-byte chunks per K/V row
    constexpr int KI = BN * DC / 256;                    // 1 KB loads per wave for each of K and V
    constexpr int V_RING = NS * K_BYTES;
    constexpr int BIAS_OFF = NS * (K_BYTES + V_BYTES);
    constexpr bool VEC = (MASK_MODE == MASK_VECTOR);
    constexpr int BIAS_KEYS = VEC ? kPipeMaxMaskKeys : 0;
    static_assert(!(VEC && CAUSAL), "per-key masks with causal masking take the streaming kernel");
    static_assert(KI * 4096 == K_BYTES && K_BYTES == V_BYTES, "a tile is KI loads of 1 KB per wave");
    typedef BoolC<true> Yes;
    typedef BoolC<false> No;

    __shared__ __attribute__((aligned(16))) unsigned char smem[BIAS_OFF + BIAS_KEYS * 4 + 64];

    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int bh = (slot / p.nq_tiles) * 8 + xcd;
    int qt = slot % p.nq_tiles;
    if (bh >= p.B * p.H) return;
    if (CAUSAL) qt = p.nq_tiles - 1 - qt;  // longest rows first
    const int b = bh / p.H, h = bh % p.H;

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 31, lh = lane >> 5;
    const int q0 = qt * BM;
    const int my_m = q0 + wave * 32 + lr;
    const int M = p.M, N = p.N;

    const T *qp = static_cast<const T *>(p.q) + b * p.qs[0] + h * p.qs[1];
    const T *kp = static_cast<const T *>(p.k) + b * p.ks[0] + h * p.ks[1];
    const T *vp = static_cast<const T *>(p.v) + b * p.vs[0] + h * p.vs[1];
    T *op = static_cast<T *>(p.o) + b * p.os[0] + h * p.os[1];

    // ---- Q fragments (MFMA "B" side: lane holds its query row, 8 consecutive features per k-step), multiplied once
    // by scale * log2(e): the MFMA result is the score in the base-2 domain
    vec8 qf[KS];
    {
        const T *qrow = qp + (int64_t)min(my_m, M - 1) * p.qs[2] + lh * 8;
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const vec8 *>(qrow + s * 16);
    }

    // ---- staging (as in attention.hip): the i-th load of a wave fills the 1 KB of 16-byte chunks
    // [256 i + 64 wave, +64) of a tile; every lane fetches the chunk of global memory that belongs at its LDS
    // position under the tile's swizzle.  Rows past the last key lie beyond the buffer resource and arrive as zeros.
    uint32_t kdma[KI], vdma[KI];
#pragma unroll
    for (int i = 0; i < KI; ++i) {
        const int qd = tid + 256 * i;
        const int row = qd / DC, cs = qd % DC;
        kdma[i] = (uint32_t)(((int64_t)row * p.ks[2] + swz_chunk<KROW>(row, cs) * 8) * 2);
        const int vsw = (row >> 1) & 1;
        vdma[i] = (uint32_t)(((int64_t)row * p.vs[2] + (cs ^ (vsw << 2)) * 8) * 2);
    }
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void *)smem;
    const uint32_t dma_base = lds_base + wave * 1024;
    const uint64_t kaddr = (uint64_t)(uintptr_t)kp, vaddr = (uint64_t)(uintptr_t)vp;
    const u32x4 krsrc = {(uint32_t)kaddr, (uint32_t)(kaddr >> 32) & 0xFFFFu,
                         (uint32_t)((((int64_t)N - 1) * p.ks[2] + D) * 2), 0x00020000u};
    const u32x4 vrsrc = {(uint32_t)vaddr, (uint32_t)(vaddr >> 32) & 0xFFFFu,
                         (uint32_t)((((int64_t)N - 1) * p.vs[2] + D) * 2), 0x00020000u};
    const int k_tile_bytes = (int)((int64_t)BN * p.ks[2] * 2), v_tile_bytes = (int)((int64_t)BN * p.vs[2] * 2);
    auto uniform = [](uint32_t x) __attribute__((always_inline)) -> uint32_t { return (uint32_t)__builtin_amdgcn_readfirstlane((int)x); };
    // Inline assembly on purpose: the compiler, seeing LDS written by a load, would make every later LDS read wait
    // for the vector-memory counter, i.e. for the prefetches themselves.  The explicit counter waits before the
    // barrier of each step are the ones that matter.
    auto dma_k = [&](int tile, int ring_slot) __attribute__((always_inline)) {
        const uint32_t soff = uniform((uint32_t)(tile * k_tile_bytes));
        const uint32_t sb = uniform(dma_base + ring_slot * K_BYTES);
        const u32x4 kr = krsrc;
#pragma unroll
        for (int i = 0; i < KI; ++i)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :: "s"(sb + i * 4096), "v"(kdma[i]), "s"(kr), "s"(soff) : "memory", "m0");
    };
    auto dma_v = [&](int tile, int ring_slot) __attribute__((always_inline)) {
        const uint32_t soff = uniform((uint32_t)(tile * v_tile_bytes));
        const uint32_t sb = uniform(dma_base + V_RING + ring_slot * V_BYTES);
        const u32x4 vr = vrsrc;
#pragma unroll
        for (int i = 0; i < KI; ++i)
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :: "s"(sb + i * 4096), "v"(vdma[i]), "s"(vr), "s"(soff) : "memory", "m0");
    };

    // ---- key tiles in processing order: positions [0, n_clean) need no masking, [n_clean, nt) take the general body
    const int n_end = CAUSAL ? min(N, q0 + BM + p.causal_off) : N;
    const int nt_all = (n_end + BN - 1) / BN;
    int nt = nt_all, n_clean = 0;
    if (!VEC) n_clean = CAUSAL ? min(N / BN, (q0 + p.causal_off + 1) / BN) : N / BN;
    n_clean = min(n_clean, nt);

    // The first positions are requested before the mask has been looked at, in natural order (what a mask that pads
    // on the right ends up with); a different order re-requests them below.  Step t requests K(t+3) and V(t+2).
    {
        const int last = nt_all - 1;
        dma_k(0, 0);
        dma_v(0, 0);
        dma_k(min(1, last), 1);
        dma_k(min(2, last), 2);
        dma_v(min(1, last), 1);
    }

    // ---- per-key mask: additive terms of all keys in LDS, relative to the largest one; tile classification
    uint32_t clean_bits = 0, gen_bits = 0;  // at most kPipeMaxMaskKeys / BN = 32 tiles; wave-uniform
    int first_tile = 0;
    float *bias_lds = reinterpret_cast<float *>(smem + BIAS_OFF);
    int *vote_lds = reinterpret_cast<int *>(smem + BIAS_OFF + BIAS_KEYS * 4 + 32);
    bool zero_q = false;
    // every wave classifies all tiles by itself from the additive terms in LDS: bit t of clean_bits = tile t is full
    // and all zero, of gen_bits = it needs the general body; tiles in neither set are so negative everywhere that they
    // contribute exactly 0.  Sets the first tile, n_clean and nt; called again by the second pass over the tiles.
    auto classify_tiles = [&]() __attribute__((always_inline)) {
        const int npad = nt_all * BN;
        uint32_t ord_bits = 0;
        clean_bits = 0;
        gen_bits = 0;
        for (int g = 0; g * 64 < npad; ++g) {
            const int n = g * 64 + lane;
            const float v = bias_lds[n];
            const bool valid = n < N;
            const bool any_nz = __ballot(valid && v != 0.0f) != 0, any_nm = __ballot(valid && v > kNegBig) != 0,
                       any_ord = __ballot(valid && v == 0.0f) != 0;
            const bool full = g * 64 + 64 <= N;
            if (any_nm) {
                if (any_nz || !full) gen_bits |= 1u << g;
                else clean_bits |= 1u << g;
            }
            if (any_ord) ord_bits |= 1u << g;
        }
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
    if (VEC) {
        const int64_t mask_base = b * p.ms[0] + h * p.ms[1];
        const int npad = nt_all * BN;
        float *red = bias_lds + BIAS_KEYS;
        constexpr int PER = VEC ? BIAS_KEYS / 256 : 1;
        float smv[PER];
        float lmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int n = tid + 256 * i;
            smv[i] = -INFINITY;
            if (n < N) {
                smv[i] = scale_mask(load_mask_value(p.mask, p.mask_dtype, mask_base + (int64_t)n * p.ms[3]), p.clamp);
                lmax = fmaxf(lmax, smv[i]);
            }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) lmax = fmaxf(lmax, __shfl_xor(lmax, off, 64));
        if (lane == 0) red[wave] = lmax;
        __syncthreads();
        // softmax does not change when every key's term moves by the same amount: the largest term becomes 0, so
        // some key is always "ordinary" and the exponent reference set by the first tile is an ordinary score.  When
        // even the largest term is a clamped -inf, fp32 scores would have absorbed q·k entirely: q is dropped, which
        // gives the plain average of V over those keys, as the reference does.
        const float bmax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        zero_q = bmax < kNegBig;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int n = tid + 256 * i;
            if (n < npad) bias_lds[n] = smv[i] - bmax;
        }
        __syncthreads();
        classify_tiles();
    }
    int order_pos = 1;
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
    int tq[4];  // tiles at positions t .. t+3
    tq[0] = first_tile;
#pragma unroll
    for (int j = 1; j < 4; ++j) tq[j] = next_tile(tq[j - 1]);
    {
        const int last = nt_all - 1;
        const bool natural = tq[0] == 0 && tq[1] == min(1, last) && tq[2] == min(2, last);
        if (!natural) {  // wave-uniform, and the same in every wave
            __builtin_amdgcn_s_waitcnt(0x0F70);
            __syncthreads();
            dma_k(tq[0], 0);
            dma_v(tq[0], 0);
            dma_k(tq[1], 1);
            dma_k(tq[2], 2);
            dma_v(tq[1], 1);
        }
    }
#pragma unroll
    for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[s][e] = from_float<T>(zero_q ? 0.0f : to_float(qf[s][e]) * p.scale_log2);

    // ---- running state of this lane's query row
    float l_i = 0.0f;
    f32x16 neg_m;
#pragma unroll
    for (int v = 0; v < 16; ++v) neg_m[v] = 0.0f;
    f32x16 o_acc[DB];
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int v = 0; v < 16; ++v) o_acc[d][v] = 0.0f;
    f32x16 Sa, Sb;      // scores of the lower / upper 32 keys of a tile
    u32x4 Pa[2], Pb[2]; // their packed probabilities

    // LDS byte offsets of this lane's operand fragments (see attention.hip)
    int k_off[KS], vt_off[DB];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_off[ks] = swz_offset<KROW>(lr, 2 * ks + lh);
    {
        const int i16 = lane & 15, g16 = lane >> 4;
        const int kq = i16 >> 2;
        const int fs = rowperm16(16 * (g16 & 1) + 4 * (i16 & 3));
        const int vsw = kq >> 1;
#pragma unroll
        for (int d = 0; d < DB; ++d) vt_off[d] = V_RING + (4 * lh + kq) * VP + ((d ^ vsw) * 64) + fs * 2;
    }
    // last key this lane's row may see (causal diagonal, end of the keys), minus the lane's own offset inside a group
    const int key_limit = (CAUSAL ? min(N - 1, my_m + p.causal_off) : N - 1) - lh * 4;

    auto k_frag = [&](int ring_slot, int half, int ks) __attribute__((always_inline)) -> vec8 {
        return *reinterpret_cast<const vec8 *>(smem + ring_slot * K_BYTES + half * 32 * KROW + k_off[ks]);
    };
    auto v_frag = [&](int ring_slot, int ps, int d) __attribute__((always_inline)) -> vec8 {
        const unsigned char *va = smem + ring_slot * V_BYTES + 16 * ps * VP + vt_off[d];
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)va);
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4 *)(va + 8 * VP));
        return __builtin_bit_cast(vec8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };
    // masking of the scores of a general tile: pair e (0..7) of the lane's scores of the half `half`, in place
    auto mask_pair = [&](f32x16 &Sc, int e, int half, int n0) __attribute__((always_inline)) {
        const int v0 = 2 * e;
        const int c0 = 32 * half + 8 * (v0 / 4) + (v0 % 4);  // key of the first score of the pair, relative to n0 + 4 lh
        if (VEC) {
            const f32x2 cb = *reinterpret_cast<const f32x2 *>(bias_lds + n0 + c0 + lh * 4);
            Sc[v0] += cb[0];
            Sc[v0 + 1] += cb[1];
        } else {
            const int rel = key_limit - n0;
            if (c0 > rel) Sc[v0] = -INFINITY;
            if (c0 + 1 > rel) Sc[v0 + 1] = -INFINITY;
        }
    };

    // Operand fragments are read from LDS LA slots before the MFMA that consumes them (an LDS read takes longer than
    // two MFMAs under load), across unit and step boundaries: F[m % LA] holds the fragment of slot m.
    // Slot m of a unit: even -> K fragment (ks = m / 2) of the unit's score half; odd -> V fragment (ps, d) of its P·V half.
    constexpr int LA = KERNL_ATTN_PIPE_LOOKAHEAD;
    vec8 F[LA];
    auto slot_frag = [&](int m, int qk_slot, int qk_half, int pv_slot, int pv_half) __attribute__((always_inline)) -> vec8 {
#ifdef WHATIF_NOLDS
        return qf[m & 3];
#endif
#ifdef WHATIF_NOLDS_K
        if ((m & 1) == 0) return qf[m & 3];
#endif
#ifdef WHATIF_NOLDS_V
        if ((m & 1) == 1) return qf[m & 3];
#endif
#ifdef WHATIF_LDS_UNUSED
        {
            vec8 r = ((m & 1) == 0) ? k_frag(qk_slot, qk_half, m >> 1) : v_frag(pv_slot, 2 * pv_half + (m >> 2), (m >> 1) & 1);
            asm volatile("" :: "v"(r));
            return qf[m & 3];
        }
#endif
        if ((m & 1) == 0) return k_frag(qk_slot, qk_half, m >> 1);
        return v_frag(pv_slot, 2 * pv_half + (m >> 2), (m >> 1) & 1);
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
    float la = 0.0f, lb = 0.0f, ce0 = 0.0f, ce1 = 0.0f;
#define KERNL_SB __builtin_amdgcn_sched_barrier(0)
    auto unit = [&](f32x16 &Scur, u32x4 (&Pcur)[2], f32x16 &Snext, u32x4 (&Pprev)[2], auto doqk_c, auto general_c, auto carry_c,
                    int qk_slot, int qk_half, int pv_slot, int pv_half, int nqk_slot, int nqk_half, int npv_slot, int npv_half,
                    int n0, int cur_half) __attribute__((always_inline)) {
        constexpr bool DO_QK = decltype(doqk_c)::value, GENERAL = decltype(general_c)::value, HAS_CARRY = decltype(carry_c)::value;
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            if ((m & 1) == 0) {
                if (DO_QK) Snext = UNIT_MFMA(F[m % LA], qf[m >> 1], m == 0 ? neg_m : Snext);
            } else {
                o_acc[(m >> 1) & 1] = UNIT_MFMA(F[m % LA], __builtin_bit_cast(vec8, Pprev[m >> 2]), o_acc[(m >> 1) & 1]);
            }
            KERNL_SB;
            if (m + LA < 8) F[m % LA] = slot_frag(m + LA, qk_slot, qk_half, pv_slot, pv_half);
            else F[m % LA] = slot_frag(m + LA - 8, nqk_slot, nqk_half, npv_slot, npv_half);
            KERNL_SB;
            if (GENERAL) mask_pair(Scur, m, cur_half, n0);
            const float e0 = __builtin_amdgcn_exp2f(Scur[2 * m]);
            KERNL_SB;
            if (m > 0 || HAS_CARRY) la += ce0;
            KERNL_SB;
            const float e1 = __builtin_amdgcn_exp2f(Scur[2 * m + 1]);
            KERNL_SB;
            if (m > 0 || HAS_CARRY) {
                lb += ce1;
                KERNL_SB;
                const uint32_t pk = pack2<T>(ce0, ce1);
                if (m == 0) Pprev[1][3] = pk;
                else Pcur[(m - 1) / 4][(m - 1) % 4] = pk;
            }
            ce0 = e0;
            ce1 = e1;
            KERNL_SB;
        }
    };
    // the pair left over by the last unit (always of the upper half of a tile: Pb)
    auto finish_carry = [&]() __attribute__((always_inline)) {
        la += ce0;
        lb += ce1;
        Pb[1][3] = pack2<T>(ce0, ce1);
    };

    // Step t >= 1 (ts = t % 4):  request K(t+3), V(t+2);
    //   unit A: scores of (t, upper half), probabilities of (t, lower half), P·V of (t-1, upper half);
    //   unit B: scores of (t+1, lower half) unless t is the last position, probabilities of (t, upper), P·V of (t, lower);
    // the unit after B is unit A of step t+1 (or, after the last position, the P·V of its upper half, whose fragments
    // sit in the odd slots just the same).
    auto step = [&](int ts, auto general_c, auto last_c) __attribute__((always_inline)) {
        constexpr bool LAST = decltype(last_c)::value;
        const int n0 = tq[0] * BN;
#ifndef WHATIF_NODMA
        if (!LAST) {
            dma_k(tq[3], (ts + 3) & 3);
            dma_v(tq[2], (ts + 2) & 3);
        }
#endif
        const int k1 = (ts + 1) & 3, v3 = (ts + 3) & 3;
        unit(Sa, Pa, Sb, Pb, Yes(), general_c, Yes(), ts, 1, v3, 1, k1, 0, ts, 0, n0, 0);
        if (LAST) unit(Sb, Pb, Sa, Pa, No(), general_c, Yes(), k1, 0, ts, 0, k1, 1, ts, 1, n0, 1);
        else unit(Sb, Pb, Sa, Pa, Yes(), general_c, Yes(), k1, 0, ts, 0, k1, 1, ts, 1, n0, 1);
        // this wave's part of K(t+2) and V(t+1) has landed (only this step's requests may still be in flight); after
        // the barrier everybody's has, and nobody reads the ring slots any more that the next step's requests overwrite
        if (!LAST) __builtin_amdgcn_s_waitcnt(0x0F70 | 4);
        else __builtin_amdgcn_s_waitcnt(0x0F70);
#ifndef WHATIF_NOBARRIER
        __builtin_amdgcn_s_barrier();
#endif
#pragma unroll
        for (int j = 0; j < 3; ++j) tq[j] = tq[j + 1];
        tq[3] = next_tile(tq[3]);
    };

    // ---- position 0: K(0) has landed -> scores (against a reference of 0), row maximum = the row's reference,
    // probabilities of the lower half; then the unit-B half of a step.
    __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
    __syncthreads();
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
            const uint32_t pk = pack2<T>(__builtin_amdgcn_exp2f(Sa[2 * e]), __builtin_amdgcn_exp2f(Sa[2 * e + 1]));
            Pa[e / 4][e % 4] = pk;
            rs = pair_sum_acc<T>(pk, rs);
        }
        l_i = rs;
        // K(1) and V(0) have landed too
        __builtin_amdgcn_s_waitcnt(0x0F70 | 4);
        __builtin_amdgcn_s_barrier();
        // the first unit: scores of (1, lower half) if there is a position 1, probabilities of (0, upper), P·V of (0, lower)
#pragma unroll
        for (int m = 0; m < LA && m < 8; ++m) F[m] = slot_frag(m, 1, 0, 0, 0);
        if (nt > 1) {
            dma_k(tq[3], 3);
            dma_v(tq[2], 2);
            unit(Sb, Pb, Sa, Pa, Yes(), No(), No(), 1, 0, 0, 0, 1, 1, 0, 1, n0, 1);
            __builtin_amdgcn_s_waitcnt(0x0F70 | 4);
        } else {
            unit(Sb, Pb, Sa, Pa, No(), No(), No(), 1, 0, 0, 0, 1, 1, 0, 1, n0, 1);
            __builtin_amdgcn_s_waitcnt(0x0F70);
        }
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int j = 0; j < 3; ++j) tq[j] = tq[j + 1];
        tq[3] = next_tile(tq[3]);
    }
    // ---- positions 1 .. nt-1: clean ones (four at a time with compile-time ring slots, then one at a time), general
    // ones, and the last position without further scores
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
    // ---- P·V of the upper half of the last position; the fragments of its first slots were read by the last unit
    finish_carry();
    l_i += la + lb;
    {
        const int ls = (nt - 1) & 3;
#pragma unroll
        for (int m = 1; m < 8; m += 2) {
            const vec8 vf = (m < LA) ? F[m % LA] : slot_frag(m, ls, 1, ls, 1);
            o_acc[(m >> 1) & 1] = mfma32(vf, __builtin_bit_cast(vec8, Pb[m >> 2]), o_acc[(m >> 1) & 1]);
        }
    }

    // ---- did some probability leave the 16-bit range?  One vote per
    // workgroup, because the tiles are loaded by all four waves together.
    float l_tot = halves32_sum(l_i);
    {
        // a probability beyond the 16-bit range enters P·V as infinity: the row's accumulator then holds infinities
        // or NaNs (0 * x keeps them and maps every finite x to 0)
        float chk = 0.0f;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int v = 0; v < 16; ++v) chk = fmaf(o_acc[d][v], 0.0f, chk);
        const bool bad = !(l_tot < 3.0e38f) || !(chk == 0.0f);
        const int any_bad = __builtin_amdgcn_ballot_w64(bad) != 0 ? 1 : 0;
        if (lane == 0) vote_lds[wave] = any_bad;
        __syncthreads();
        const int redo = vote_lds[0] | vote_lds[1] | vote_lds[2] | vote_lds[3];
        if (__builtin_amdgcn_readfirstlane(redo) != 0) {
            // Plain loop over the same tiles in the same order: one tile at a time through ring slot 0, running
            // maximum as the reference, everything rescaled when it moves.
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
                dma_k(tile, 0);
                dma_v(tile, 0);
                __builtin_amdgcn_s_waitcnt(0x0F70);
                __syncthreads();
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    Sa = mfma32(k_frag(0, 0, ks), qf[ks], ks == 0 ? neg_m : Sa);
                    Sb = mfma32(k_frag(0, 1, ks), qf[ks], ks == 0 ? neg_m : Sb);
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
                    const uint32_t pa = pack2<T>(__builtin_amdgcn_exp2f(Sa[2 * e] - m_use), __builtin_amdgcn_exp2f(Sa[2 * e + 1] - m_use));
                    const uint32_t pb = pack2<T>(__builtin_amdgcn_exp2f(Sb[2 * e] - m_use), __builtin_amdgcn_exp2f(Sb[2 * e + 1] - m_use));
                    Pa[e / 4][e % 4] = pa;
                    Pb[e / 4][e % 4] = pb;
                    rs = pair_sum_acc<T>(pa, rs);
                    rs = pair_sum_acc<T>(pb, rs);
                }
                l_i = l_i * alpha + rs;
#pragma unroll
                for (int d = 0; d < DB; ++d)
#pragma unroll
                    for (int v = 0; v < 16; ++v) o_acc[d][v] *= alpha;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    o_acc[i & 1] = mfma32(v_frag(0, i >> 1, i & 1), __builtin_bit_cast(vec8, Pa[i >> 1]), o_acc[i & 1]);
                    o_acc[i & 1] = mfma32(v_frag(0, 2 + (i >> 1), i & 1), __builtin_bit_cast(vec8, Pb[i >> 1]), o_acc[i & 1]);
                }
                tile = next_tile(tile);
            }
            l_tot = halves32_sum(l_i);
        }
    }

    // ---- normalise and store: lane holds features 32 d + 16 lh + (0..15) of row my_m
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

template <typename T>
static void launch_pipe_t(const AttnParams &p, int mask_mode, bool causal, hipStream_t st) {
    const int bh_padded = ((p.B * p.H + 7) / 8) * 8;
    dim3 grid((unsigned)(bh_padded * p.nq_tiles)), block(256);
    if (mask_mode == MASK_VECTOR) hipLaunchKernelGGL((attention_pipe_kernel<T, MASK_VECTOR, false>), grid, block, 0, st, p);
    else if (causal) hipLaunchKernelGGL((attention_pipe_kernel<T, MASK_NONE, true>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((attention_pipe_kernel<T, MASK_NONE, false>), grid, block, 0, st, p);
}

// true if the problem was launched here; false: not covered, the caller takes the streaming kernel
bool launch_attention_pipe(const AttnParams &p, int D, int dtype, int mask_mode, bool causal, hipStream_t st) {
    if (D != 64) return false;
    if (mask_mode == MASK_MATRIX) return false;
    if (mask_mode == MASK_VECTOR && (causal || p.N > kPipeMaxMaskKeys)) return false;
    if (dtype == KERNL_F16) launch_pipe_t<f16>(p, mask_mode, causal, st);
    else launch_pipe_t<bf16>(p, mask_mode, causal, st);
    return true;
}

}  // namespace kernl
