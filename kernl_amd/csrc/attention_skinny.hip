// Split-K attention for very few query rows (decoding: one query against a long key sequence).
//
// Semantics are those of attention.hip; the decomposition follows the reference's two-kernel skinny attention
// (src/kernl/implementations/attention_skinny.py:59-367: part 1 computes per key-range maxima, sums and partial
// products, part 2 merges them) because a single query row offers no parallelism over rows: the keys of every
// (batch, head, query row) are split into ranges, one workgroup per range, and a second kernel merges the ranges.
//
// The problem is vector x matrix, i.e. bound by reading K and V once from HBM, so there is no MFMA here: D/8
// lanes share a key row (16-byte loads), a wave covers 512/D keys per load, every lane group runs its own online
// softmax and the groups are merged once at the end (registers -> LDS -> workspace).
#include <math.h>

#include <type_traits>

#include "common.h"

namespace kernl {

static constexpr float kSkLog2e = 1.4426950408889634f;
static constexpr float kSkClampFloor = -1.7014118e38f;

struct SkinnyParams {
    const void *q, *k, *v, *mask;
    void *o;
    float *ws;  // [rows][splits][D + 2] : running maximum (log2 domain), sum, un-normalised output
    int B, H, M, N, D, splits;
    int64_t qs[4], ks[4], vs[4], os[4], ms[4];
    int mask_dtype, has_mask, causal;
    int kv8;  // k and v hold one byte per element: fp8 e5m2, the upper byte of the fp16 encoding
    float scale_log2, clamp;
};

__device__ __forceinline__ float sk_mask_value(const void *mask, int dtype, int64_t off, float clamp) {
    float mv;
    if (dtype == KERNL_F32) mv = static_cast<const float *>(mask)[off];
    else if (dtype == KERNL_F16) mv = (float)static_cast<const f16 *>(mask)[off];
    else mv = (float)static_cast<const bf16 *>(mask)[off];
    if (mv == -INFINITY) mv = clamp;
    return fmaxf(mv * kSkLog2e, kSkClampFloor);
}

// merge the online-softmax state (m, l, acc[8]) of another lane group / wave into this one
__device__ __forceinline__ void sk_merge(float &m, float &l, float (&acc)[8], float m2, float l2, const float (&acc2)[8]) {
    const float mn = fmaxf(m, m2);
    const float a = (m == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m - mn);
    const float b = (m2 == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m2 - mn);
    l = l * a + l2 * b;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = acc[e] * a + acc2[e] * b;
    m = mn;
}

// 8 features of a key or value row as they lie in memory: 8 bytes of fp8 e5m2 storage, or 16 bytes of the 16-bit type
template <bool KV8>
struct SkRaw {
    typedef typename std::conditional<KV8, uint2, u32x4>::type type;
};

template <typename T, bool KV8>
__device__ __forceinline__ typename SkRaw<KV8>::type sk_load_raw(const void *base, int64_t elem_off) {
    typedef typename SkRaw<KV8>::type raw_t;
    if constexpr (KV8) return *reinterpret_cast<const raw_t *>(static_cast<const unsigned char *>(base) + elem_off);
    else return *reinterpret_cast<const raw_t *>(static_cast<const T *>(base) + elem_off);
}

// ... as fp32: from the 16-bit storage type, or from fp8 e5m2 bytes — those are the upper bytes of fp16 values, so
// decoding is a shift (reference: the int8 caches bit-cast to float8e5 and widened to fp16,
// experimental/llama-v2/kernel/fused_kernel_attention.py:69-71,90-92).
template <typename T, bool KV8>
__device__ __forceinline__ void sk_widen8(const typename SkRaw<KV8>::type &raw, float (&f)[8]) {
    if constexpr (KV8) {
        const uint32_t w[2] = {raw.x, raw.y};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const unsigned short h = (unsigned short)(((w[e >> 2] >> (8 * (e & 3))) & 0xFFu) << 8);
            f[e] = (float)__builtin_bit_cast(_Float16, h);
        }
    } else {
        typedef typename Vec8<T>::type vec8;
        const vec8 v = __builtin_bit_cast(vec8, raw);
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = (float)v[e];
    }
}

// ... as four packed fp16 pairs (fp16 queries only): fp8 e5m2 bytes become fp16 values by moving each byte into the
// upper half of a 16-bit lane, one byte-permute per pair; fp16 storage is used as it lies.
template <bool KV8>
__device__ __forceinline__ void sk_pairs8(const typename SkRaw<KV8>::type &raw, uint32_t (&pk)[4]) {
    if constexpr (KV8) {
        pk[0] = __builtin_amdgcn_perm(0u, raw.x, 0x010c000cu);  // bytes {0, b0, 0, b1}
        pk[1] = __builtin_amdgcn_perm(0u, raw.x, 0x030c020cu);
        pk[2] = __builtin_amdgcn_perm(0u, raw.y, 0x010c000cu);
        pk[3] = __builtin_amdgcn_perm(0u, raw.y, 0x030c020cu);
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) pk[j] = raw[j];
    }
}

// DL = D / 8 lanes per key (a power of two, 1..64); KPI keys per lane and trip of the loop
template <typename T, int DL, bool KV8, int KPI>
__global__ void __launch_bounds__(256) attention_skinny_part1(const SkinnyParams p) {
    typedef typename Vec8<T>::type vec8;
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    constexpr int KPW = 64 / DL;  // keys per wave and step
    __shared__ float red[4][DL][10];
    const int row = blockIdx.y, split = blockIdx.x;
    const int m = row % p.M, bh = row / p.M, b = bh / p.H, h = bh % p.H;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int dl = lane % DL, kg = lane / DL;

    const T *qp = static_cast<const T *>(p.q) + b * p.qs[0] + h * p.qs[1] + (int64_t)m * p.qs[2] + dl * 8;
    const int64_t k_base = b * p.ks[0] + h * p.ks[1] + dl * 8, v_base = b * p.vs[0] + h * p.vs[1] + dl * 8;
    const int64_t mask_base = p.has_mask ? b * p.ms[0] + h * p.ms[1] + (int64_t)m * p.ms[2] : 0;

    const int n_end = p.causal ? min(p.N, m + 1) : p.N;
    // key ranges are multiples of the 4 KPW keys a workgroup takes per step
    const int step = 4 * KPW;
    const int per_split = ((n_end + p.splits - 1) / p.splits + step - 1) / step * step;
    const int c0 = split * per_split, c1 = min(n_end, c0 + per_split);

    float qf[8];
    uint32_t qpk[4];  // the same 8 query features as packed pairs, unscaled (fp16 path)
    {
        const vec8 qv = *reinterpret_cast<const vec8 *>(qp);
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[e] = (float)qv[e] * p.scale_log2;
        const u32x4 qraw = __builtin_bit_cast(u32x4, qv);
#pragma unroll
        for (int j = 0; j < 4; ++j) qpk[j] = qraw[j];
    }
    float mi = -INFINITY, li = 0.0f, acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    // KPI keys per lane and trip: all their loads are issued before the first is used (the cross-lane sums keep the
    // compiler from unrolling this loop by itself), and they share one move of the softmax reference
    for (int n0 = c0 + wave * KPW; n0 < c1; n0 += step * KPI) {
        typename SkRaw<KV8>::type kr[KPI], vr[KPI];
        bool valid[KPI];
        int nn[KPI];
#pragma unroll
        for (int u = 0; u < KPI; ++u) {
            const int n = n0 + u * step + kg;
            valid[u] = n < c1;
            nn[u] = valid[u] ? n : c1 - 1;  // c1 > c0 here, so c1 - 1 is a valid key
            kr[u] = sk_load_raw<T, KV8>(p.k, k_base + (int64_t)nn[u] * p.ks[2]);
            vr[u] = sk_load_raw<T, KV8>(p.v, v_base + (int64_t)nn[u] * p.vs[2]);
        }
        float s[KPI];
        float mn = mi;
#pragma unroll
        for (int u = 0; u < KPI; ++u) {
            float su = 0.0f;
            if constexpr (std::is_same<T, f16>::value) {
                // fp16: four two-element dot products with fp32 accumulation on the packed pairs
                uint32_t kpk[4];
                sk_pairs8<KV8>(kr[u], kpk);
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    su = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, kpk[j]), __builtin_bit_cast(h2, qpk[j]), su, false);
                su *= p.scale_log2;
            } else {
                float kv[8];
                sk_widen8<T, KV8>(kr[u], kv);
#pragma unroll
                for (int e = 0; e < 8; ++e) su += qf[e] * kv[e];
            }
            // sum over the DL lanes of the key: quad permutes and row mirrors on DPP, no trip through LDS
            if (DL >= 2) su += dpp_mov<0xB1>(su);
            if (DL >= 4) su += dpp_mov<0x4E>(su);
            if (DL >= 8) su += dpp_mov<0x141>(su);
            if (DL >= 16) su += dpp_mov<0x140>(su);
            if (DL >= 32) su += __shfl_xor(su, 16, 64);
            if (p.has_mask) su += sk_mask_value(p.mask, p.mask_dtype, mask_base + (int64_t)nn[u] * p.ms[3], p.clamp);
            if (!valid[u]) su = -INFINITY;
            s[u] = su;
            mn = fmaxf(mn, su);
        }
        const float mu = (mn == -INFINITY) ? 0.0f : mn;
        const float alpha = __builtin_amdgcn_exp2f(mi - mu);
        li *= alpha;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] *= alpha;
#pragma unroll
        for (int u = 0; u < KPI; ++u) {
            // P is rounded to the storage dtype before P·V, as in the tiled kernel and the reference (attention.py:424)
            const float pr = (float)from_float<T>(__builtin_amdgcn_exp2f(s[u] - mu));
            li += pr;
            float vv[8];
            if constexpr (std::is_same<T, f16>::value) {
                uint32_t vpk[4];
                sk_pairs8<KV8>(vr[u], vpk);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const h2 two = __builtin_bit_cast(h2, vpk[j]);
                    vv[2 * j] = (float)two[0];
                    vv[2 * j + 1] = (float)two[1];
                }
            } else {
                sk_widen8<T, KV8>(vr[u], vv);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] += pr * vv[e];
        }
        mi = mn;
    }
    // merge the KPW lane groups of the wave (same dl, different kg)
#pragma unroll
    for (int off = DL; off < 64; off <<= 1) {
        const float m2 = __shfl_xor(mi, off, 64), l2 = __shfl_xor(li, off, 64);
        float a2[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) a2[e] = __shfl_xor(acc[e], off, 64);
        sk_merge(mi, li, acc, m2, l2, a2);
    }
    // merge the 4 waves through LDS
    if (kg == 0) {
        red[wave][dl][0] = mi;
        red[wave][dl][1] = li;
#pragma unroll
        for (int e = 0; e < 8; ++e) red[wave][dl][2 + e] = acc[e];
    }
    __syncthreads();
    if (wave == 0 && kg == 0) {
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            float a2[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) a2[e] = red[w][dl][2 + e];
            sk_merge(mi, li, acc, red[w][dl][0], red[w][dl][1], a2);
        }
        if (p.splits == 1) {
            T *op = static_cast<T *>(p.o) + b * p.os[0] + h * p.os[1] + (int64_t)m * p.os[2];
            const float inv = 1.0f / li;
#pragma unroll
            for (int e = 0; e < 8; ++e) op[(int64_t)(dl * 8 + e) * p.os[3]] = from_float<T>(acc[e] * inv);
        } else {
            float *w = p.ws + ((int64_t)row * p.splits + split) * (p.D + 2);
            if (dl == 0) {
                w[0] = mi;
                w[1] = li;
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) w[2 + dl * 8 + e] = acc[e];
        }
    }
}

// Merge of the key ranges of one row.  256 threads: thread (g, d) sums the ranges g, g + G, ... (G = 256 / D) for
// output feature d, then the G partial sums meet in LDS.  Maxima and sums of all ranges are staged in LDS first so
// that no thread walks a chain of dependent global loads.
template <typename T>
__global__ void __launch_bounds__(256) attention_skinny_part2(const SkinnyParams p) {
    __shared__ float sm[256], sl[256], part[256];
    __shared__ float s_max;
    const int row = blockIdx.x, tid = threadIdx.x;
    const int m = row % p.M, bh = row / p.M, b = bh / p.H, h = bh % p.H;
    const float *w = p.ws + (int64_t)row * p.splits * (p.D + 2);
    if (tid < p.splits) {  // splits <= 256
        sm[tid] = w[(int64_t)tid * (p.D + 2)];
        sl[tid] = w[(int64_t)tid * (p.D + 2) + 1];
    }
    __syncthreads();
    if (tid < 64) {
        float mx = -INFINITY;
        for (int s = tid; s < p.splits; s += 64) mx = fmaxf(mx, sm[s]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        if (tid == 0) s_max = mx;
    }
    __syncthreads();
    const float mx = s_max;
    const int G = 256 / p.D, g = tid / p.D, d = tid % p.D;
    float a = 0.0f;
    if (g < G) {
#pragma unroll 4
        for (int s = g; s < p.splits; s += G) {
            const float f = (sm[s] == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(sm[s] - mx);
            a += w[(int64_t)s * (p.D + 2) + 2 + d] * f;
        }
    }
    part[tid] = a;
    __syncthreads();
    if (tid < p.D) {
        float l = 0.0f;
        for (int s = 0; s < p.splits; ++s) l += (sm[s] == -INFINITY) ? 0.0f : sl[s] * __builtin_amdgcn_exp2f(sm[s] - mx);
        float tot = 0.0f;
        for (int gg = 0; gg < G; ++gg) tot += part[gg * p.D + tid];
        T *op = static_cast<T *>(p.o) + b * p.os[0] + h * p.os[1] + (int64_t)m * p.os[2];
        op[(int64_t)tid * p.os[3]] = from_float<T>(tot / l);
    }
}

// key ranges per row: about `workgroups` workgroups over the whole grid.  With 64 bytes of keys and of values in flight
// per lane, one workgroup per CU reaches the bandwidth for 16-bit storage and two for one-byte storage; more ranges
// only add to the merge.
constexpr int kSkWorkgroups16 = 256, kSkWorkgroups8 = 512;
static int skinny_splits(int64_t rows, int64_t N, int D, int workgroups) {
    const int step = 4 * (64 / (D / 8));
    int64_t want = (workgroups + rows - 1) / rows;
    const int64_t most = (N + step - 1) / step;
    if (want > most) want = most;
    if (want > 64) want = 64;
    return (int)(want < 1 ? 1 : want);
}

template <typename T, bool KV8, int KPI>
static void launch_skinny_part1(const SkinnyParams &p, hipStream_t st) {
    dim3 grid((unsigned)p.splits, (unsigned)(p.B * p.H * p.M));
    switch (p.D / 8) {
        case 1: hipLaunchKernelGGL((attention_skinny_part1<T, 1, KV8, KPI>), grid, dim3(256), 0, st, p); break;
        case 2: hipLaunchKernelGGL((attention_skinny_part1<T, 2, KV8, KPI>), grid, dim3(256), 0, st, p); break;
        case 4: hipLaunchKernelGGL((attention_skinny_part1<T, 4, KV8, KPI>), grid, dim3(256), 0, st, p); break;
        case 8: hipLaunchKernelGGL((attention_skinny_part1<T, 8, KV8, KPI>), grid, dim3(256), 0, st, p); break;
        case 16: hipLaunchKernelGGL((attention_skinny_part1<T, 16, KV8, KPI>), grid, dim3(256), 0, st, p); break;
        default: hipLaunchKernelGGL((attention_skinny_part1<T, 32, KV8, KPI>), grid, dim3(256), 0, st, p); break;
    }
}

template <typename T, bool KV8>
static void launch_skinny(const SkinnyParams &p, hipStream_t st) {
    // keys per lane and trip: 64 bytes of keys and as many of values in flight per lane with either storage
    launch_skinny_part1<T, KV8, KV8 ? 8 : 4>(p, st);
    if (p.splits > 1)
        hipLaunchKernelGGL((attention_skinny_part2<T>), dim3((unsigned)(p.B * p.H * p.M)), dim3(256), 0, st, p);
}

}  // namespace kernl

extern "C" int64_t kernl_attention_skinny_workspace_bytes(int64_t B, int64_t H, int64_t M, int64_t N, int64_t D) {
    using namespace kernl;
    if (B <= 0 || H <= 0 || M <= 0 || N <= 0 || D < 8 || D % 8 != 0) return 0;
    const int64_t rows = B * H * M;
    const int splits = skinny_splits(rows, N, (int)D, kSkWorkgroups8);  // enough for either storage of the keys and values
    return splits > 1 ? rows * splits * (D + 2) * (int64_t)sizeof(float) : 0;
}

static int skinny_entry(const void *q, const void *k, const void *v, void *out, const void *mask, void *workspace,
                        int64_t workspace_bytes, int64_t B, int64_t H, int64_t M, int64_t N, int64_t D,
                        const int64_t q_strides[4], const int64_t k_strides[4], const int64_t v_strides[4],
                        const int64_t o_strides[4], const int64_t mask_sizes[4], const int64_t mask_strides[4],
                        int mask_dtype, float sm_scale, int is_causal, float mask_min_clamp, int dtype, bool kv8,
                        void *stream) {
    using namespace kernl;
    if (q == nullptr || k == nullptr || v == nullptr || out == nullptr || q_strides == nullptr ||
        k_strides == nullptr || v_strides == nullptr || o_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "skinny attention: q, k, v, out and their strides must not be NULL");
    if (B < 0 || H <= 0 || M < 0 || N <= 0 || D <= 0)
        return set_error(KERNL_ERR_INVALID_ARG, "skinny attention: bad sizes B=%lld H=%lld M=%lld N=%lld D=%lld",
                         (long long)B, (long long)H, (long long)M, (long long)N, (long long)D);
    if (dtype != KERNL_F16 && dtype != KERNL_BF16)
        return set_error(KERNL_ERR_UNSUPPORTED, "skinny attention: only f16 and bf16 are supported, got dtype %d", dtype);
    const bool pow2 = (D & (D - 1)) == 0;
    if (D < 8 || D > 256 || !pow2)
        return set_error(KERNL_ERR_UNSUPPORTED, "skinny attention: head size %lld is not a power of two in 8..256",
                         (long long)D);
    auto rows_ok = [](const void *ptr, const int64_t s[4]) {
        return s[3] == 1 && s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0 && aligned16(ptr);
    };
    // one-byte keys and values: 8 of them are an 8-byte load, and their strides count bytes
    auto rows8_ok = [](const void *ptr, const int64_t s[4]) {
        return s[3] == 1 && s[0] % 8 == 0 && s[1] % 8 == 0 && s[2] % 8 == 0 && (reinterpret_cast<uintptr_t>(ptr) & 7) == 0;
    };
    const bool kv_ok = kv8 ? rows8_ok(k, k_strides) && rows8_ok(v, v_strides) : rows_ok(k, k_strides) && rows_ok(v, v_strides);
    if (!rows_ok(q, q_strides) || !kv_ok)
        return set_error(KERNL_ERR_UNSUPPORTED, "skinny attention: q, k, v need unit feature stride and 16-byte aligned rows "
                         "(8-byte aligned rows for one-byte keys and values)");
    if (N > (1 << 24)) return set_error(KERNL_ERR_UNSUPPORTED, "skinny attention: more than 2^24 keys");
    SkinnyParams p;
    p.has_mask = mask != nullptr;
    if (mask != nullptr) {
        if (mask_sizes == nullptr || mask_strides == nullptr)
            return set_error(KERNL_ERR_INVALID_ARG, "skinny attention: mask given without sizes/strides");
        if ((mask_sizes[0] != B && mask_sizes[0] != 1) || (mask_sizes[1] != H && mask_sizes[1] != 1) ||
            (mask_sizes[2] != M && mask_sizes[2] != 1) || mask_sizes[3] != N)
            return set_error(KERNL_ERR_INVALID_ARG, "skinny attention: mask sizes do not broadcast to [B,H,M,N]");
        if (mask_dtype != KERNL_F16 && mask_dtype != KERNL_BF16 && mask_dtype != KERNL_F32)
            return set_error(KERNL_ERR_UNSUPPORTED, "skinny attention: unknown mask dtype %d", mask_dtype);
        p.ms[0] = mask_sizes[0] == 1 ? 0 : mask_strides[0];
        p.ms[1] = mask_sizes[1] == 1 ? 0 : mask_strides[1];
        p.ms[2] = mask_sizes[2] == 1 ? 0 : mask_strides[2];
        p.ms[3] = mask_strides[3];
    } else {
        p.ms[0] = p.ms[1] = p.ms[2] = p.ms[3] = 0;
    }
    if (B == 0 || M == 0) return KERNL_OK;

    const int64_t rows = B * H * M;
    if (rows > 65535) return set_error(KERNL_ERR_UNSUPPORTED, "skinny attention: more than 65535 (batch, head, query) rows");
    int splits = skinny_splits(rows, N, (int)D, kv8 ? kSkWorkgroups8 : kSkWorkgroups16);
    if (splits > 1) {
        const int64_t per_split = rows * (D + 2) * (int64_t)sizeof(float);
        const int64_t fit = workspace != nullptr ? workspace_bytes / per_split : 0;
        if (fit < splits) splits = (int)(fit < 1 ? 1 : fit);  // a small workspace only costs parallelism
    }
    p.q = q; p.k = k; p.v = v; p.o = out; p.mask = mask;
    p.ws = static_cast<float *>(workspace);
    p.B = (int)B; p.H = (int)H; p.M = (int)M; p.N = (int)N; p.D = (int)D; p.splits = splits;
    for (int i = 0; i < 4; ++i) {
        p.qs[i] = q_strides[i]; p.ks[i] = k_strides[i]; p.vs[i] = v_strides[i]; p.os[i] = o_strides[i];
    }
    p.mask_dtype = mask_dtype;
    p.causal = is_causal != 0;
    p.kv8 = kv8 ? 1 : 0;
    p.scale_log2 = sm_scale * 1.4426950408889634f;
    p.clamp = mask_min_clamp;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (kv8) {
        if (dtype == KERNL_F16) launch_skinny<f16, true>(p, st);
        else launch_skinny<bf16, true>(p, st);
    } else {
        if (dtype == KERNL_F16) launch_skinny<f16, false>(p, st);
        else launch_skinny<bf16, false>(p, st);
    }
    return check_launch("attention (skinny)");
}

// ----------------------------------------------------------------------------------------------------
// Entry point that allocates nothing: the partial results live in a file-scope device array instead of a
// caller-provided workspace.  Every GPU holds its own copy of the array at its own address; the address is
// looked up once per device (with that device current) and kept.
// ----------------------------------------------------------------------------------------------------
namespace kernl {

static constexpr int64_t kSkScratchBytes = 512ll << 10;
static constexpr int kSkMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kSkScratchBytes];

// per-device address of `scratch`; written once per device under the lock, read through an acquire load
static void *g_scratch_ptr[kSkMaxDevices] = {nullptr};
static int g_scratch_lock = 0;

static int skinny_scratch(void **ptr_out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return set_error(KERNL_ERR_LAUNCH, "skinny attention (static): hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kSkMaxDevices)
        return set_error(KERNL_ERR_UNSUPPORTED, "skinny attention (static): device index %d outside 0..%d", dev, kSkMaxDevices - 1);
    void *ptr = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (ptr == nullptr) {
        while (__atomic_exchange_n(&g_scratch_lock, 1, __ATOMIC_ACQUIRE) != 0) {
        }
        ptr = g_scratch_ptr[dev];
        if (ptr == nullptr) {
            e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
            if (e == hipSuccess && ptr != nullptr) __atomic_store_n(&g_scratch_ptr[dev], ptr, __ATOMIC_RELEASE);
        }
        __atomic_store_n(&g_scratch_lock, 0, __ATOMIC_RELEASE);
        if (e != hipSuccess || ptr == nullptr)
            return set_error(KERNL_ERR_LAUNCH, "skinny attention (static): hipGetSymbolAddress: %s", hipGetErrorString(e));
    }
    *ptr_out = ptr;
    return KERNL_OK;
}

}  // namespace kernl

extern "C" int64_t kernl_attention_skinny_static_max_bytes(void) { return kernl::kSkScratchBytes; }

// The once-per-device address lookup on its own, for callers whose first use of the static entry point would fall
// inside a stream capture: a symbol lookup may load the code object, which a capturing stream does not allow.
extern "C" int kernl_attention_skinny_static_init(void) {
    void *ptr = nullptr;
    return kernl::skinny_scratch(&ptr);
}

extern "C" int kernl_attention_skinny_static_fwd(const void *q, const void *k, const void *v, void *out,
                                                 const void *mask, int64_t B, int64_t H, int64_t M, int64_t N,
                                                 int64_t D, const int64_t q_strides[4], const int64_t k_strides[4],
                                                 const int64_t v_strides[4], const int64_t o_strides[4],
                                                 const int64_t mask_sizes[4], const int64_t mask_strides[4],
                                                 int mask_dtype, float sm_scale, int is_causal, float mask_min_clamp,
                                                 int dtype, void *stream) {
    using namespace kernl;
    // the same number of key ranges as kernl_attention_skinny_fwd takes with a workspace of the reported size, so
    // both entry points add the ranges in the same order; problems whose partial results do not fit are refused
    const int64_t need = kernl_attention_skinny_workspace_bytes(B, H, M, N, D);
    if (need > kSkScratchBytes)
        return set_error(KERNL_ERR_UNSUPPORTED,
                         "skinny attention (static): partial results need %lld bytes, the static buffer holds %lld; "
                         "use kernl_attention_skinny_fwd with a workspace",
                         (long long)need, (long long)kSkScratchBytes);
    void *ws = nullptr;
    if (need > 0) {
        const int st = skinny_scratch(&ws);
        if (st != KERNL_OK) return st;
    }
    return skinny_entry(q, k, v, out, mask, ws, need, B, H, M, N, D, q_strides, k_strides, v_strides, o_strides,
                        mask_sizes, mask_strides, mask_dtype, sm_scale, is_causal, mask_min_clamp, dtype, false, stream);
}

extern "C" int kernl_attention_skinny_fwd(const void *q, const void *k, const void *v, void *out, const void *mask,
                                          void *workspace, int64_t workspace_bytes, int64_t B, int64_t H, int64_t M,
                                          int64_t N, int64_t D, const int64_t q_strides[4],
                                          const int64_t k_strides[4], const int64_t v_strides[4],
                                          const int64_t o_strides[4], const int64_t mask_sizes[4],
                                          const int64_t mask_strides[4], int mask_dtype, float sm_scale, int is_causal,
                                          float mask_min_clamp, int dtype, void *stream) {
    return skinny_entry(q, k, v, out, mask, workspace, workspace_bytes, B, H, M, N, D, q_strides, k_strides, v_strides,
                        o_strides, mask_sizes, mask_strides, mask_dtype, sm_scale, is_causal, mask_min_clamp, dtype,
                        false, stream);
}

extern "C" int kernl_attention_skinny_kv8_fwd(const void *q, const void *k, const void *v, void *out, const void *mask,
                                              void *workspace, int64_t workspace_bytes, int64_t B, int64_t H, int64_t M,
                                              int64_t N, int64_t D, const int64_t q_strides[4],
                                              const int64_t k_strides[4], const int64_t v_strides[4],
                                              const int64_t o_strides[4], const int64_t mask_sizes[4],
                                              const int64_t mask_strides[4], int mask_dtype, float sm_scale,
                                              int is_causal, float mask_min_clamp, int dtype, void *stream) {
    return skinny_entry(q, k, v, out, mask, workspace, workspace_bytes, B, H, M, N, D, q_strides, k_strides, v_strides,
                        o_strides, mask_sizes, mask_strides, mask_dtype, sm_scale, is_causal, mask_min_clamp, dtype,
                        true, stream);
}
