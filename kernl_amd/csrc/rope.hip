// Rotary position embedding, half-split convention:  out = x·cos + rotate_half(x)·sin  with
// rotate_half(x)[d] = -x[d + D/2] for d < D/2 and x[d - D/2] otherwise — the form Hugging Face decoders trace into
// eight element-wise kernels per tensor (two slices, neg, cat, two muls, add).  The reference fuses the same rotation,
// in Meta's interleaved-pair convention, into its query/key projection (experimental/llama-v2/kernel/
// fused_kernel_proj_qkv.py:69-100, `rbe_triton`; eager form experimental/llama-v2/llama/model.py:78-88).
//
// HBM bound: x is read once and written once (cos/sin are [S, D] tables shared by all heads and stay in cache).  A
// thread owns one 16-byte chunk of the lower half of a row and its partner chunk D/2 further: two loads, two stores,
// fp32 arithmetic, one rounding to the storage dtype.
#include <algorithm>

#include "common.h"

namespace kernl {

struct RopeParams {
    const void *x, *cos, *sin;
    void *out;
    int B, H, S, D;
    int64_t xs[4], os[4], cs[4], ss[4];  // element strides {batch, head, position, feature}; 0 on broadcast dims
    int cs_dtype;
};

__device__ __forceinline__ float rope_table(const void *t, int dtype, int64_t off) {
    if (dtype == KERNL_F32) return static_cast<const float *>(t)[off];
    if (dtype == KERNL_F16) return (float)static_cast<const f16 *>(t)[off];
    return (float)static_cast<const bf16 *>(t)[off];
}

// VEC: feature stride 1 and 16-byte aligned rows everywhere, tables of the same 16-bit dtype as x or fp32
template <typename T, bool VEC, bool TABLE_F32>
__global__ void __launch_bounds__(256) rope_kernel(const RopeParams p) {
    const int half = p.D / 2;
    const int chunks = VEC ? half / 8 : half;  // work items per row
    const int64_t total = (int64_t)p.B * p.H * p.S * chunks;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        const int c = (int)(i % chunks);
        int64_t r = i / chunks;
        const int s = (int)(r % p.S);
        r /= p.S;
        const int h = (int)(r % p.H), b = (int)(r / p.H);
        const T *xr = static_cast<const T *>(p.x) + b * p.xs[0] + h * p.xs[1] + (int64_t)s * p.xs[2];
        T *orow = static_cast<T *>(p.out) + b * p.os[0] + h * p.os[1] + (int64_t)s * p.os[2];
        const int64_t cbase = b * p.cs[0] + h * p.cs[1] + (int64_t)s * p.cs[2];
        const int64_t sbase = b * p.ss[0] + h * p.ss[1] + (int64_t)s * p.ss[2];
        if constexpr (VEC) {
            typedef typename Vec8<T>::type vec8;
            const int d = c * 8;
            const vec8 lo = *reinterpret_cast<const vec8 *>(xr + d);
            const vec8 hi = *reinterpret_cast<const vec8 *>(xr + d + half);
            float cl[8], ch[8], sl[8], sh[8];
            if (TABLE_F32) {
                const float *cp = static_cast<const float *>(p.cos) + cbase, *sp = static_cast<const float *>(p.sin) + sbase;
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const f32x4 a = *reinterpret_cast<const f32x4 *>(cp + d + 4 * q);
                    const f32x4 bq = *reinterpret_cast<const f32x4 *>(cp + d + half + 4 * q);
                    const f32x4 e = *reinterpret_cast<const f32x4 *>(sp + d + 4 * q);
                    const f32x4 f = *reinterpret_cast<const f32x4 *>(sp + d + half + 4 * q);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        cl[4 * q + k] = a[k];
                        ch[4 * q + k] = bq[k];
                        sl[4 * q + k] = e[k];
                        sh[4 * q + k] = f[k];
                    }
                }
            } else {
                const T *cp = static_cast<const T *>(p.cos) + cbase, *sp = static_cast<const T *>(p.sin) + sbase;
                const vec8 a = *reinterpret_cast<const vec8 *>(cp + d), bq = *reinterpret_cast<const vec8 *>(cp + d + half);
                const vec8 e = *reinterpret_cast<const vec8 *>(sp + d), f = *reinterpret_cast<const vec8 *>(sp + d + half);
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    cl[k] = (float)a[k];
                    ch[k] = (float)bq[k];
                    sl[k] = (float)e[k];
                    sh[k] = (float)f[k];
                }
            }
            vec8 olo, ohi;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const float xl = (float)lo[k], xh = (float)hi[k];
                olo[k] = from_float<T>(xl * cl[k] - xh * sl[k]);
                ohi[k] = from_float<T>(xh * ch[k] + xl * sh[k]);
            }
            *reinterpret_cast<vec8 *>(orow + d) = olo;
            *reinterpret_cast<vec8 *>(orow + d + half) = ohi;
        } else {
            const int d = c;
            const float xl = to_float(xr[(int64_t)d * p.xs[3]]), xh = to_float(xr[(int64_t)(d + half) * p.xs[3]]);
            const float cl = rope_table(p.cos, p.cs_dtype, cbase + (int64_t)d * p.cs[3]);
            const float ch = rope_table(p.cos, p.cs_dtype, cbase + (int64_t)(d + half) * p.cs[3]);
            const float sl = rope_table(p.sin, p.cs_dtype, sbase + (int64_t)d * p.ss[3]);
            const float sh = rope_table(p.sin, p.cs_dtype, sbase + (int64_t)(d + half) * p.ss[3]);
            orow[(int64_t)d * p.os[3]] = from_float<T>(xl * cl - xh * sl);
            orow[(int64_t)(d + half) * p.os[3]] = from_float<T>(xh * ch + xl * sh);
        }
    }
}

template <typename T>
static void launch_rope(const RopeParams &p, bool vec, bool table_f32, hipStream_t st) {
    const int64_t items = (int64_t)p.B * p.H * p.S * (vec ? p.D / 16 : p.D / 2);
    int64_t blocks = (items + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    const dim3 grid((unsigned)blocks), block(256);
    if (vec && table_f32) hipLaunchKernelGGL((rope_kernel<T, true, true>), grid, block, 0, st, p);
    else if (vec) hipLaunchKernelGGL((rope_kernel<T, true, false>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((rope_kernel<T, false, false>), grid, block, 0, st, p);
}

}  // namespace kernl

extern "C" int kernl_rope_fwd(const void *x, const void *cos, const void *sin, void *out, int64_t B, int64_t H,
                              int64_t S, int64_t D, const int64_t x_strides[4], const int64_t out_strides[4],
                              const int64_t table_sizes[4], const int64_t cos_strides[4],
                              const int64_t sin_strides[4], int table_dtype, int dtype, void *stream) {
    using namespace kernl;
    if (x == nullptr || cos == nullptr || sin == nullptr || out == nullptr || x_strides == nullptr ||
        out_strides == nullptr || table_sizes == nullptr || cos_strides == nullptr || sin_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "rope: pointers and stride arrays must not be NULL");
    if (B < 0 || H <= 0 || S < 0 || D <= 0 || D % 2 != 0)
        return set_error(KERNL_ERR_INVALID_ARG, "rope: bad sizes B=%lld H=%lld S=%lld D=%lld (D must be even)",
                         (long long)B, (long long)H, (long long)S, (long long)D);
    if (dtype != KERNL_F16 && dtype != KERNL_BF16 && dtype != KERNL_F32)
        return set_error(KERNL_ERR_UNSUPPORTED, "rope: unknown dtype %d", dtype);
    if (table_dtype != KERNL_F16 && table_dtype != KERNL_BF16 && table_dtype != KERNL_F32)
        return set_error(KERNL_ERR_UNSUPPORTED, "rope: unknown table dtype %d", table_dtype);
    if ((table_sizes[0] != B && table_sizes[0] != 1) || (table_sizes[1] != H && table_sizes[1] != 1) ||
        table_sizes[2] != S || table_sizes[3] != D)
        return set_error(KERNL_ERR_INVALID_ARG, "rope: cos/sin sizes must be [B|1, H|1, S, D]");
    if (B * H * S * D >= (1ll << 40)) return set_error(KERNL_ERR_UNSUPPORTED, "rope: tensor too large");
    if (B == 0 || S == 0) return KERNL_OK;
    RopeParams p;
    p.x = x; p.cos = cos; p.sin = sin; p.out = out;
    p.B = (int)B; p.H = (int)H; p.S = (int)S; p.D = (int)D;
    for (int i = 0; i < 4; ++i) {
        p.xs[i] = x_strides[i];
        p.os[i] = out_strides[i];
        const bool broadcast = i < 2 && table_sizes[i] == 1;
        p.cs[i] = broadcast ? 0 : cos_strides[i];
        p.ss[i] = broadcast ? 0 : sin_strides[i];
    }
    p.cs_dtype = table_dtype;
    auto rows16 = [](const void *ptr, const int64_t s[4], int64_t elem) {
        const int64_t per16 = 16 / elem;
        return s[3] == 1 && s[0] % per16 == 0 && s[1] % per16 == 0 && s[2] % per16 == 0 && aligned16(ptr);
    };
    const int64_t telem = table_dtype == KERNL_F32 ? 4 : 2;
    const bool vec = dtype != KERNL_F32 && D % 16 == 0 && rows16(x, p.xs, 2) && rows16(out, p.os, 2) && rows16(cos, p.cs, telem) &&
                     rows16(sin, p.ss, telem) && (table_dtype == KERNL_F32 || table_dtype == dtype);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == KERNL_F16) launch_rope<f16>(p, vec, table_dtype == KERNL_F32, st);
    else if (dtype == KERNL_BF16) launch_rope<bf16>(p, vec, table_dtype == KERNL_F32, st);
    else hipLaunchKernelGGL((rope_kernel<float, false, false>), dim3((unsigned)std::min<int64_t>((B * H * S * (D / 2) + 255) / 256, 16384)),
                            dim3(256), 0, st, p);
    return check_launch("rope");
}
