// Rate probes: what this chip SUSTAINS on the instruction mixes and memory streams the kernels of this library are
// made of, measured on the box the benchmark runs on.  The published peaks (2.5 PFLOP/s dense fp16 at the 2.4 GHz
// boost clock, 8 TB/s) are what roofline fractions are divided by; these probes say how much of that a register-only
// loop, or a plain streaming pass, reaches on the same GPU at the same moment — and at which shader clock.
//
//   kind 0  v_mfma_f32_32x32x16_f16, operands and 256 accumulator registers in registers only, random fp16 data,
//           one wave per SIMD on every CU (the geometry of the 8-wave linear kernels and of attention)
//   kind 1  v_mfma_f32_16x16x32_f16, same geometry (the wide linear kernels' instruction)
//   kind 2  kind 0 on all-zero operands: the same instruction stream without data toggling
//   kind 3  the attention tile loop's mix, one or two waves per SIMD: per 32x32x16 MFMA two v_exp_f32 and four plain
//           VALU instructions on registers that depend on nothing the MFMAs produce
//   kind 4  read-only pass over a buffer (16-byte loads, every byte once)
//   kind 5  copy of a buffer (16-byte loads and stores)
//
// Every workgroup's first lane records the shader-clock and the 100 MHz wall-clock ticks its loop took; their ratio is
// the clock the loop sustained.  The host side times the launch with events and turns iterations into flops or bytes.
#include "common.h"

namespace kernl {

typedef unsigned long long u64;

__device__ __forceinline__ void probe_stamp(u64 &shader, u64 &wall) {
    wall = wall_clock64();
    shader = clock64();
}

template <int SHAPE, bool ZERO>
__global__ void __launch_bounds__(256, 1) probe_mfma_kernel(const f16x8 *__restrict__ src, int iters, u64 *__restrict__ stats,
                                                            float *__restrict__ sink) {
    f16x8 fa[8], fb[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        fa[j] = src[((blockIdx.x & 255) * 16 + j) * 256 + threadIdx.x];
        fb[j] = src[((blockIdx.x & 255) * 16 + 8 + j) * 256 + threadIdx.x];
        if (ZERO) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                fa[j][e] = (f16)0.0f;
                fb[j][e] = (f16)0.0f;
            }
        }
    }
    float s = 0.0f;
    u64 c0, w0, c1, w1;
    if (SHAPE == 32) {
        f32x16 c[16];
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) c[i][v] = 0.0f;
        probe_stamp(c0, w0);
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int m = 0; m < 16; ++m)
                    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c[m]) : "v"(fa[(m % 4) + 4 * h]), "v"(fb[(m / 4) + 4 * h]));
        }
        probe_stamp(c1, w1);
#pragma unroll
        for (int i = 0; i < 16; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) s += c[i][v];
    } else {
        f32x4_acc c[64];
#pragma unroll
        for (int i = 0; i < 64; ++i) c[i] = f32x4_acc{0.0f, 0.0f, 0.0f, 0.0f};
        probe_stamp(c0, w0);
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int m = 0; m < 64; ++m)
                asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c[m]) : "v"(fa[m % 8]), "v"(fb[m / 8]));
        }
        probe_stamp(c1, w1);
#pragma unroll
        for (int i = 0; i < 64; ++i)
#pragma unroll
            for (int v = 0; v < 4; ++v) s += c[i][v];
    }
    if (threadIdx.x == 0) {
        stats[2 * blockIdx.x] = c1 - c0;
        stats[2 * blockIdx.x + 1] = w1 - w0;
    }
    sink[blockIdx.x * 256 + threadIdx.x] = s;
}

// 16 MFMAs (32x32x16) per iteration on four independent accumulators, each followed by two exponentials and four
// multiply-adds on private registers: one key tile of the attention loop without its memory traffic.
__global__ void __launch_bounds__(256, 2) probe_mix_kernel(const f16x8 *__restrict__ src, int iters, u64 *__restrict__ stats,
                                                           float *__restrict__ sink) {
    f16x8 fa[4], fb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        fa[j] = src[((blockIdx.x & 255) * 16 + j) * 256 + threadIdx.x];
        fb[j] = src[((blockIdx.x & 255) * 16 + 8 + j) * 256 + threadIdx.x];
    }
    f32x16 c[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) c[i][v] = 0.0f;
    // e: arguments of the exponentials (negative fractions, rewritten once per iteration), y: their results in (0.5, 1],
    // z: running sums of products of results — nothing overflows and nothing depends on the MFMAs
    float e[4], y[4], z[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        e[i] = -0.001f * (float)(threadIdx.x + i);
        y[i] = 1.0f;
        z[i] = 0.0f;
    }
    u64 c0, w0, c1, w1;
    probe_stamp(c0, w0);
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int m = 0; m < 16; ++m) {
            asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c[m % 4]) : "v"(fa[m % 4]), "v"(fb[(m / 4) % 4]));
            asm volatile("v_exp_f32 %0, %1" : "=v"(y[(2 * m) % 4]) : "v"(e[(2 * m) % 4]));
            asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(z[0]) : "v"(y[1]), "v"(y[2]));
            asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(z[1]) : "v"(y[2]), "v"(y[3]));
            asm volatile("v_exp_f32 %0, %1" : "=v"(y[(2 * m + 1) % 4]) : "v"(e[(2 * m + 1) % 4]));
            asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(z[2]) : "v"(y[3]), "v"(y[0]));
            asm volatile("v_fma_f32 %0, %1, %2, %0" : "+v"(z[3]) : "v"(y[0]), "v"(y[1]));
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) e[i] = -__builtin_amdgcn_fractf(z[i]);
    }
    probe_stamp(c1, w1);
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) s += c[i][v];
#pragma unroll
    for (int i = 0; i < 4; ++i) s += z[i] + y[i];
    if (threadIdx.x == 0) {
        stats[2 * blockIdx.x] = c1 - c0;
        stats[2 * blockIdx.x + 1] = w1 - w0;
    }
    sink[blockIdx.x * 256 + threadIdx.x] = s;
}

// Streaming passes: thread t of workgroup b walks chunks t + 256 (b + grid * i); four 16-byte loads are in flight per
// lane before the first is used.
template <bool COPY>
__global__ void __launch_bounds__(256) probe_stream_kernel(const u32x4 *__restrict__ src, u32x4 *__restrict__ dst, int64_t chunks,
                                                           u64 *__restrict__ stats, float *__restrict__ sink) {
    u64 c0, w0, c1, w1;
    probe_stamp(c0, w0);
    const int64_t stride = (int64_t)gridDim.x * 256;
    u32x4 acc = {0, 0, 0, 0};
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    for (; i + 3 * stride < chunks; i += 4 * stride) {
        const u32x4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
        if (COPY) {
            dst[i] = a;
            dst[i + stride] = b;
            dst[i + 2 * stride] = c;
            dst[i + 3 * stride] = d;
        } else {
            acc ^= a ^ b ^ c ^ d;
        }
    }
    for (; i < chunks; i += stride) {
        const u32x4 a = src[i];
        if (COPY) dst[i] = a;
        else acc ^= a;
    }
    probe_stamp(c1, w1);
    if (threadIdx.x == 0) {
        stats[2 * blockIdx.x] = c1 - c0;
        stats[2 * blockIdx.x + 1] = w1 - w0;
    }
    if (!COPY) sink[(blockIdx.x & 511) * 256 + threadIdx.x] = __builtin_bit_cast(float, acc[0] ^ acc[1] ^ acc[2] ^ acc[3]);
}

}  // namespace kernl

extern "C" int kernl_probe_rate(int kind, int iters, int workgroups, const void *src, void *dst, int64_t bytes, void *stats,
                                void *sink, void *stream) {
    using namespace kernl;
    if (src == nullptr || stats == nullptr || sink == nullptr) return set_error(KERNL_ERR_INVALID_ARG, "probe: src, stats and sink must not be NULL");
    if (workgroups < 1 || workgroups > 512 * 16) return set_error(KERNL_ERR_INVALID_ARG, "probe: 1 .. 8192 workgroups, got %d", workgroups);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const f16x8 *s8 = static_cast<const f16x8 *>(src);
    u64 *stp = static_cast<u64 *>(stats);
    float *sk = static_cast<float *>(sink);
    dim3 grid((unsigned)workgroups), block(256);
    if (kind <= 3) {
        // the operand table: 256 workgroups x 16 fragments x 256 lanes x 16 bytes
        if (bytes < (int64_t)256 * 16 * 256 * 16) return set_error(KERNL_ERR_INVALID_ARG, "probe: the operand table needs 16 MiB, got %lld bytes", (long long)bytes);
        if (iters < 1) return set_error(KERNL_ERR_INVALID_ARG, "probe: iters must be positive");
    }
    switch (kind) {
    case 0: hipLaunchKernelGGL((probe_mfma_kernel<32, false>), grid, block, 0, st, s8, iters, stp, sk); break;
    case 1: hipLaunchKernelGGL((probe_mfma_kernel<16, false>), grid, block, 0, st, s8, iters, stp, sk); break;
    case 2: hipLaunchKernelGGL((probe_mfma_kernel<32, true>), grid, block, 0, st, s8, iters, stp, sk); break;
    case 3: hipLaunchKernelGGL(probe_mix_kernel, grid, block, 0, st, s8, iters, stp, sk); break;
    case 4:
    case 5:
        if (bytes < 16 || (bytes & 15) != 0 || !aligned16(src)) return set_error(KERNL_ERR_INVALID_ARG, "probe: a 16-byte aligned buffer of a multiple of 16 bytes");
        if (kind == 5 && (dst == nullptr || !aligned16(dst))) return set_error(KERNL_ERR_INVALID_ARG, "probe: copy needs a 16-byte aligned destination");
        if (kind == 4)
            hipLaunchKernelGGL((probe_stream_kernel<false>), grid, block, 0, st, static_cast<const u32x4 *>(src), nullptr, bytes / 16, stp, sk);
        else
            hipLaunchKernelGGL((probe_stream_kernel<true>), grid, block, 0, st, static_cast<const u32x4 *>(src), static_cast<u32x4 *>(dst), bytes / 16, stp, sk);
        break;
    default: return set_error(KERNL_ERR_INVALID_ARG, "probe: unknown kind %d", kind);
    }
    return check_launch("rate probe");
}
