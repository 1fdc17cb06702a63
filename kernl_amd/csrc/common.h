// Shared device/host helpers for the gfx950 kernels: vector types, MFMA wrappers, wave64 reductions,
// LDS swizzles and the thread-local error slot behind kernl_last_error_string().
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/kernl_hip.h"
#include "../../include/kernl_hip_test.h"
#include "index_math.h"

namespace kernl {

// ----------------------------------------------------------------------------------------------------
// vector types
// ----------------------------------------------------------------------------------------------------
typedef _Float16 f16;
typedef __bf16 bf16;
typedef f16 f16x2 __attribute__((ext_vector_type(2)));
typedef f16 f16x4 __attribute__((ext_vector_type(4)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x3 __attribute__((ext_vector_type(3), aligned(4)));  // 12 bytes at any dword boundary

static constexpr int kWave = 64;

// compile-time constants passed as (empty) arguments to generic lambdas
template <bool B>
struct BoolC {
    static constexpr bool value = B;
};
template <int I>
struct IntC {
    static constexpr int value = I;
};

// 16-bit storage types map to their 8-wide MFMA operand vector.
template <typename T>
struct Vec8;
template <>
struct Vec8<f16> {
    typedef f16x8 type;
};
template <>
struct Vec8<bf16> {
    typedef bf16x8 type;
};

// D[32x32] += A[32x16] * B[16x32], fp32 accumulate (v_mfma_f32_32x32x16_{f16,bf16}, 8 passes).
// Operand layout, lane l of the wave: A holds row (l % 32), k = 8*(l/32) .. +7; B holds column (l % 32),
// same k range; D element v (0..15) of lane l is row 8*(v/4) + 4*(l/32) + (v%4), column (l % 32).
__device__ __forceinline__ f32x16 mfma32(f16x8 a, f16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// D[16x16] += A[16x32] * B[32x16], fp32 accumulate (v_mfma_f32_16x16x32_{f16,bf16}, 4 passes).  Same flops per cycle
// as the 32x32x16 form with a quarter of the accumulator traffic per flop: under the board's power limit it sustains
// a higher clock.  Lane l: A holds row (l % 16), k = 8*(l/16) .. +7; B holds column (l % 16), same k range; D element
// e (0..3) of lane l is row 4*(l/16) + e, column (l % 16).
typedef float f32x4_acc __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4_acc mfma16(f16x8 a, f16x8 b, f32x4_acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ f32x4_acc mfma16(bf16x8 a, bf16x8 b, f32x4_acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// The same instruction with the accumulator pinned to the accumulation registers and updated in place.  With 64
// four-register accumulators per wave the register allocator otherwise migrates some of them to ordinary registers and
// copies them back at the loop head.
__device__ __forceinline__ void mfma16_inplace(f16x8 a, f16x8 b, f32x4_acc &c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma16_inplace(bf16x8 a, bf16x8 b, f32x4_acc &c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
// First product of an output tile: the accumulator is WRITTEN as a * b + 0 (the inline constant), so a tile never
// zeroes its 256 accumulator registers.
__device__ __forceinline__ void mfma16_start(f16x8 a, f16x8 b, f32x4_acc &c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma16_start(bf16x8 a, bf16x8 b, f32x4_acc &c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
}
// To the compiler the instruction above is opaque text: it inserts none of the wait states that a read of a matrix
// instruction's result needs (11 after an 8-pass instruction), so the copies out of the accumulation registers with
// which an epilogue begins could follow the last MFMA directly and see registers that some lanes' results have not
// reached yet.  Call this between the last mfma16_inplace and the first use of the accumulators: 16 wait states, then
// every accumulator passes through an empty statement that the copies depend on (volatile statements keep their
// order, and a copy cannot move above the statement that produces its source).
template <int NA, int NB_>
__device__ __forceinline__ void mfma16_inplace_results_landed(f32x4_acc (&acc)[NA][NB_]) {
    asm volatile("s_nop 15");
#pragma unroll
    for (int i = 0; i < NA; ++i)
#pragma unroll
        for (int j = 0; j < NB_; ++j) asm volatile("" : "+a"(acc[i][j]));
}

// ----------------------------------------------------------------------------------------------------
// conversions
// ----------------------------------------------------------------------------------------------------
__device__ __forceinline__ float to_float(f16 x) { return (float)x; }
__device__ __forceinline__ float to_float(bf16 x) { return (float)x; }
__device__ __forceinline__ float to_float(float x) { return x; }

// element `off` of a table of fp32, fp16 or bf16 values (the rotation tables of the decoding kernels)
__device__ __forceinline__ float table_value(const void *t, int dtype, int64_t off) {
    if (dtype == KERNL_F32) return static_cast<const float *>(t)[off];
    if (dtype == KERNL_F16) return (float)static_cast<const f16 *>(t)[off];
    return (float)static_cast<const bf16 *>(t)[off];
}

template <typename T>
__device__ __forceinline__ T from_float(float x);
template <>
__device__ __forceinline__ f16 from_float<f16>(float x) {
    return (f16)x;
}
template <>
__device__ __forceinline__ bf16 from_float<bf16>(float x) {
    return (bf16)x;
}
template <>
__device__ __forceinline__ float from_float<float>(float x) {
    return x;
}

// Two fp32 -> packed pair of 16-bit values in one 32-bit register (round to nearest even).
template <typename T>
__device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <>
__device__ __forceinline__ uint32_t pack2<f16>(float lo, float hi) {
    f16x2 p = {(f16)lo, (f16)hi};
    return __builtin_bit_cast(uint32_t, p);
}
template <>
__device__ __forceinline__ uint32_t pack2<bf16>(float lo, float hi) {
    bf16x2 p = {(bf16)lo, (bf16)hi};
    return __builtin_bit_cast(uint32_t, p);
}

// acc + lo + hi of a packed pair of 16-bit values, accumulated in fp32 (v_dot2c_f32_{f16,bf16} against (1, 1)).
template <typename T>
__device__ __forceinline__ float pair_sum_acc(uint32_t packed, float acc);
template <>
__device__ __forceinline__ float pair_sum_acc<f16>(uint32_t packed, float acc) {
    const f16x2 ones = {(f16)1.0f, (f16)1.0f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, packed), ones, acc, false);
}
template <>
__device__ __forceinline__ float pair_sum_acc<bf16>(uint32_t packed, float acc) {
    const bf16x2 ones = {(bf16)1.0f, (bf16)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, packed), ones, acc, false);
}

// ----------------------------------------------------------------------------------------------------
// wave64 reductions: quad permutes and row mirrors on DPP, the last two steps through scalar lane reads.
// Every lane receives the full result.
// ----------------------------------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}

__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_mov<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_mov<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_mov<0x141>(v);  // row_half_mirror
    v += dpp_mov<0x140>(v);  // row_mirror
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return (r0 + r1) + (r2 + r3);
}

__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_mov<0xB1>(v));
    v = fmaxf(v, dpp_mov<0x4E>(v));
    v = fmaxf(v, dpp_mov<0x141>(v));
    v = fmaxf(v, dpp_mov<0x140>(v));
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
}

// sums over the lower and over the upper 32 lanes of the wave, both to every lane
__device__ __forceinline__ void half_wave_sums(float v, float &lo, float &hi) {
    v = row16_sum(v);
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    lo = r0 + r1;
    hi = r2 + r3;
}

// Both 32-lane halves of the wave exchange a value: afterwards every lane has the value its counterpart in the
// lower half held (`lo`) and the one its counterpart in the upper half held (`hi`).
// v_permlane32_swap exchanges the upper 32 lanes of its first operand with the lower 32 lanes of its second; fed
// the same value twice, the first result is the lower half replicated, the second the upper half replicated.
__device__ __forceinline__ void halves32(float v, float &lo, float &hi) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, v);
    const auto r = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
    lo = __builtin_bit_cast(float, (uint32_t)r[0]);
    hi = __builtin_bit_cast(float, (uint32_t)r[1]);
}
__device__ __forceinline__ float halves32_max(float v) {
    float lo, hi;
    halves32(v, lo, hi);
    return fmaxf(lo, hi);
}
__device__ __forceinline__ float halves32_sum(float v) {
    float lo, hi;
    halves32(v, lo, hi);
    return lo + hi;
}

// ----------------------------------------------------------------------------------------------------
// host side
// ----------------------------------------------------------------------------------------------------
int set_error(int status, const char *fmt, ...);
int check_launch(const char *what);

__host__ __device__ static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace kernl
