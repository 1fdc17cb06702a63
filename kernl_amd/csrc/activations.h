// Activations of the linear kernels' epilogues, applied to the fp32 accumulator.
#pragma once

#include "common.h"

namespace kernl {

// ----------------------------------------------------------------------------------------------------
// activations on the fp32 accumulator (reference: src/kernl/implementations/activation_func.py:28-49)
// ----------------------------------------------------------------------------------------------------
static constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ float act_tanh(float x) {
    // tanh(x) = 1 - 2 / (exp(2x) + 1); saturates correctly through exp2 -> inf / 0.
    const float t = __builtin_amdgcn_exp2f(x * (2.0f * kLog2e));
    return 1.0f - 2.0f * __builtin_amdgcn_rcpf(t + 1.0f);
}
__device__ __forceinline__ float act_sigmoid(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-kLog2e * x));
}
__device__ __forceinline__ float act_gelu_tanh(float x) {
    // 0.5 x (1 + tanh(u)) = x * sigmoid(2u) = x / (1 + 2^(-log2(e) 2u)),  u = sqrt(2/pi) (x + 0.044715 x^3);
    // the factor -log2(e) is folded into the two coefficients of 2u
    const float t = x * (-1.5957691216057308f * kLog2e + (-0.07135481627f * kLog2e) * x * x);
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(t));
}
__device__ __forceinline__ float act_gelu_erf(float x) {
    // 0.5 x (1 + erf(x / sqrt 2)) with erf from Abramowitz & Stegun 7.1.26 (|error| <= 1.5e-7):
    // erf(z) = 1 - (a1 t + ... + a5 t^5) exp(-z^2),  t = 1 / (1 + p z),  z >= 0.
    const float ax = fabsf(x);
    const float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * 0.7071067811865476f * ax);
    float poly = 1.061405429f;
    poly = poly * t - 1.453152027f;
    poly = poly * t + 1.421413741f;
    poly = poly * t - 0.284496736f;
    poly = poly * t + 0.254829592f;
    poly *= t;
    const float e = __builtin_amdgcn_exp2f(-0.5f * kLog2e * x * x);
    const float erf_abs = 1.0f - poly * e;
    return 0.5f * (x + ax * erf_abs);
}

// erf-GELU for 16-bit outputs: x * sigmoid(x (a + b s + c s^2)), s = min(x^2, 49) — the form of the tanh variant with
// one more term, fitted to x Phi(x): |error| <= 2.6e-5 everywhere (a tenth of an fp16 ulp at 1), for two
// transcendental and five plain instructions instead of two and fourteen.  The clamp keeps the polynomial on its fitted
// range (it changes sign beyond |x| = 11); at |x| = 7 the sigmoid has long saturated.
__device__ __forceinline__ float act_gelu_erf_fast(float x) {
    const float s = fminf(x * x, 49.0f);
    // the polynomial carries the factor -log2(e) of the base-2 exponential: x * sigmoid(x p) = x / (1 + 2^(x q))
    const float q = ((0.0007030433895f * kLog2e) * s - 0.07401135561f * kLog2e) * s - 1.595015695f * kLog2e;
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * q));
}

// activation of the MFMA kernels, whose outputs are fp16 / bf16
__device__ __forceinline__ float apply_act16(float x, int act) {
    // (with a run-time `act` the switch becomes a tree of scalar branches per element: the common case leaves first)
    if (act == KERNL_ACT_NONE) return x;
    switch (act) {
        case KERNL_ACT_RELU: return fmaxf(x, 0.0f);
        case KERNL_ACT_TANH: return act_tanh(x);
        case KERNL_ACT_GELU_ERF: return act_gelu_erf_fast(x);
        case KERNL_ACT_GELU_TANH: return act_gelu_tanh(x);
        case KERNL_ACT_SILU: return x * act_sigmoid(x);
        default: return x;
    }
}

__device__ __forceinline__ float apply_act(float x, int act) {
    switch (act) {
        case KERNL_ACT_RELU: return fmaxf(x, 0.0f);
        case KERNL_ACT_TANH: return act_tanh(x);
        case KERNL_ACT_GELU_ERF: return act_gelu_erf(x);
        case KERNL_ACT_GELU_TANH: return act_gelu_tanh(x);
        case KERNL_ACT_SILU: return x * act_sigmoid(x);
        default: return x;
    }
}

}  // namespace kernl
