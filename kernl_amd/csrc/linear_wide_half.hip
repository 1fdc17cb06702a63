// Launchers of the 128-row wide kernel and its split-over-K form (see linear_kernels.h): a translation unit of its own
// for build time.
#include "linear_kernels.h"

namespace kernl {

void run_wide_half(const LinearArgs &a, int dtype, int cols) {
    if (cols == 192) {
        if (dtype == KERNL_F16) launch_wide_half<f16, 6>(a);
        else launch_wide_half<bf16, 6>(a);
    } else {
        if (dtype == KERNL_F16) launch_wide_half<f16, 8>(a);
        else launch_wide_half<bf16, 8>(a);
    }
}

// one-byte weights (K % 64 == 0)
static void launch_wide_half_w8(const LinearArgs &a) {
    switch (a.act) {
        case KERNL_ACT_RELU: launch_wide_half_act<f16, KERNL_ACT_RELU, 8, true>(a); break;
        case KERNL_ACT_TANH: launch_wide_half_act<f16, KERNL_ACT_TANH, 8, true>(a); break;
        case KERNL_ACT_GELU_ERF: launch_wide_half_act<f16, KERNL_ACT_GELU_ERF, 8, true>(a); break;
        case KERNL_ACT_GELU_TANH: launch_wide_half_act<f16, KERNL_ACT_GELU_TANH, 8, true>(a); break;
        case KERNL_ACT_SILU: launch_wide_half_act<f16, KERNL_ACT_SILU, 8, true>(a); break;
        default: launch_wide_half_act<f16, KERNL_ACT_NONE, 8, true>(a); break;
    }
}

void run_wide_half_w8(const LinearArgs &a) { launch_wide_half_w8(a); }

void run_half_split(const LinearArgs &a, const HalfSplitPlan &p, float *part, int dtype) {
    if (dtype == KERNL_F16) launch_half_split<f16>(a, p, part);
    else launch_half_split<bf16>(a, p, part);
}

}  // namespace kernl
