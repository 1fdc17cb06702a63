// Launchers of the 256-row wide kernel (see linear_kernels.h): a translation unit of its own for build time.
#include "linear_kernels.h"

namespace kernl {

void run_wide(const LinearArgs &a, int dtype, int cols) {
    if (cols == 192) {
        if (dtype == KERNL_F16) launch_wide192<f16>(a);
        else launch_wide192<bf16>(a);
    } else {
        if (dtype == KERNL_F16) launch_wide<f16>(a);
        else launch_wide<bf16>(a);
    }
}

// one-byte weights (K % 64 == 0)
static void launch_wide_w8(const LinearArgs &a) {
    switch (a.act) {
        case KERNL_ACT_RELU: launch_wide_act<f16, KERNL_ACT_RELU, 8, true>(a); break;
        case KERNL_ACT_TANH: launch_wide_act<f16, KERNL_ACT_TANH, 8, true>(a); break;
        case KERNL_ACT_GELU_ERF: launch_wide_act<f16, KERNL_ACT_GELU_ERF, 8, true>(a); break;
        case KERNL_ACT_GELU_TANH: launch_wide_act<f16, KERNL_ACT_GELU_TANH, 8, true>(a); break;
        case KERNL_ACT_SILU: launch_wide_act<f16, KERNL_ACT_SILU, 8, true>(a); break;
        default: launch_wide_act<f16, KERNL_ACT_NONE, 8, true>(a); break;
    }
}

void run_wide_w8(const LinearArgs &a) { launch_wide_w8(a); }

}  // namespace kernl
