// Fused linear layer: dispatch and C entry points (kernels and launchers: linear_kernels.h).
#include "linear_kernels.h"

namespace kernl {

int g_linear_force_tile = 0;

template <typename T>
static int linear_mfma_dispatch(const LinearArgs &a) {
    constexpr int kDtype = std::is_same<T, f16>::value ? KERNL_F16 : KERNL_BF16;
    int pick = g_linear_force_tile;
    // few rows of x: stream the weight once with every CU (9 forces this kernel where it applies)
    const bool small_first = pick == 0 && !(a.act & kGluBit) && small_problem_kind(a.M, a.N, a.K) != 0;
    if ((pick == 0 || pick == 9) && !small_first && a.M <= 64 && a.K % 64 == 0) {
        if (a.act & kGluBit) launch_skinny<T, true>(a);
        else launch_skinny<T, false>(a);
        return check_launch("linear (skinny)");
    }
    // small problems: one launch of small tiles over the whole K (10 / 11 / 15 force its 32 x 64 / 64 x 64 / 64 x 128 form)
    if (pick == 0 && !(a.act & kGluBit)) pick = small_problem_kind(a.M, a.N, a.K);
    if ((pick == 12 || pick == 13 || pick == 14) && !(a.act & kGluBit)) {
        run_small_dealt(a, kDtype, pick == 12 ? 16 : pick == 13 ? 32 : 64);
        return check_launch("linear (small tiles, dealt k-tiles)");
    }
    if ((pick == 10 || pick == 11 || pick == 15) && !(a.act & kGluBit)) {
        run_small(a, kDtype, pick == 10 ? 32 : 64, pick == 15 ? 128 : 64);
        return check_launch("linear (small tiles)");
    }
    if (pick == 0 || pick == 9) pick = pick_tile(a.M, a.N, a.K, (a.act & kGluBit) != 0);
    if (a.act & kGluBit) {
        if (pick == 5) run_wide(a, kDtype, 256);
        else if (pick == 3) launch_mfma_glu<T, Tile128x128>(a);
        else launch_mfma_glu<T, Tile256x256>(a);
        return check_launch("gated linear (mfma)");
    }
    if (pick == 5) run_wide(a, kDtype, 256);
    else if (pick == 6) run_wide(a, kDtype, 192);
    else if (pick == 7) run_wide_half(a, kDtype, 256);
    else if (pick == 8) run_wide_half(a, kDtype, 192);
    else if (pick == 1) launch_mfma_cfg<T, Tile256x256>(a);
    else if (pick == 2) launch_mfma_cfg<T, Tile256x192>(a);
    else if (pick == 4) launch_mfma_cfg<T, Tile256x128k32>(a);
    else launch_mfma_cfg<T, Tile128x128>(a);
    return check_launch("linear (mfma)");
}

template <typename T>
static int linear_fma_dispatch(const LinearArgs &a) {
    dim3 grid((a.N + 63) / 64, (a.M + 63) / 64);
    hipLaunchKernelGGL((linear_fma_kernel<T>), grid, dim3(256), 0, a.st, static_cast<const T *>(a.x),
                       static_cast<const T *>(a.w), static_cast<const T *>(a.bias), static_cast<T *>(a.out),
                       static_cast<T *>(a.act_in), a.M, a.N, a.K, a.x_rs, a.x_cs, a.out_rs, a.out_cs, a.ai_rs,
                       a.ai_cs, a.act);
    return check_launch("linear (fma)");
}

}  // namespace kernl

extern "C" int kernl_linear_small_kind(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || K % 8 != 0) return 0;
    return kernl::small_problem_kind(M, N, K);
}

extern "C" int kernl_linear_wide_kind(int64_t M, int64_t N, int64_t K) {
    using namespace kernl;
    if (M <= 64 || N <= 0 || K <= 0 || K % 8 != 0 || M > INT32_MAX || N > INT32_MAX || K >= (1 << 22)) return 0;
    if (small_problem_kind(M, N, K) != 0) return 0;
    const int pick = pick_tile((int)M, (int)N, (int)K, false);
    return pick >= 5 && pick <= 8 ? pick : 0;
}

// Tuning hook used by the sweep tests: force a tile shape (0 restores the heuristic).
extern "C" void kernl_linear_force_tile(int which) { kernl::g_linear_force_tile = which; }

extern "C" int kernl_linear_fwd(const void *x, const void *w, const void *bias, void *out, void *act_in,
                                int64_t M, int64_t N, int64_t K, const int64_t x_strides[2],
                                const int64_t out_strides[2], const int64_t act_in_strides[2], int activation,
                                int dtype, void *stream) {
    using namespace kernl;
    if (x == nullptr || w == nullptr || out == nullptr || x_strides == nullptr || out_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "linear: x, w, out and their strides must not be NULL");
    if (act_in != nullptr && act_in_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "linear: act_in given without strides");
    if (M < 0 || N <= 0 || K <= 0)
        return set_error(KERNL_ERR_INVALID_ARG, "linear: bad sizes M=%lld N=%lld K=%lld", (long long)M,
                         (long long)N, (long long)K);
    if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX)
        return set_error(KERNL_ERR_UNSUPPORTED, "linear: sizes must fit in 31 bits");
    if (activation < KERNL_ACT_NONE || activation > KERNL_ACT_SILU)
        return set_error(KERNL_ERR_INVALID_ARG, "linear: unknown activation %d", activation);
    if (M == 0) return KERNL_OK;

    LinearArgs a;
    a.x = x; a.w = w; a.bias = bias; a.out = out; a.act_in = act_in;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.x_rs = x_strides[0]; a.x_cs = x_strides[1];
    a.out_rs = out_strides[0]; a.out_cs = out_strides[1];
    a.ai_rs = act_in ? act_in_strides[0] : 0; a.ai_cs = act_in ? act_in_strides[1] : 0;
    a.act = activation;
    a.st = static_cast<hipStream_t>(stream);

    if (dtype == KERNL_F16 || dtype == KERNL_BF16) {
        const bool mfma_ok = a.x_cs == 1 && K % 8 == 0 && a.x_rs % 8 == 0 && aligned16(x) && aligned16(w) &&
                             a.x_rs < (1 << 22) && K < (1 << 22);  // per-thread byte offsets inside a tile fit 32 bits
        if (mfma_ok) return dtype == KERNL_F16 ? linear_mfma_dispatch<f16>(a) : linear_mfma_dispatch<bf16>(a);
        if ((M + 63) / 64 > 65535) return set_error(KERNL_ERR_UNSUPPORTED, "linear: M too large for the strided path");
        return dtype == KERNL_F16 ? linear_fma_dispatch<f16>(a) : linear_fma_dispatch<bf16>(a);
    }
    if (dtype == KERNL_F32) {
        if ((M + 63) / 64 > 65535) return set_error(KERNL_ERR_UNSUPPORTED, "linear: M too large for the fp32 path");
        return linear_fma_dispatch<float>(a);
    }
    return set_error(KERNL_ERR_UNSUPPORTED, "linear: unknown dtype %d", dtype);
}

extern "C" int64_t kernl_linear_splitk_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    using namespace kernl;
    if (M <= 0 || N <= 0 || K <= 0 || K % 64 != 0 || M > INT32_MAX || N > INT32_MAX || K >= (1 << 22)) return 0;
    return half_split_plan(M, N, K).bytes;
}

extern "C" int kernl_linear_splitk_fwd(const void *x, const void *w, const void *bias, void *out, void *act_in,
                                       void *workspace, int64_t workspace_bytes, int64_t M, int64_t N, int64_t K,
                                       const int64_t x_strides[2], const int64_t out_strides[2],
                                       const int64_t act_in_strides[2], int activation, int dtype, void *stream) {
    using namespace kernl;
    if (x == nullptr || w == nullptr || out == nullptr || x_strides == nullptr || out_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "linear (split K): x, w, out and their strides must not be NULL");
    if (act_in != nullptr && act_in_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "linear (split K): act_in given without strides");
    if (M <= 0 || N <= 0 || K <= 0 || workspace_bytes < 0)
        return set_error(KERNL_ERR_INVALID_ARG, "linear (split K): bad sizes M=%lld N=%lld K=%lld", (long long)M,
                         (long long)N, (long long)K);
    if (activation < KERNL_ACT_NONE || activation > KERNL_ACT_SILU)
        return set_error(KERNL_ERR_INVALID_ARG, "linear (split K): unknown activation %d", activation);
    if (dtype != KERNL_F16 && dtype != KERNL_BF16)
        return set_error(KERNL_ERR_UNSUPPORTED, "linear (split K): only f16 and bf16 are supported, got dtype %d", dtype);
    if (M > INT32_MAX || N > INT32_MAX || K % 64 != 0 || K >= (1 << 22) || x_strides[0] >= (1 << 22) ||
        x_strides[1] != 1 || x_strides[0] % 8 != 0 || !aligned16(x) || !aligned16(w))
        return set_error(KERNL_ERR_UNSUPPORTED, "linear (split K): K must be a multiple of 64, x needs unit feature stride "
                         "and 16-byte aligned rows, the weight a 16-byte aligned base");
    const HalfSplitPlan p = half_split_plan(M, N, K);
    if (p.splits < 2)
        return set_error(KERNL_ERR_UNSUPPORTED, "linear (split K): nothing to split for M=%lld N=%lld K=%lld "
                         "(kernl_linear_splitk_workspace_bytes returns 0): use kernl_linear_fwd", (long long)M, (long long)N,
                         (long long)K);
    if (workspace == nullptr || workspace_bytes < p.bytes || !aligned16(workspace))
        return set_error(KERNL_ERR_INVALID_ARG, "linear (split K): the workspace must hold %lld bytes, 16-byte aligned",
                         (long long)p.bytes);
    LinearArgs a;
    a.x = x; a.w = w; a.bias = bias; a.out = out; a.act_in = act_in;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.x_rs = x_strides[0]; a.x_cs = x_strides[1];
    a.out_rs = out_strides[0]; a.out_cs = out_strides[1];
    a.ai_rs = act_in ? act_in_strides[0] : 0; a.ai_cs = act_in ? act_in_strides[1] : 0;
    a.act = activation;
    a.st = static_cast<hipStream_t>(stream);
    run_half_split(a, p, static_cast<float *>(workspace), dtype);
    return check_launch("linear (split K)");
}

extern "C" int kernl_linear_glu_fwd(const void *x, const void *w, const void *bias, void *out, int64_t M, int64_t N,
                                    int64_t K, const int64_t x_strides[2], const int64_t out_strides[2],
                                    int activation, int dtype, void *stream) {
    using namespace kernl;
    if (x == nullptr || w == nullptr || out == nullptr || x_strides == nullptr || out_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "gated linear: x, w, out and their strides must not be NULL");
    if (M < 0 || N <= 0 || K <= 0)
        return set_error(KERNL_ERR_INVALID_ARG, "gated linear: bad sizes M=%lld N=%lld K=%lld", (long long)M,
                         (long long)N, (long long)K);
    if (N % 32 != 0)
        return set_error(KERNL_ERR_UNSUPPORTED, "gated linear: output width %lld must be a multiple of 32 (the "
                         "interleaving block)", (long long)N);
    if (M > INT32_MAX || 2 * N > INT32_MAX || K > INT32_MAX)
        return set_error(KERNL_ERR_UNSUPPORTED, "gated linear: sizes must fit in 31 bits");
    if (activation < KERNL_ACT_NONE || activation > KERNL_ACT_SILU)
        return set_error(KERNL_ERR_INVALID_ARG, "gated linear: unknown activation %d", activation);
    if (dtype != KERNL_F16 && dtype != KERNL_BF16)
        return set_error(KERNL_ERR_UNSUPPORTED, "gated linear: only f16 and bf16 are supported, got dtype %d", dtype);
    LinearArgs a;
    a.x = x; a.w = w; a.bias = bias; a.out = out; a.act_in = nullptr;
    a.M = (int)M; a.N = (int)(2 * N); a.K = (int)K;  // the kernels see the interleaved weight: twice the output width
    a.x_rs = x_strides[0]; a.x_cs = x_strides[1];
    a.out_rs = out_strides[0]; a.out_cs = out_strides[1];
    a.ai_rs = 0; a.ai_cs = 0;
    a.act = kGluBit | activation;
    a.st = static_cast<hipStream_t>(stream);
    const bool mfma_ok = a.x_cs == 1 && K % 8 == 0 && a.x_rs % 8 == 0 && aligned16(x) && aligned16(w) &&
                         a.x_rs < (1 << 22) && K < (1 << 22);
    if (!mfma_ok)
        return set_error(KERNL_ERR_UNSUPPORTED, "gated linear: x must have unit feature stride, 16-byte aligned rows "
                         "and K a multiple of 8");
    if (M == 0) return KERNL_OK;
    return dtype == KERNL_F16 ? linear_mfma_dispatch<f16>(a) : linear_mfma_dispatch<bf16>(a);
}

extern "C" int kernl_linear_scaled_fwd(const void *x, const void *w, const void *bias, const float *row_scale, void *out,
                                       int64_t M, int64_t N, int64_t K, const int64_t x_strides[2],
                                       const int64_t out_strides[2], int activation, int gated, int dtype, void *stream) {
    using namespace kernl;
    if (x == nullptr || w == nullptr || out == nullptr || row_scale == nullptr || x_strides == nullptr || out_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "scaled linear: x, w, row_scale, out and their strides must not be NULL");
    if (M < 0 || N <= 0 || K <= 0)
        return set_error(KERNL_ERR_INVALID_ARG, "scaled linear: bad sizes M=%lld N=%lld K=%lld", (long long)M, (long long)N,
                         (long long)K);
    const int64_t rows_w = gated ? 2 * N : N;  // the kernels see the interleaved weight of the gated form
    if (M > INT32_MAX || rows_w > INT32_MAX || K > INT32_MAX)
        return set_error(KERNL_ERR_UNSUPPORTED, "scaled linear: sizes must fit in 31 bits");
    if (gated && N % 32 != 0)
        return set_error(KERNL_ERR_UNSUPPORTED, "scaled linear: gated output width %lld must be a multiple of 32 (the "
                         "interleaving block)", (long long)N);
    if (activation < KERNL_ACT_NONE || activation > KERNL_ACT_SILU)
        return set_error(KERNL_ERR_INVALID_ARG, "scaled linear: unknown activation %d", activation);
    if (activation != (gated ? KERNL_ACT_SILU : KERNL_ACT_NONE))
        return set_error(KERNL_ERR_UNSUPPORTED, "scaled linear: built for plain sums without activation and for SiLU gates "
                         "(the projections an RMSNorm feeds in a SwiGLU decoder), got activation %d, gated %d", activation, gated);
    if (dtype != KERNL_F16 && dtype != KERNL_BF16)
        return set_error(KERNL_ERR_UNSUPPORTED, "scaled linear: only f16 and bf16 are supported, got dtype %d", dtype);
    if (x_strides[1] != 1 || K % 8 != 0 || x_strides[0] % 8 != 0 || !aligned16(x) || !aligned16(w) || !aligned16(row_scale) ||
        x_strides[0] >= (1 << 22) || K >= (1 << 22))
        return set_error(KERNL_ERR_UNSUPPORTED, "scaled linear: x must have unit feature stride, 16-byte aligned rows and K a "
                         "multiple of 8; w and row_scale 16-byte aligned bases");
    if (M == 0) return KERNL_OK;
    LinearArgs a;
    a.x = x; a.w = w; a.bias = bias; a.out = out; a.act_in = nullptr;
    a.M = (int)M; a.N = (int)rows_w; a.K = (int)K;
    a.x_rs = x_strides[0]; a.x_cs = x_strides[1];
    a.out_rs = out_strides[0]; a.out_cs = out_strides[1];
    a.ai_rs = 0; a.ai_cs = 0;
    a.act = gated ? (kGluBit | activation) : activation;
    a.st = static_cast<hipStream_t>(stream);
    a.row_scale = row_scale;
    // only the wide kernels take per-row factors (5 / 6: 256-row tiles, 7 / 8: 128-row tiles; gated: 256 x 256 only)
    int pick = g_linear_force_tile >= 5 && g_linear_force_tile <= 8 ? g_linear_force_tile : pick_tile(a.M, a.N, a.K, gated != 0, true);
    if (gated) pick = 5;
    if (pick == 5) run_wide(a, dtype, 256);
    else if (pick == 6) run_wide(a, dtype, 192);
    else if (pick == 7) run_wide_half(a, dtype, 256);
    else run_wide_half(a, dtype, 192);
    return check_launch("scaled linear");
}

extern "C" int kernl_linear_residual_fwd(const void *x, const void *w, const void *bias, const void *residual, void *out,
                                         int64_t M, int64_t N, int64_t K, const int64_t x_strides[2],
                                         const int64_t out_strides[2], const int64_t residual_strides[2], int dtype,
                                         void *stream) {
    using namespace kernl;
    if (x == nullptr || w == nullptr || out == nullptr || residual == nullptr || x_strides == nullptr ||
        out_strides == nullptr || residual_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "linear + residual: x, w, residual, out and their strides must not be NULL");
    if (M < 0 || N <= 0 || K <= 0)
        return set_error(KERNL_ERR_INVALID_ARG, "linear + residual: bad sizes M=%lld N=%lld K=%lld", (long long)M, (long long)N,
                         (long long)K);
    if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX)
        return set_error(KERNL_ERR_UNSUPPORTED, "linear + residual: sizes must fit in 31 bits");
    if (dtype != KERNL_F16 && dtype != KERNL_BF16)
        return set_error(KERNL_ERR_UNSUPPORTED, "linear + residual: only f16 and bf16 are supported, got dtype %d", dtype);
    if (x_strides[1] != 1 || K % 8 != 0 || x_strides[0] % 8 != 0 || !aligned16(x) || !aligned16(w) ||
        x_strides[0] >= (1 << 22) || K >= (1 << 22))
        return set_error(KERNL_ERR_UNSUPPORTED, "linear + residual: x must have unit feature stride, 16-byte aligned rows and K "
                         "a multiple of 8; w a 16-byte aligned base");
    if (M == 0) return KERNL_OK;
    LinearArgs a;
    a.x = x; a.w = w; a.bias = bias; a.out = out; a.act_in = nullptr;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.x_rs = x_strides[0]; a.x_cs = x_strides[1];
    a.out_rs = out_strides[0]; a.out_cs = out_strides[1];
    a.ai_rs = 0; a.ai_cs = 0;
    a.act = KERNL_ACT_NONE;
    a.st = static_cast<hipStream_t>(stream);
    a.residual = residual;
    a.res_rs = residual_strides[0]; a.res_cs = residual_strides[1];
    // only the wide kernels add a residual (5 / 6: 256-row tiles, 7 / 8: 128-row tiles)
    const int pick = g_linear_force_tile >= 5 && g_linear_force_tile <= 8 ? g_linear_force_tile : pick_tile(a.M, a.N, a.K, false, true);
    if (pick == 5) run_wide(a, dtype, 256);
    else if (pick == 6) run_wide(a, dtype, 192);
    else if (pick == 7) run_wide_half(a, dtype, 256);
    else run_wide_half(a, dtype, 192);
    return check_launch("linear + residual");
}

extern "C" int kernl_linear_w8_fwd(const void *x, const void *w8, const void *bias, void *out, void *act_in, int64_t M,
                                   int64_t N, int64_t K, const int64_t x_strides[2], const int64_t out_strides[2],
                                   const int64_t act_in_strides[2], int activation, int dtype, void *stream) {
    using namespace kernl;
    if (x == nullptr || w8 == nullptr || out == nullptr || x_strides == nullptr || out_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "linear (fp8 weight): x, w, out and their strides must not be NULL");
    if (act_in != nullptr && act_in_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "linear (fp8 weight): act_in given without strides");
    if (M < 0 || N <= 0 || K <= 0)
        return set_error(KERNL_ERR_INVALID_ARG, "linear (fp8 weight): bad sizes M=%lld N=%lld K=%lld", (long long)M,
                         (long long)N, (long long)K);
    if (activation < KERNL_ACT_NONE || activation > KERNL_ACT_SILU)
        return set_error(KERNL_ERR_INVALID_ARG, "linear (fp8 weight): unknown activation %d", activation);
    if (dtype != KERNL_F16)
        return set_error(KERNL_ERR_UNSUPPORTED, "linear (fp8 weight): activations must be f16, got dtype %d", dtype);
    if (M > INT32_MAX || N > INT32_MAX || K > INT32_MAX || K >= (1 << 22) || x_strides[0] >= (1 << 22))
        return set_error(KERNL_ERR_UNSUPPORTED, "linear (fp8 weight): sizes too large");
    if (K % 8 != 0)
        return set_error(KERNL_ERR_UNSUPPORTED, "linear (fp8 weight): K must be a multiple of 8 (K=%lld)", (long long)K);
    if (x_strides[1] != 1 || x_strides[0] % 8 != 0 || !aligned16(x) || !aligned16(w8))
        return set_error(KERNL_ERR_UNSUPPORTED, "linear (fp8 weight): x needs unit feature stride and 16-byte aligned "
                         "rows, the weight a 16-byte aligned base");
    if (M == 0) return KERNL_OK;
    LinearArgs a;
    a.x = x; a.w = w8; a.bias = bias; a.out = out; a.act_in = act_in;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.x_rs = x_strides[0]; a.x_cs = x_strides[1];
    a.out_rs = out_strides[0]; a.out_cs = out_strides[1];
    a.ai_rs = act_in ? act_in_strides[0] : 0; a.ai_cs = act_in ? act_in_strides[1] : 0;
    a.act = activation;
    a.st = static_cast<hipStream_t>(stream);
    // few rows of x: the kernel that streams the weight once with every CU; otherwise the tiled MFMA kernel, which
    // widens the bytes on their way into LDS
    if (M <= 64 && K % 64 == 0) {
        launch_skinny<f16, false, true>(a);
        return check_launch("linear (skinny, fp8 weight)");
    }
    // the tile rule of the 16-bit path: its wide family maps to the wide kernel's 256x256 form, the rest to the 8-wave
    // kernel (hook values 1 / 3 / 5 of kernl_linear_force_tile choose by hand)
    int pick = g_linear_force_tile != 0 ? g_linear_force_tile : pick_tile((int)M, (int)N, (int)K, false);
    if (pick >= 5 && pick <= 8 && K % 64 == 0) {
        // 128-row tiles where 256-row tiles leave CUs idle, and always for at most 128 rows
        if (pick >= 7 || (M <= 128 && g_linear_force_tile == 0)) run_wide_half_w8(a);
        else run_wide_w8(a);
        return check_launch("linear (wide, fp8 weight)");
    }
    if (pick == 3 || pick >= 5) launch_mfma_w8<Tile128x128>(a);
    else launch_mfma_w8<Tile256x256>(a);
    return check_launch("linear (mfma, fp8 weight)");
}

extern "C" int kernl_linear_rms_fwd(const void *x, const void *rms_weight, float eps, const void *w, const void *bias,
                                    void *out, int64_t M, int64_t N, int64_t K, const int64_t x_strides[2],
                                    const int64_t out_strides[2], int activation, int gated, int dtype, void *stream) {
    using namespace kernl;
    if (x == nullptr || rms_weight == nullptr || w == nullptr || out == nullptr || x_strides == nullptr ||
        out_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "rms linear: x, rms_weight, w, out and their strides must not be NULL");
    if (M < 0 || N <= 0 || K <= 0)
        return set_error(KERNL_ERR_INVALID_ARG, "rms linear: bad sizes M=%lld N=%lld K=%lld", (long long)M, (long long)N,
                         (long long)K);
    if (activation < KERNL_ACT_NONE || activation > KERNL_ACT_SILU)
        return set_error(KERNL_ERR_INVALID_ARG, "rms linear: unknown activation %d", activation);
    if (dtype != KERNL_F16 && dtype != KERNL_BF16)
        return set_error(KERNL_ERR_UNSUPPORTED, "rms linear: only f16 and bf16 are supported, got dtype %d", dtype);
    if (gated && N % 32 != 0)
        return set_error(KERNL_ERR_UNSUPPORTED, "rms linear: gated output width %lld must be a multiple of 32", (long long)N);
    if (M > 64 || K % 64 != 0 || 2 * N > INT32_MAX || K > INT32_MAX)
        return set_error(KERNL_ERR_UNSUPPORTED, "rms linear: at most 64 rows of x and K a multiple of 64 (M=%lld K=%lld); "
                         "normalise and multiply separately for larger inputs", (long long)M, (long long)K);
    if (x_strides[1] != 1 || x_strides[0] % 8 != 0 || !aligned16(x) || !aligned16(w) || !aligned16(rms_weight))
        return set_error(KERNL_ERR_UNSUPPORTED, "rms linear: x needs unit feature stride and 16-byte aligned rows, the "
                         "weights 16-byte aligned bases");
    if (M == 0) return KERNL_OK;
    LinearArgs a;
    a.x = x; a.w = w; a.bias = bias; a.out = out; a.act_in = nullptr;
    a.M = (int)M; a.N = (int)(gated ? 2 * N : N); a.K = (int)K;
    a.x_rs = x_strides[0]; a.x_cs = x_strides[1];
    a.out_rs = out_strides[0]; a.out_cs = out_strides[1];
    a.ai_rs = 0; a.ai_cs = 0;
    a.act = activation;
    a.st = static_cast<hipStream_t>(stream);
    if (dtype == KERNL_F16) {
        if (gated) launch_skinny_rms<f16, true>(a, rms_weight, eps);
        else launch_skinny_rms<f16, false>(a, rms_weight, eps);
    } else {
        if (gated) launch_skinny_rms<bf16, true>(a, rms_weight, eps);
        else launch_skinny_rms<bf16, false>(a, rms_weight, eps);
    }
    return check_launch("rms linear (skinny)");
}

extern "C" int kernl_linear_decode_fwd(const void *x, const void *rms_weight, float eps, const void *w, const void *bias,
                                       const void *residual, void *out, int64_t M, int64_t N, int64_t K,
                                       const int64_t x_strides[2], const int64_t out_strides[2],
                                       const int64_t residual_strides[2], const void *cos, const void *sin,
                                       int64_t head_dim, int64_t rope_cols, int64_t rows_per_batch,
                                       const int64_t table_strides[3], int table_dtype, int dtype, void *stream) {
    using namespace kernl;
    if (x == nullptr || w == nullptr || out == nullptr || x_strides == nullptr || out_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "decode linear: x, w, out and their strides must not be NULL");
    if (residual != nullptr && residual_strides == nullptr)
        return set_error(KERNL_ERR_INVALID_ARG, "decode linear: residual given without strides");
    if (M < 0 || N <= 0 || K <= 0)
        return set_error(KERNL_ERR_INVALID_ARG, "decode linear: bad sizes M=%lld N=%lld K=%lld", (long long)M, (long long)N,
                         (long long)K);
    if (dtype != KERNL_F16 && dtype != KERNL_BF16)
        return set_error(KERNL_ERR_UNSUPPORTED, "decode linear: only f16 and bf16 are supported, got dtype %d", dtype);
    if (M > 64 || K % 64 != 0 || N > INT32_MAX || K > INT32_MAX)
        return set_error(KERNL_ERR_UNSUPPORTED, "decode linear: at most 64 rows of x and K a multiple of 64 (M=%lld K=%lld)",
                         (long long)M, (long long)K);
    if (x_strides[1] != 1 || x_strides[0] % 8 != 0 || !aligned16(x) || !aligned16(w) ||
        (rms_weight != nullptr && !aligned16(rms_weight)))
        return set_error(KERNL_ERR_UNSUPPORTED, "decode linear: x needs unit feature stride and 16-byte aligned rows, the "
                         "weights 16-byte aligned bases");
    const bool rope = cos != nullptr || sin != nullptr;
    SkinnyExtra ex = {};
    if (rope) {
        if (cos == nullptr || sin == nullptr || table_strides == nullptr)
            return set_error(KERNL_ERR_INVALID_ARG, "decode linear: rotation needs cos, sin and their strides");
        if (table_dtype != KERNL_F16 && table_dtype != KERNL_BF16 && table_dtype != KERNL_F32)
            return set_error(KERNL_ERR_UNSUPPORTED, "decode linear: unknown table dtype %d", table_dtype);
        if (head_dim < 32 || head_dim % 32 != 0 || N % head_dim != 0 || rope_cols < 0 || rope_cols > N ||
            rope_cols % head_dim != 0 || rows_per_batch <= 0 || table_strides[2] != 1)
            return set_error(KERNL_ERR_UNSUPPORTED, "decode linear: rotation needs a head size that is a multiple of 32 "
                             "and divides N and rope_cols, tables with unit feature stride and rows_per_batch > 0");
        if (rms_weight == nullptr)
            return set_error(KERNL_ERR_UNSUPPORTED, "decode linear: the rotating form is built with the RMSNorm prologue only");
        ex.cos = cos; ex.sin = sin;
        ex.t_bs = table_strides[0]; ex.t_ss = table_strides[1];
        ex.table_dtype = table_dtype;
        ex.half = (int)(head_dim / 2);
        ex.rope_cols = (int)rope_cols;
        ex.rows_per_batch = (int)rows_per_batch;
    } else {
        ex.rows_per_batch = 1;
    }
    if (residual != nullptr) {
        ex.residual = residual;
        ex.res_rs = residual_strides[0];
        ex.res_cs = residual_strides[1];
    }
    if (M == 0) return KERNL_OK;
    LinearArgs a;
    a.x = x; a.w = w; a.bias = bias; a.out = out; a.act_in = nullptr;
    a.M = (int)M; a.N = (int)N; a.K = (int)K;
    a.x_rs = x_strides[0]; a.x_cs = x_strides[1];
    a.out_rs = out_strides[0]; a.out_cs = out_strides[1];
    a.ai_rs = 0; a.ai_cs = 0;
    a.act = KERNL_ACT_NONE;
    a.st = static_cast<hipStream_t>(stream);
    if (dtype == KERNL_F16) launch_skinny_decode<f16>(a, rms_weight, eps, ex);
    else launch_skinny_decode<bf16>(a, rms_weight, eps, ex);
    return check_launch("decode linear (skinny)");
}
