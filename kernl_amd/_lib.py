"""ctypes binding of libkernl_hip.so (C ABI: include/kernl_hip.h).

The library is built in-tree by `kernl_amd/csrc/Makefile` (see `kernl_amd.build`).  There is no fallback:
if the shared object is missing or a call fails, the error is raised to the caller.
"""
import ctypes
import os
from typing import Optional, Sequence

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libkernl_hip.so")
_lib: Optional[ctypes.CDLL] = None

KERNL_F16, KERNL_BF16, KERNL_F32 = 0, 1, 2
DTYPE_CODE = {torch.float16: KERNL_F16, torch.bfloat16: KERNL_BF16, torch.float32: KERNL_F32}

ACT_NONE, ACT_RELU, ACT_TANH, ACT_GELU_ERF, ACT_GELU_TANH, ACT_SILU = range(6)

# every symbol declared in include/kernl_hip.h
EXPORTED_SYMBOLS = (
    "kernl_version",
    "kernl_last_error_string",
    "kernl_attention_fwd",
    "kernl_attention_cached_fwd",
    "kernl_attention_skinny_workspace_bytes",
    "kernl_attention_skinny_fwd",
    "kernl_attention_skinny_kv8_fwd",
    "kernl_attention_kv8_fwd",
    "kernl_attention_skinny_static_max_bytes",
    "kernl_attention_skinny_static_init",
    "kernl_attention_skinny_static_fwd",
    "kernl_rope_fwd",
    "kernl_linear_fwd",
    "kernl_linear_small_kind",
    "kernl_linear_w8_fwd",
    "kernl_linear_rms_fwd",
    "kernl_linear_scaled_fwd",
    "kernl_linear_residual_fwd",
    "kernl_linear_wide_kind",
    "kernl_embedding_layernorm_fwd",
    "kernl_linear_decode_fwd",
    "kernl_linear_splitk_workspace_bytes",
    "kernl_linear_splitk_fwd",
    "kernl_linear_fewrow_workspace_bytes",
    "kernl_linear_fewrow_fwd",
    "kernl_linear_fewrow_w8_fwd",
    "kernl_linear_glu_fwd",
    "kernl_layernorm_fwd",
    "kernl_add_layernorm_fwd",
    "kernl_add_rms_stats_fwd",
)

# the process-wide test and tuning hooks of include/kernl_hip_test.h (bound for the tests and benchmarks only)
TEST_HOOK_SYMBOLS = (
    "kernl_linear_force_tile",
    "kernl_attention_force_scalar",
    "kernl_attention_set_variant",
    "kernl_probe_rate",
)

_i64 = ctypes.c_int64
_vp = ctypes.c_void_p
_i64p = ctypes.POINTER(ctypes.c_int64)


class KernlLibraryError(RuntimeError):
    pass


def lib_path() -> str:
    return _LIB_PATH


def load() -> ctypes.CDLL:
    """Load (once) and return the shared library; raises KernlLibraryError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise KernlLibraryError(
            f"{_LIB_PATH} not found: build it with `python -m kernl_amd.build` (needs hipcc, targets gfx950)"
        )
    lib = ctypes.CDLL(_LIB_PATH)
    lib.kernl_version.restype = ctypes.c_int
    lib.kernl_version.argtypes = []
    lib.kernl_last_error_string.restype = ctypes.c_char_p
    lib.kernl_last_error_string.argtypes = []
    lib.kernl_attention_fwd.restype = ctypes.c_int
    lib.kernl_attention_fwd.argtypes = (
        [_vp] * 5 + [_i64] * 5 + [_i64p] * 6 + [ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_float, ctypes.c_int, _vp]
    )
    lib.kernl_attention_cached_fwd.restype = ctypes.c_int
    lib.kernl_attention_cached_fwd.argtypes = (
        [_vp] * 5 + [_i64] * 5 + [_i64p] * 6 + [ctypes.c_int, ctypes.c_float, _i64, ctypes.c_float, ctypes.c_int, _vp]
    )
    lib.kernl_attention_kv8_fwd.restype = ctypes.c_int
    lib.kernl_attention_kv8_fwd.argtypes = (
        [_vp] * 5 + [_i64] * 5 + [_i64p] * 6
        + [ctypes.c_int, ctypes.c_float, ctypes.c_int, _i64, ctypes.c_float, ctypes.c_int, _vp]
    )
    lib.kernl_attention_skinny_workspace_bytes.restype = _i64
    lib.kernl_attention_skinny_workspace_bytes.argtypes = [_i64] * 5
    lib.kernl_attention_skinny_fwd.restype = ctypes.c_int
    lib.kernl_attention_skinny_fwd.argtypes = (
        [_vp] * 6 + [_i64] * 6 + [_i64p] * 6 + [ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_float, ctypes.c_int, _vp]
    )
    lib.kernl_attention_skinny_kv8_fwd.restype = ctypes.c_int
    lib.kernl_attention_skinny_kv8_fwd.argtypes = (
        [_vp] * 6 + [_i64] * 6 + [_i64p] * 6 + [ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_float, ctypes.c_int, _vp]
    )
    lib.kernl_attention_skinny_static_max_bytes.restype = _i64
    lib.kernl_attention_skinny_static_max_bytes.argtypes = []
    lib.kernl_attention_skinny_static_init.restype = ctypes.c_int
    lib.kernl_attention_skinny_static_init.argtypes = []
    lib.kernl_attention_skinny_static_fwd.restype = ctypes.c_int
    lib.kernl_attention_skinny_static_fwd.argtypes = (
        [_vp] * 5 + [_i64] * 5 + [_i64p] * 6 + [ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_float, ctypes.c_int, _vp]
    )
    lib.kernl_rope_fwd.restype = ctypes.c_int
    lib.kernl_rope_fwd.argtypes = [_vp] * 4 + [_i64] * 4 + [_i64p] * 5 + [ctypes.c_int, ctypes.c_int, _vp]
    lib.kernl_linear_fwd.restype = ctypes.c_int
    lib.kernl_linear_fwd.argtypes = [_vp] * 5 + [_i64] * 3 + [_i64p] * 3 + [ctypes.c_int, ctypes.c_int, _vp]
    lib.kernl_linear_w8_fwd.restype = ctypes.c_int
    lib.kernl_linear_w8_fwd.argtypes = [_vp] * 5 + [_i64] * 3 + [_i64p] * 3 + [ctypes.c_int, ctypes.c_int, _vp]
    lib.kernl_linear_decode_fwd.restype = ctypes.c_int
    lib.kernl_linear_decode_fwd.argtypes = (
        [_vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp] + [_i64] * 3 + [_i64p] * 3 + [_vp, _vp] + [_i64] * 3
        + [_i64p, ctypes.c_int, ctypes.c_int, _vp]
    )
    lib.kernl_linear_splitk_workspace_bytes.restype = _i64
    lib.kernl_linear_splitk_workspace_bytes.argtypes = [_i64] * 3
    lib.kernl_linear_splitk_fwd.restype = ctypes.c_int
    lib.kernl_linear_splitk_fwd.argtypes = [_vp] * 6 + [_i64] * 4 + [_i64p] * 3 + [ctypes.c_int, ctypes.c_int, _vp]
    lib.kernl_linear_fewrow_workspace_bytes.restype = _i64
    lib.kernl_linear_fewrow_workspace_bytes.argtypes = [_i64] * 3 + [ctypes.c_int] * 2
    lib.kernl_linear_fewrow_fwd.restype = ctypes.c_int
    lib.kernl_linear_fewrow_fwd.argtypes = (
        [_vp, _vp, ctypes.c_float] + [_vp] * 5 + [_i64] * 4 + [_i64p] * 3 + [_vp, _vp] + [_i64] * 3
        + [_i64p] + [ctypes.c_int] * 4 + [_vp]
    )
    lib.kernl_linear_fewrow_w8_fwd.restype = ctypes.c_int
    lib.kernl_linear_fewrow_w8_fwd.argtypes = lib.kernl_linear_fewrow_fwd.argtypes
    lib.kernl_linear_rms_fwd.restype = ctypes.c_int
    lib.kernl_linear_rms_fwd.argtypes = (
        [_vp, _vp, ctypes.c_float, _vp, _vp, _vp] + [_i64] * 3 + [_i64p] * 2 + [ctypes.c_int] * 3 + [_vp]
    )
    lib.kernl_linear_scaled_fwd.restype = ctypes.c_int
    lib.kernl_linear_scaled_fwd.argtypes = [_vp] * 5 + [_i64] * 3 + [_i64p] * 2 + [ctypes.c_int] * 3 + [_vp]
    lib.kernl_linear_residual_fwd.restype = ctypes.c_int
    lib.kernl_linear_residual_fwd.argtypes = [_vp] * 5 + [_i64] * 3 + [_i64p] * 3 + [ctypes.c_int, _vp]
    lib.kernl_embedding_layernorm_fwd.restype = ctypes.c_int
    lib.kernl_embedding_layernorm_fwd.argtypes = [_vp, _vp, _i64, _i64, _i64] * 3 + [_vp, _vp, _vp, _i64, _i64, _i64,
                                                                                      ctypes.c_float, ctypes.c_int, _vp]
    lib.kernl_add_rms_stats_fwd.restype = ctypes.c_int
    lib.kernl_add_rms_stats_fwd.argtypes = [_vp] * 4 + [_i64] * 5 + [ctypes.c_float, ctypes.c_int, _vp]
    lib.kernl_linear_small_kind.restype = ctypes.c_int
    lib.kernl_linear_small_kind.argtypes = [_i64] * 3
    lib.kernl_linear_wide_kind.restype = ctypes.c_int
    lib.kernl_linear_wide_kind.argtypes = [_i64] * 3
    lib.kernl_linear_glu_fwd.restype = ctypes.c_int
    lib.kernl_linear_glu_fwd.argtypes = [_vp] * 4 + [_i64] * 3 + [_i64p] * 2 + [ctypes.c_int, ctypes.c_int, _vp]
    lib.kernl_layernorm_fwd.restype = ctypes.c_int
    lib.kernl_layernorm_fwd.argtypes = [_vp] * 6 + [_i64] * 6 + [ctypes.c_float, ctypes.c_int, ctypes.c_int, _vp]
    lib.kernl_add_layernorm_fwd.restype = ctypes.c_int
    lib.kernl_add_layernorm_fwd.argtypes = [_vp] * 7 + [_i64] * 8 + [ctypes.c_float, ctypes.c_int, ctypes.c_int, _vp]
    lib.kernl_linear_force_tile.restype = None
    lib.kernl_linear_force_tile.argtypes = [ctypes.c_int]
    lib.kernl_attention_force_scalar.restype = None
    lib.kernl_attention_force_scalar.argtypes = [ctypes.c_int]
    lib.kernl_attention_set_variant.restype = None
    lib.kernl_attention_set_variant.argtypes = [ctypes.c_int]
    lib.kernl_probe_rate.restype = ctypes.c_int
    lib.kernl_probe_rate.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, _vp, _vp, _i64, _vp, _vp, _vp]
    _lib = lib
    return lib


def _arr(values: Sequence[int]):
    return (ctypes.c_int64 * len(values))(*values)


def _check(status: int, what: str) -> None:
    if status != 0:
        msg = load().kernl_last_error_string().decode("utf-8", "replace")
        raise KernlLibraryError(f"{what} failed with status {status}: {msg}")


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _require_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernlLibraryError("kernl_amd kernels need tensors on a GPU device (there is no CPU path)")


def attention_fwd(q, k, v, out, mask, sm_scale: float, is_causal: bool, mask_min_clamp: float) -> None:
    _require_gpu(q, k, v, out, mask)
    B, H, M, D = q.shape
    N = k.shape[2]
    lib = load()
    if mask is not None:
        msizes, mstrides, mdtype, mptr = _arr(mask.shape), _arr(mask.stride()), DTYPE_CODE[mask.dtype], mask.data_ptr()
    else:
        msizes, mstrides, mdtype, mptr = None, None, KERNL_F32, None
    with torch.cuda.device(q.device):
        st = lib.kernl_attention_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), mptr,
            B, H, M, N, D,
            _arr(q.stride()), _arr(k.stride()), _arr(v.stride()), _arr(out.stride()),
            msizes, mstrides, mdtype,
            float(sm_scale), int(bool(is_causal)), float(mask_min_clamp), DTYPE_CODE[q.dtype], _stream(q),
        )
    _check(st, "kernl_attention_fwd")


def attention_cached_fwd(q, k, v, out, mask, sm_scale: float, start_position: int, mask_min_clamp: float) -> None:
    """Causal attention of the rows of q, which sit at positions start_position.. of the sequence held in k / v."""
    _require_gpu(q, k, v, out, mask)
    B, H, M, D = q.shape
    N = k.shape[2]
    lib = load()
    if mask is not None:
        msizes, mstrides, mdtype, mptr = _arr(mask.shape), _arr(mask.stride()), DTYPE_CODE[mask.dtype], mask.data_ptr()
    else:
        msizes, mstrides, mdtype, mptr = None, None, KERNL_F32, None
    with torch.cuda.device(q.device):
        st = lib.kernl_attention_cached_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), mptr,
            B, H, M, N, D,
            _arr(q.stride()), _arr(k.stride()), _arr(v.stride()), _arr(out.stride()),
            msizes, mstrides, mdtype,
            float(sm_scale), int(start_position), float(mask_min_clamp), DTYPE_CODE[q.dtype], _stream(q),
        )
    _check(st, "kernl_attention_cached_fwd")


def attention_kv8_fwd(q, k8, v8, out, mask, sm_scale: float, is_causal: bool, start_position: int, mask_min_clamp: float) -> None:
    """k8, v8 [B, H, N, D]: fp8 e5m2 bytes (int8 / uint8 / float8_e5m2); q and out fp16."""
    _require_gpu(q, k8, v8, out, mask)
    B, H, M, D = q.shape
    N = k8.shape[2]
    lib = load()
    if mask is not None:
        msizes, mstrides, mdtype, mptr = _arr(mask.shape), _arr(mask.stride()), DTYPE_CODE[mask.dtype], mask.data_ptr()
    else:
        msizes, mstrides, mdtype, mptr = None, None, KERNL_F32, None
    with torch.cuda.device(q.device):
        st = lib.kernl_attention_kv8_fwd(
            q.data_ptr(), k8.data_ptr(), v8.data_ptr(), out.data_ptr(), mptr,
            B, H, M, N, D,
            _arr(q.stride()), _arr(k8.stride()), _arr(v8.stride()), _arr(out.stride()),
            msizes, mstrides, mdtype,
            float(sm_scale), int(bool(is_causal)), int(start_position), float(mask_min_clamp), DTYPE_CODE[q.dtype], _stream(q),
        )
    _check(st, "kernl_attention_kv8_fwd")


def attention_skinny_workspace_bytes(B: int, H: int, M: int, N: int, D: int) -> int:
    return int(load().kernl_attention_skinny_workspace_bytes(B, H, M, N, D))


def attention_skinny_fwd(q, k, v, out, mask, workspace, sm_scale: float, is_causal: bool, mask_min_clamp: float) -> None:
    _require_gpu(q, k, v, out, mask, workspace)
    B, H, M, D = q.shape
    N = k.shape[2]
    lib = load()
    if mask is not None:
        msizes, mstrides, mdtype, mptr = _arr(mask.shape), _arr(mask.stride()), DTYPE_CODE[mask.dtype], mask.data_ptr()
    else:
        msizes, mstrides, mdtype, mptr = None, None, KERNL_F32, None
    ws_ptr = None if workspace is None else workspace.data_ptr()
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    with torch.cuda.device(q.device):
        one_byte = k.dtype in (torch.int8, torch.uint8, torch.float8_e5m2)
        entry = lib.kernl_attention_skinny_kv8_fwd if one_byte else lib.kernl_attention_skinny_fwd
        st = entry(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), mptr, ws_ptr, ws_bytes,
            B, H, M, N, D,
            _arr(q.stride()), _arr(k.stride()), _arr(v.stride()), _arr(out.stride()),
            msizes, mstrides, mdtype,
            float(sm_scale), int(bool(is_causal)), float(mask_min_clamp), DTYPE_CODE[q.dtype], _stream(q),
        )
    _check(st, "kernl_attention_skinny_fwd")


def attention_skinny_static_init(device=None) -> None:
    """Look up the static partial-result buffer of `device` (default: the current one): to be called outside graph
    capture before `attention_skinny_static_fwd` is captured for the first time on that device."""
    lib = load()
    with torch.cuda.device(device):
        st = lib.kernl_attention_skinny_static_init()
    _check(st, "kernl_attention_skinny_static_init")


def attention_skinny_static_fwd(q, k, v, out, mask, sm_scale: float, is_causal: bool, mask_min_clamp: float) -> None:
    """`attention_skinny_fwd` on the library's own static partial-result buffer: no workspace, no allocation."""
    _require_gpu(q, k, v, out, mask)
    B, H, M, D = q.shape
    N = k.shape[2]
    lib = load()
    if mask is not None:
        msizes, mstrides, mdtype, mptr = _arr(mask.shape), _arr(mask.stride()), DTYPE_CODE[mask.dtype], mask.data_ptr()
    else:
        msizes, mstrides, mdtype, mptr = None, None, KERNL_F32, None
    with torch.cuda.device(q.device):
        st = lib.kernl_attention_skinny_static_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), mptr,
            B, H, M, N, D,
            _arr(q.stride()), _arr(k.stride()), _arr(v.stride()), _arr(out.stride()),
            msizes, mstrides, mdtype,
            float(sm_scale), int(bool(is_causal)), float(mask_min_clamp), DTYPE_CODE[q.dtype], _stream(q),
        )
    _check(st, "kernl_attention_skinny_static_fwd")


def rope_fwd(x, cos, sin, out) -> None:
    """x, out [B,H,S,D]; cos, sin [B|1,H|1,S,D] of the same dtype as each other."""
    _require_gpu(x, cos, sin, out)
    B, H, S, D = x.shape
    lib = load()
    with torch.cuda.device(x.device):
        st = lib.kernl_rope_fwd(
            x.data_ptr(), cos.data_ptr(), sin.data_ptr(), out.data_ptr(), B, H, S, D,
            _arr(x.stride()), _arr(out.stride()), _arr(cos.shape), _arr(cos.stride()), _arr(sin.stride()),
            DTYPE_CODE[cos.dtype], DTYPE_CODE[x.dtype], _stream(x),
        )
    _check(st, "kernl_rope_fwd")


def linear_small_kind(M: int, N: int, K: int) -> int:
    """Non-zero when `kernl_linear_fwd` runs an M x N x K problem on one of its small-problem kernels."""
    return int(load().kernl_linear_small_kind(int(M), int(N), int(K)))


def linear_wide_kind(M: int, N: int, K: int) -> int:
    """Non-zero when `kernl_linear_fwd` runs a plain 16-bit M x N x K problem on one of its wide tile kernels."""
    return int(load().kernl_linear_wide_kind(int(M), int(N), int(K)))


def linear_fwd(x2d, weight, bias, out2d, act_in2d, activation: int) -> None:
    _require_gpu(x2d, weight, bias, out2d, act_in2d)
    M, K = x2d.shape
    N = weight.shape[0]
    lib = load()
    with torch.cuda.device(x2d.device):
        st = lib.kernl_linear_fwd(
            x2d.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(), out2d.data_ptr(),
            None if act_in2d is None else act_in2d.data_ptr(),
            M, N, K,
            _arr(x2d.stride()), _arr(out2d.stride()), None if act_in2d is None else _arr(act_in2d.stride()),
            int(activation), DTYPE_CODE[x2d.dtype], _stream(x2d),
        )
    _check(st, "kernl_linear_fwd")


def linear_w8_supported(x2d, weight8) -> bool:
    """What `kernl_linear_w8_fwd` takes: fp16 rows with unit feature stride, 16-byte aligned, K a multiple of 8."""
    M, K = x2d.shape
    return (
        x2d.dtype == torch.float16 and K % 8 == 0 and K < (1 << 22) and x2d.stride(1) == 1 and x2d.stride(0) % 8 == 0
        and x2d.stride(0) < (1 << 22)
        and x2d.data_ptr() % 16 == 0 and weight8.is_contiguous() and weight8.data_ptr() % 16 == 0
    )


def linear_w8_fwd(x2d, weight8, bias, out2d, act_in2d, activation: int) -> None:
    """weight8 [N, K]: fp8 e5m2 bytes (int8 / uint8 / float8_e5m2)."""
    _require_gpu(x2d, weight8, bias, out2d, act_in2d)
    M, K = x2d.shape
    N = weight8.shape[0]
    lib = load()
    with torch.cuda.device(x2d.device):
        st = lib.kernl_linear_w8_fwd(
            x2d.data_ptr(), weight8.data_ptr(), None if bias is None else bias.data_ptr(), out2d.data_ptr(),
            None if act_in2d is None else act_in2d.data_ptr(),
            M, N, K,
            _arr(x2d.stride()), _arr(out2d.stride()), None if act_in2d is None else _arr(act_in2d.stride()),
            int(activation), DTYPE_CODE[x2d.dtype], _stream(x2d),
        )
    _check(st, "kernl_linear_w8_fwd")


def linear_rms_supported(x2d) -> bool:
    """What `kernl_linear_rms_fwd` takes: 16-bit rows, at most 64 of them, K a multiple of 64."""
    M, K = x2d.shape
    return (
        x2d.dtype in (torch.float16, torch.bfloat16) and M <= 64 and K % 64 == 0 and x2d.stride(1) == 1
        and x2d.stride(0) % 8 == 0 and x2d.data_ptr() % 16 == 0
    )


def linear_rms_fwd(x2d, rms_weight, eps: float, weight, bias, out2d, activation: int, gated: bool) -> None:
    _require_gpu(x2d, rms_weight, weight, bias, out2d)
    M, K = x2d.shape
    N = out2d.shape[1]
    lib = load()
    with torch.cuda.device(x2d.device):
        st = lib.kernl_linear_rms_fwd(
            x2d.data_ptr(), rms_weight.data_ptr(), float(eps), weight.data_ptr(),
            None if bias is None else bias.data_ptr(), out2d.data_ptr(), M, N, K,
            _arr(x2d.stride()), _arr(out2d.stride()), int(activation), int(bool(gated)), DTYPE_CODE[x2d.dtype],
            _stream(x2d),
        )
    _check(st, "kernl_linear_rms_fwd")


def linear_scaled_supported(x2d, weight) -> bool:
    """What `kernl_linear_scaled_fwd` takes: 16-bit rows with unit feature stride, 16-byte aligned, K a multiple of 8."""
    M, K = x2d.shape
    return (
        x2d.dtype in (torch.float16, torch.bfloat16) and weight.dtype == x2d.dtype and K % 8 == 0 and x2d.stride(1) == 1
        and x2d.stride(0) % 8 == 0 and x2d.stride(0) < (1 << 22) and K < (1 << 22) and x2d.data_ptr() % 16 == 0
        and weight.is_contiguous() and weight.data_ptr() % 16 == 0
    )


def linear_scaled_fwd(x2d, weight, bias, row_scale, out2d, activation: int, gated: bool) -> None:
    """out = act((x @ w^T) * row_scale[:, None] + bias); gated: w and bias interleaved as for `linear_glu_fwd`."""
    _require_gpu(x2d, weight, bias, row_scale, out2d)
    M, K = x2d.shape
    N = out2d.shape[1]
    if row_scale.dtype != torch.float32 or row_scale.numel() != M or not row_scale.is_contiguous():
        raise ValueError("row_scale must be a contiguous fp32 vector with one entry per row of x")
    lib = load()
    with torch.cuda.device(x2d.device):
        st = lib.kernl_linear_scaled_fwd(
            x2d.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(), row_scale.data_ptr(),
            out2d.data_ptr(), M, N, K, _arr(x2d.stride()), _arr(out2d.stride()), int(activation), int(bool(gated)),
            DTYPE_CODE[x2d.dtype], _stream(x2d),
        )
    _check(st, "kernl_linear_scaled_fwd")


def linear_residual_fwd(x2d, weight, bias, residual2d, out2d) -> None:
    """out = round(x @ w^T + bias) + residual in the epilogue of the wide tile kernels (`linear_scaled_supported` says
    which x and w they take; residual and out are [M, N] of x's dtype and must not overlap)."""
    _require_gpu(x2d, weight, bias, residual2d, out2d)
    M, K = x2d.shape
    N = out2d.shape[1]
    if residual2d.shape != out2d.shape or residual2d.dtype != x2d.dtype or out2d.dtype != x2d.dtype:
        raise ValueError("residual and out must have shape [M, N] and the dtype of x")
    lib = load()
    with torch.cuda.device(x2d.device):
        st = lib.kernl_linear_residual_fwd(
            x2d.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(), residual2d.data_ptr(),
            out2d.data_ptr(), M, N, K, _arr(x2d.stride()), _arr(out2d.stride()), _arr(residual2d.stride()),
            DTYPE_CODE[x2d.dtype], _stream(x2d),
        )
    _check(st, "kernl_linear_residual_fwd")


def embedding_layernorm_fwd(tables, ids, weight, bias, out, eps: float) -> None:
    """out[b, s] = LayerNorm(sum of tables[i][ids[i][b, s]]) (rows added one after the other in the tables' dtype).
    tables: 1 to 3 contiguous [rows, N] matrices; ids: int64 [batch, seq] views (stride 0 allowed); out [batch, seq, N]."""
    _require_gpu(*tables, *ids, weight, bias, out)
    batch, seq, n = out.shape
    if not 1 <= len(tables) <= 3 or len(ids) != len(tables):
        raise ValueError("one to three tables, each with its ids")
    if not out.is_contiguous() or any(not t.is_contiguous() or t.shape[1] != n or t.dtype != out.dtype for t in tables):
        raise ValueError("tables and out must be contiguous, of one dtype and one width")
    if any(i.dtype != torch.int64 or tuple(i.shape) != (batch, seq) for i in ids):
        raise ValueError("ids must be int64 [batch, seq] (expanded views are fine)")
    args = []
    for k in range(3):
        if k < len(tables):
            args += [tables[k].data_ptr(), ids[k].data_ptr(), ids[k].stride(0), ids[k].stride(1), tables[k].shape[0]]
        else:
            args += [None, None, 0, 0, 0]
    lib = load()
    with torch.cuda.device(out.device):
        st = lib.kernl_embedding_layernorm_fwd(*args, weight.data_ptr(), None if bias is None else bias.data_ptr(), out.data_ptr(),
                                               batch, seq, n, float(eps), DTYPE_CODE[out.dtype], _stream(out))
    _check(st, "kernl_embedding_layernorm_fwd")


def add_rms_stats_fwd(a2d, b2d, sum2d, rstd, eps: float) -> None:
    """sum = a + b (b and sum may be None: statistics of `a` alone), rstd[m] = 1 / sqrt(mean(sum[m]^2) + eps)."""
    _require_gpu(a2d, b2d, sum2d, rstd)
    M, N = a2d.shape
    if rstd.dtype != torch.float32 or rstd.numel() != M or not rstd.is_contiguous():
        raise ValueError("rstd must be a contiguous fp32 vector with one entry per row")
    if a2d.stride(1) != 1 or (b2d is not None and (b2d.stride(1) != 1 or sum2d.stride(1) != 1)):
        raise ValueError("add_rms_stats needs unit feature strides")
    lib = load()
    with torch.cuda.device(a2d.device):
        st = lib.kernl_add_rms_stats_fwd(
            a2d.data_ptr(), None if b2d is None else b2d.data_ptr(), None if sum2d is None else sum2d.data_ptr(),
            rstd.data_ptr(), M, N, a2d.stride(0), 0 if b2d is None else b2d.stride(0),
            0 if sum2d is None else sum2d.stride(0), float(eps), DTYPE_CODE[a2d.dtype], _stream(a2d),
        )
    _check(st, "kernl_add_rms_stats_fwd")


def linear_decode_supported(x2d, weight) -> bool:
    """What `kernl_linear_decode_fwd` takes: 16-bit rows, at most 64 of them, K a multiple of 64, a 16-bit weight."""
    M, K = x2d.shape
    return (
        x2d.dtype in (torch.float16, torch.bfloat16) and weight.dtype == x2d.dtype and M <= 64 and K % 64 == 0
        and x2d.stride(1) == 1 and x2d.stride(0) % 8 == 0 and x2d.data_ptr() % 16 == 0
        and weight.is_contiguous() and weight.data_ptr() % 16 == 0
    )


def linear_decode_fwd(x2d, rms_weight, eps: float, weight, bias, residual2d, out2d, cos=None, sin=None, head_dim: int = 0,
                      rope_cols: int = 0, rows_per_batch: int = 1) -> None:
    """cos / sin: [batch | 1, positions, head_dim] tables (unit feature stride) or None; row m of x2d is position
    m % rows_per_batch of batch entry m / rows_per_batch."""
    _require_gpu(x2d, rms_weight, weight, bias, residual2d, out2d, cos, sin)
    M, K = x2d.shape
    N = out2d.shape[1]
    lib = load()
    if cos is not None:
        tstrides = _arr((0 if cos.shape[0] == 1 else cos.stride(0), cos.stride(1), cos.stride(2)))
        tdtype, cptr, sptr = DTYPE_CODE[cos.dtype], cos.data_ptr(), sin.data_ptr()
    else:
        tstrides, tdtype, cptr, sptr = None, KERNL_F32, None, None
    with torch.cuda.device(x2d.device):
        st = lib.kernl_linear_decode_fwd(
            x2d.data_ptr(), None if rms_weight is None else rms_weight.data_ptr(), float(eps), weight.data_ptr(),
            None if bias is None else bias.data_ptr(), None if residual2d is None else residual2d.data_ptr(),
            out2d.data_ptr(), M, N, K, _arr(x2d.stride()), _arr(out2d.stride()),
            None if residual2d is None else _arr(residual2d.stride()), cptr, sptr, int(head_dim), int(rope_cols),
            int(rows_per_batch), tstrides, tdtype, DTYPE_CODE[x2d.dtype], _stream(x2d),
        )
    _check(st, "kernl_linear_decode_fwd")


def linear_splitk_workspace_bytes(x2d, weight) -> int:
    """Bytes of workspace `linear_splitk_fwd` wants for this product; 0: splitting K does not pay (or the input is not
    what the kernel takes) and `linear_fwd` is the call to make."""
    M, K = x2d.shape
    if not (
        x2d.dtype in (torch.float16, torch.bfloat16) and weight.dtype == x2d.dtype and K % 64 == 0 and K < (1 << 22)
        and x2d.stride(1) == 1 and x2d.stride(0) % 8 == 0 and x2d.stride(0) < (1 << 22) and x2d.data_ptr() % 16 == 0
        and weight.is_contiguous() and weight.data_ptr() % 16 == 0
    ):
        return 0
    return int(load().kernl_linear_splitk_workspace_bytes(M, weight.shape[0], K))


def linear_splitk_fwd(x2d, weight, bias, out2d, act_in2d, activation: int, workspace) -> None:
    _require_gpu(x2d, weight, bias, out2d, act_in2d, workspace)
    M, K = x2d.shape
    N = out2d.shape[1]
    lib = load()
    with torch.cuda.device(x2d.device):
        st = lib.kernl_linear_splitk_fwd(
            x2d.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(), out2d.data_ptr(),
            None if act_in2d is None else act_in2d.data_ptr(), workspace.data_ptr(),
            workspace.numel() * workspace.element_size(), M, N, K, _arr(x2d.stride()), _arr(out2d.stride()),
            None if act_in2d is None else _arr(act_in2d.stride()), int(activation), DTYPE_CODE[x2d.dtype], _stream(x2d),
        )
    _check(st, "kernl_linear_splitk_fwd")


def linear_fewrow_supported(x2d, weight) -> bool:
    """What `kernl_linear_fewrow_fwd` / `_w8_fwd` take: 16-bit rows, at most 128 of them, K a multiple of 64 from 256 on,
    a weight of the same type or — fp16 rows only — fp8 e5m2 bytes."""
    M, K = x2d.shape
    one_byte = weight.dtype in (torch.int8, torch.uint8, torch.float8_e5m2)
    return (
        x2d.dtype in (torch.float16, torch.bfloat16) and 0 < M <= 128
        and (weight.dtype == x2d.dtype or (one_byte and x2d.dtype == torch.float16))
        and K % 64 == 0 and K >= 256 and x2d.stride(1) == 1 and x2d.stride(0) % 8 == 0 and x2d.data_ptr() % 16 == 0
        and weight.is_contiguous() and weight.data_ptr() % 16 == 0
    )


def linear_fewrow_workspace_bytes(M: int, N: int, K: int, gated: bool = False, rotated: bool = False) -> int:
    """N: output width (the gated form's weight has twice as many rows)."""
    return int(load().kernl_linear_fewrow_workspace_bytes(M, N, K, int(bool(gated)), int(bool(rotated))))


def linear_fewrow_fwd(x2d, weight, bias, residual2d, out2d, activation: int, workspace=None, rms_weight=None,
                      eps: float = 0.0, gated: bool = False, cos=None, sin=None, head_dim: int = 0, rope_cols: int = 0,
                      rows_per_batch: int = 1) -> None:
    """`workspace`: device tensor of at least `linear_fewrow_workspace_bytes` bytes; allocated here when None (a fresh
    allocation per call: stream-ordered, so calls on different streams never share one).  cos / sin as for
    `linear_decode_fwd`; `gated`: weight and bias interleaved as for `linear_glu_fwd`, out2d half as wide."""
    _require_gpu(x2d, weight, bias, residual2d, out2d, workspace, rms_weight, cos, sin)
    M, K = x2d.shape
    N = out2d.shape[1]
    lib = load()
    if workspace is None:
        need = linear_fewrow_workspace_bytes(M, N, K, gated, cos is not None)
        if need:
            workspace = torch.empty(need, dtype=torch.uint8, device=x2d.device)
    ws_ptr = None if workspace is None else workspace.data_ptr()
    ws_bytes = 0 if workspace is None else workspace.numel() * workspace.element_size()
    if cos is not None:
        tstrides = _arr((0 if cos.shape[0] == 1 else cos.stride(0), cos.stride(1), cos.stride(2)))
        tdtype, cptr, sptr = DTYPE_CODE[cos.dtype], cos.data_ptr(), sin.data_ptr()
    else:
        tstrides, tdtype, cptr, sptr = None, KERNL_F32, None, None
    entry = lib.kernl_linear_fewrow_fwd if weight.element_size() == 2 else lib.kernl_linear_fewrow_w8_fwd
    with torch.cuda.device(x2d.device):
        st = entry(
            x2d.data_ptr(), None if rms_weight is None else rms_weight.data_ptr(), float(eps), weight.data_ptr(),
            None if bias is None else bias.data_ptr(), None if residual2d is None else residual2d.data_ptr(),
            out2d.data_ptr(), ws_ptr, ws_bytes, M, N, K, _arr(x2d.stride()), _arr(out2d.stride()),
            None if residual2d is None else _arr(residual2d.stride()), cptr, sptr, int(head_dim), int(rope_cols),
            int(rows_per_batch), tstrides, tdtype, int(activation), int(bool(gated)), DTYPE_CODE[x2d.dtype], _stream(x2d),
        )
    _check(st, "kernl_linear_fewrow_fwd")


def linear_glu_fwd(x2d, weight_interleaved, bias_interleaved, out2d, activation: int) -> None:
    _require_gpu(x2d, weight_interleaved, bias_interleaved, out2d)
    M, K = x2d.shape
    N = weight_interleaved.shape[0] // 2
    lib = load()
    with torch.cuda.device(x2d.device):
        st = lib.kernl_linear_glu_fwd(
            x2d.data_ptr(), weight_interleaved.data_ptr(),
            None if bias_interleaved is None else bias_interleaved.data_ptr(), out2d.data_ptr(),
            M, N, K, _arr(x2d.stride()), _arr(out2d.stride()), int(activation), DTYPE_CODE[x2d.dtype], _stream(x2d),
        )
    _check(st, "kernl_linear_glu_fwd")


def layernorm_fwd(x2d, weight, bias, out2d, mean, rstd, eps: float, is_rms: bool, residual2d=None) -> None:
    _require_gpu(x2d, weight, bias, out2d, mean, rstd, residual2d)
    M, N = x2d.shape
    lib = load()
    with torch.cuda.device(x2d.device):
        if residual2d is None:
            st = lib.kernl_layernorm_fwd(
                x2d.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(), out2d.data_ptr(),
                None if mean is None else mean.data_ptr(), None if rstd is None else rstd.data_ptr(),
                M, N, x2d.stride(0), x2d.stride(1), out2d.stride(0), out2d.stride(1),
                float(eps), int(bool(is_rms)), DTYPE_CODE[x2d.dtype], _stream(x2d),
            )
            _check(st, "kernl_layernorm_fwd")
        else:
            st = lib.kernl_add_layernorm_fwd(
                x2d.data_ptr(), residual2d.data_ptr(), weight.data_ptr(), None if bias is None else bias.data_ptr(),
                out2d.data_ptr(), None if mean is None else mean.data_ptr(), None if rstd is None else rstd.data_ptr(),
                M, N, x2d.stride(0), x2d.stride(1), residual2d.stride(0), residual2d.stride(1),
                out2d.stride(0), out2d.stride(1),
                float(eps), int(bool(is_rms)), DTYPE_CODE[x2d.dtype], _stream(x2d),
            )
            _check(st, "kernl_add_layernorm_fwd")
