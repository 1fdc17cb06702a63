"""The C-ABI library loads without a GPU, exports every symbol include/kernl_hip.h declares, and rejects bad
arguments before any launch (no compute calls here)."""
import ctypes
import os
import re

import pytest
import torch

from kernl_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols(header="kernl_hip.h"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kernl_[a-z_0-9]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert _declared_symbols() == sorted(_lib.EXPORTED_SYMBOLS)
    # the process-wide tuning hooks live in a header of their own, outside the re-entrant interface
    assert _declared_symbols("kernl_hip_test.h") == sorted(_lib.TEST_HOOK_SYMBOLS)
    assert not set(_lib.TEST_HOOK_SYMBOLS) & set(_declared_symbols())


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in _declared_symbols() + _declared_symbols("kernl_hip_test.h"):
        assert hasattr(lib, name), f"{name} declared under include/ but not exported"
    assert lib.kernl_version() == 100


def test_bad_arguments_are_rejected_before_launch():
    lib = _lib.load()
    i64x4 = ctypes.c_int64 * 4
    i64x2 = ctypes.c_int64 * 2
    s4, s2 = i64x4(1, 1, 1, 1), i64x2(1, 1)
    fake = ctypes.c_void_p(16)  # never dereferenced: validation fails first
    # NULL tensors
    assert lib.kernl_linear_fwd(None, None, None, None, None, 4, 4, 4, s2, s2, None, 0, 0, None) == -1
    assert b"must not be NULL" in lib.kernl_last_error_string()
    assert lib.kernl_layernorm_fwd(None, None, None, None, None, None, 4, 4, 4, 1, 4, 1, 1e-5, 0, 0, None) == -1
    assert lib.kernl_attention_fwd(None, None, None, None, None, 1, 1, 1, 1, 64, s4, s4, s4, s4, None, None, 2,
                                   1.0, 0, 0.0, 0, None) == -1
    # bad sizes / enums
    assert lib.kernl_linear_fwd(fake, fake, None, fake, None, 4, 0, 4, s2, s2, None, 0, 0, None) == -1
    assert lib.kernl_linear_fwd(fake, fake, None, fake, None, 4, 4, 4, s2, s2, None, 99, 0, None) == -1
    assert b"unknown activation" in lib.kernl_last_error_string()
    assert lib.kernl_linear_fwd(fake, fake, None, fake, None, 4, 4, 4, s2, s2, None, 0, 7, None) == -2
    assert lib.kernl_layernorm_fwd(fake, fake, None, fake, None, None, 4, 0, 4, 1, 4, 1, 1e-5, 0, 0, None) == -1
    assert lib.kernl_layernorm_fwd(fake, fake, None, fake, None, None, 4, 4, 4, 1, 4, 1, 1e-5, 0, 9, None) == -2
    assert lib.kernl_add_layernorm_fwd(fake, None, fake, None, fake, None, None, 4, 4, 4, 1, 4, 1, 4, 1, 1e-5, 0, 0, None) == -1
    # attention: fp32 is not supported; mask broadcast rules (reference attention.py:485-494)
    assert lib.kernl_attention_fwd(fake, fake, fake, fake, None, 1, 1, 1, 1, 64, s4, s4, s4, s4, None, None, 2,
                                   1.0, 0, 0.0, 2, None) == -2
    bad_mask = i64x4(3, 1, 1, 16)
    assert lib.kernl_attention_fwd(fake, fake, fake, fake, fake, 2, 1, 16, 16, 64, s4, s4, s4, s4, bad_mask, s4, 2,
                                   1.0, 0, 0.0, 0, None) == -1
    assert b"batch" in lib.kernl_last_error_string()
    bad_mask = i64x4(2, 1, 1, 15)
    assert lib.kernl_attention_fwd(fake, fake, fake, fake, fake, 2, 1, 16, 16, 64, s4, s4, s4, s4, bad_mask, s4, 2,
                                   1.0, 0, 0.0, 0, None) == -1
    # empty work is a no-op
    assert lib.kernl_linear_fwd(fake, fake, None, fake, None, 0, 4, 4, s2, s2, None, 0, 0, None) == 0
    assert lib.kernl_layernorm_fwd(fake, fake, None, fake, None, None, 0, 4, 4, 1, 4, 1, 1e-5, 0, 0, None) == 0


def test_host_wrappers_refuse_cpu_tensors():
    # there is no CPU path: the operators must fail loudly instead of computing on the host
    from kernl_amd.implementations.attention import attention_forward
    from kernl_amd.implementations.layer_norm import layer_norm
    from kernl_amd.implementations.linear_layer import linear_layer

    x = torch.zeros((4, 8), dtype=torch.float16)
    w = torch.zeros((8, 8), dtype=torch.float16)
    with pytest.raises(_lib.KernlLibraryError):
        linear_layer(x, w, None)
    with pytest.raises(_lib.KernlLibraryError):
        layer_norm(x, torch.ones(8, dtype=torch.float16), None, 1e-5)
    q = torch.zeros((1, 1, 4, 64), dtype=torch.float16)
    with pytest.raises(_lib.KernlLibraryError):
        attention_forward(q, q, q, torch.empty_like(q), 1.0)


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "kernl_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "import oracle" not in text and "from oracle" not in text, f"{f} uses the oracle"
