import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# the `benchmark` fixture, --benchmark-group-by and the comparison tables at the end of the session
pytest_plugins = ["kernl_amd.benchmark.plugin"]


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(autouse=True)
def set_seed():
    torch.manual_seed(0)
    yield


# Tolerance of the fp16/bf16 kernels against the fp32 oracle on the same (already rounded) inputs:
# max-abs-error <= 1e-2 and mean relative error <= 1e-3 for fp16 outputs of unit scale.  bf16 has 3 fewer mantissa
# bits than fp16, so its bounds are 8x wider.  Outputs of larger magnitude scale the absolute bound: a number, or
# "magnitude" for max|expected| / 4 (never below 1) — the spacing of fp16 values doubles with every power of two,
# and at |y| = 4 the unit bound of 1e-2 is 2.5 spacings.
# fp32 outputs (the FMA linear kernel, LayerNorm, rotary embedding on fp32 tensors) have a tier of their own: nothing is
# rounded to 16 bits on the way, so what is left is the order of the fp32 additions and the kernels' fp32 function
# approximations — max-abs <= 1e-4 (a 768-term dot product of unit-scale terms is exact to about K * 2^-24 = 5e-5 in the
# worst case) and mean relative error <= 1e-5, a hundred times tighter than the fp16 tier.
def check_close(actual: torch.Tensor, expected: torch.Tensor, dtype=torch.float16, scale=1.0, what: str = ""):
    a = actual.detach().float().cpu()
    e = expected.detach().float().cpu()
    assert a.shape == e.shape, f"{what}: shape {tuple(a.shape)} != {tuple(e.shape)}"
    assert torch.isfinite(a).all(), f"{what}: non-finite values in the kernel output"
    widen = 8.0 if dtype == torch.bfloat16 else 1.0
    abs_unit, rel_unit = (1e-4, 1e-5) if dtype == torch.float32 else (1e-2, 1e-3)
    if scale == "magnitude":
        scale = max(1.0, e.abs().max().item() / 4)
    max_abs = (a - e).abs().max().item()
    mean_rel = ((a - e).abs().mean() / e.abs().mean().clamp_min(1e-12)).item()
    assert max_abs <= abs_unit * widen * scale, f"{what}: max abs error {max_abs:.3e} > {abs_unit * widen * scale:.1e}"
    assert mean_rel <= rel_unit * widen, f"{what}: mean relative error {mean_rel:.3e} > {rel_unit * widen:.1e}"
    return max_abs, mean_rel


@pytest.fixture
def close():
    return check_close
