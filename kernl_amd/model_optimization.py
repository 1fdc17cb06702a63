"""`optimize_model`: the public entry point (reference: src/kernl/model_optimization.py:27-66).

The model's `forward` is wrapped in TorchDynamo with a backend that (1) rewrites the captured torch.fx graph so that
attention, linear(+activation) and LayerNorm/RMSNorm sub-graphs call the fused gfx950 kernels and (2) captures the
rewritten graph in a hipGraph fed from a static input pool.
"""
from typing import List

import torch
import torch._dynamo as torchdynamo

from kernl_amd import _lib
from kernl_amd.optimizer.cuda_graph import cuda_graphs_wrapper, static_inputs_pool
from kernl_amd.optimizer.dynamo_backend import dynamo_backend_ofi


# Module level so that several forwards of one model (encoder / decoder) share it
# (reference: model_optimization.py:25-29).
def _compiler(gm: torch.fx.GraphModule, example_inputs: List[torch.Tensor]):
    dynamo_backend_ofi(gm)
    return cuda_graphs_wrapper(gm, example_inputs)


def optimize_model(model: torch.nn.Module) -> None:
    """Replace `model.forward` by the optimized version, in place; the original stays as `model.forward_original`.

        model = AutoModel.from_pretrained(...).eval().cuda()
        optimize_model(model)
        model(**inputs)

    Needs a gfx950 (MI355X) device, the model on it, and the built `libkernl_hip.so`; there is no fallback.
    """
    assert torch.cuda.is_available(), "A ROCm GPU is required to use kernl_amd"
    arch = getattr(torch.cuda.get_device_properties(torch.cuda.current_device()), "gcnArchName", "")
    if not arch.startswith("gfx950"):
        raise RuntimeError(f"kernl_amd kernels are built for gfx950 (MI355X) only, found '{arch}'")
    assert next(model.parameters()).device.type == "cuda", "Model must be on GPU"
    _lib.load()  # fail now, not in the middle of the first forward
    static_inputs_pool.clear()
    model.forward_original = model.forward
    # Generation with a growing key/value cache meets a new shape at every step.  TorchDynamo gives up on a function
    # (and silently runs it unoptimised) after `recompile_limit` compilations, 8 by default: far fewer than the steps
    # of a generate() call.  The reference's own benchmarks raise the same limit to 512
    # (experimental/benchmarks/inductor.py sets torchdynamo.config.cache_size_limit = 512).
    for name in ("recompile_limit", "cache_size_limit"):
        if hasattr(torchdynamo.config, name) and getattr(torchdynamo.config, name) < 512:
            setattr(torchdynamo.config, name, 512)
    if hasattr(torchdynamo.config, "accumulated_recompile_limit") and torchdynamo.config.accumulated_recompile_limit < 4096:
        torchdynamo.config.accumulated_recompile_limit = 4096

    # Static shapes: a hipGraph is specific to its shapes, so every new input shape is a new (cached) compilation,
    # exactly as with the reference's default TorchDynamo settings.
    @torchdynamo.optimize(_compiler, dynamic=False)
    def run(*args, **kwargs):
        return model.forward_original(*args, **kwargs)

    model.forward = run
