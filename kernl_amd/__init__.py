"""kernl_amd — MI355X-native fused transformer inference kernels behind kernl's API.

The public surface mirrors ELS-RD/kernl (reference: src/kernl/model_optimization.py:32):

    from kernl_amd.model_optimization import optimize_model
    optimize_model(model)          # model.forward now runs the rewritten, hipGraph-captured graph

The three operators (`attention_forward`, `linear_layer`, `layer_norm`) live in
`kernl_amd.implementations` and launch hand-written gfx950 HIP kernels from `libkernl_hip.so`
through the C ABI declared in `include/kernl_hip.h`.
"""

__version__ = "0.1.0"
