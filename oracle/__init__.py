"""CPU oracle for the kernl hot path — TEST INFRASTRUCTURE ONLY.

Nothing in `kernl_amd/` may import this package.  It is used by `tests/`, by `__graft_entry__.smoke()` and by
the `cpu_baseline` leg of `bench.py` as the checker / the CPU timing baseline, never as the product path.
"""
from oracle.ops import (  # noqa: F401
    ACTIVATION_NAMES,
    activation_oracle,
    attention_oracle,
    attention_tiled_oracle,
    e5m2_decode_oracle,
    effective_eps,
    embedding_layer_norm_oracle,
    glu_oracle,
    layer_norm_oracle,
    layer_norm_welford_oracle,
    linear_oracle,
    rms_norm_oracle,
    rotary_complex_oracle,
    rotary_oracle,
)
