"""Benchmark harness for the fused operators: a pytest `benchmark` fixture, per-test statistics and a grouped
comparison table at the end of the session (reference: src/kernl/benchmark/*.py and the fixture wiring in conftest.py).

Enable it in a test tree with `pytest_plugins = ["kernl_amd.benchmark.plugin"]`.
"""
from kernl_amd.benchmark.stats import Samples  # noqa: F401
from kernl_amd.benchmark.timing import Measurement, measure  # noqa: F401
