"""pytest plugin: the `benchmark` fixture, `--benchmark-group-by`, and the comparison tables printed when the session
ends (reference: conftest.py:56-83, src/kernl/benchmark/benchmark_result.py:25-55, benchmark_session.py:28-116).

A test calls `benchmark(fn, *args, **kwargs)`; it gets `fn`'s return value back, and the timings are kept under the
test's name.  Results are compared inside groups.  A result's own `group` is its parameter set WITHOUT the parameter
called "implementation", so that parametrising a test over implementations puts them side by side.
"""
from collections import OrderedDict
from typing import Dict, List, Optional

import pytest

from kernl_amd.benchmark.stats import Samples
from kernl_amd.benchmark.timing import measure

COLUMNS = ("median", "mean", "min", "max")


class Result:
    def __init__(self, name: str, fullname: str, param: Optional[str], params: Optional[dict], device: Samples, wall: Samples):
        self.name, self.fullname, self.param, self.params = name, fullname, param, params
        self.device, self.wall = device, wall
        self.group = str({k: v for k, v in (params or {}).items() if k != "implementation"})

    @property
    def func(self) -> str:
        return self.name.split("[")[0]

    @property
    def fullfunc(self) -> str:
        return self.fullname.split("[")[0]

    def to_dict(self) -> dict:
        return {"name": self.name, "group": self.group, "fullname": self.fullname, "func": self.func, "fullfunc": self.fullfunc,
                "params": self.params, "data_gpu": self.device.to_dict(), "data_full": self.wall.to_dict()}


def group_key(result: Result, group_by: str) -> str:
    """`group_by`: comma-separated list of group | name | fullname | func | fullfunc | param | param:NAME."""
    parts = []
    for item in group_by.split(","):
        if item in ("group", "name", "fullname", "func", "fullfunc", "param"):
            parts.append(getattr(result, item))
        elif item.startswith("param:"):
            name = item[len("param:"):]
            parts.append(f"{name}={(result.params or {})[name]}")
        else:
            raise NotImplementedError(f"Unsupported grouping {item!r}.")
    return " ".join(str(p) for p in parts)


def grouped(results: List[Result], group_by: str) -> "OrderedDict[str, List[Result]]":
    """Results per group, groups in alphabetical order, members by (full) name."""
    groups: Dict[str, List[Result]] = {}
    for r in results:
        groups.setdefault(group_key(r, group_by), []).append(r)
    by = (lambda r: r.fullname) if "full" in group_by else (lambda r: r.name)
    return OrderedDict((k, sorted(groups[k], key=by)) for k in sorted(groups))


def comparison_table(results: List[Result]) -> str:
    """One row per result: device and wall-clock median / mean / min / max in ms, each followed by how many times
    smaller it is than the group's largest value; `*` marks the best of a column, `!` the worst."""
    from tabulate import tabulate

    cells = [[getattr(r.device, c) for c in COLUMNS] + [getattr(r.wall, c) for c in COLUMNS] for r in results]
    rows = []
    for i, r in enumerate(results):
        row = [r.name]
        for j, v in enumerate(cells[i]):
            column = [c[j] for c in cells]
            best, worst = min(column), max(column)
            text = f"{round(v, 4)} ({round(worst / v, 2) if v > 0 else 0.0})"
            if len(results) > 1 and v == best:
                text += " *"
            elif len(results) > 1 and v == worst:
                text += " !"
            row.append(text)
        rows.append(row)
    headers = ["Name"] + [f"{c.capitalize()} (HIP)" for c in COLUMNS] + [c.capitalize() for c in COLUMNS]
    return tabulate(rows, headers=headers)


class Session:
    def __init__(self, group_by: str):
        self.group_by = group_by
        self.results: List[Result] = []

    def report(self) -> str:
        out = []
        for key, members in grouped(self.results, self.group_by).items():
            out.append("")
            out.append(key)
            out.append(comparison_table(members))
        return "\n".join(out)


class Benchmark:
    """What the `benchmark` fixture hands to a test."""

    def __init__(self, node, session: Session, warmup_ms: float = 25.0, rep_ms: float = 100.0, grad_to_none=None):
        self.node, self.session = node, session
        self.warmup_ms, self.rep_ms, self.grad_to_none = warmup_ms, rep_ms, grad_to_none

    def __call__(self, fn, *args, **kwargs):
        m = measure(fn, *args, warmup_ms=self.warmup_ms, rep_ms=self.rep_ms, grad_to_none=self.grad_to_none, **kwargs)
        callspec = getattr(self.node, "callspec", None)
        self.session.results.append(
            Result(self.node.name, self.node.nodeid, callspec.id if callspec else None,
                   dict(callspec.params) if callspec else None, m.device, m.wall)
        )
        return m.return_value


def pytest_addoption(parser):
    parser.addoption(
        "--benchmark-group-by", action="store", default="fullname",
        help="Comma-separated categories by which benchmark results are grouped for comparison: group, name, fullname, "
        "func, fullfunc, param or param:NAME (a name given to @pytest.mark.parametrize).  Default: fullname",
    )


def pytest_configure(config):
    config._kernl_benchmarks = Session(config.getoption("--benchmark-group-by"))


@pytest.fixture
def benchmark(request):
    return Benchmark(request.node, request.config._kernl_benchmarks)


def pytest_terminal_summary(terminalreporter, exitstatus, config):
    session = getattr(config, "_kernl_benchmarks", None)
    if session is not None and session.results:
        terminalreporter.write_line(session.report())
