"""The benchmark harness on the CPU: statistics against hand-computed answers, grouping rules (reference:
src/kernl/benchmark/benchmark_session.py:83-116, benchmark_result.py:25-28), the comparison table, and the fixture
driven through a real pytest session."""
import subprocess
import sys
import textwrap

import pytest

from kernl_amd.benchmark.plugin import Result, comparison_table, group_key, grouped
from kernl_amd.benchmark.stats import Samples
from kernl_amd.benchmark.timing import measure


def test_samples_known_answers():
    s = Samples([4.0, 1.0, 3.0, 2.0])
    assert (s.rounds, s.total, s.min, s.max, s.mean) == (4, 10.0, 1.0, 4.0, 2.5)
    assert s.median == 2.0                                   # lower middle value of an even count
    assert s.quartiles == (1.75, 2.5, 3.25)                  # linear interpolation between order statistics
    assert s.stddev == pytest.approx((5.0 / 3.0) ** 0.5)     # sum of squared deviations 5, n - 1 = 3
    assert s.stddev_outliers == 2                            # 1 and 4 lie outside 2.5 +- 1.29
    assert s.ops == pytest.approx(0.4)
    assert Samples([7.0]).stddev == 0.0 and Samples([7.0]).median == 7.0
    assert Samples([1.0, 5.0, 2.0]).median == 2.0
    assert set(s.to_dict()) == {"median", "ops", "q1", "q3", "rounds", "stddev_outliers", "stddev", "mean", "max", "min", "total"}
    with pytest.raises(ValueError):
        Samples([])


def _result(name, params, device_ms, wall_ms=None):
    fullname = f"tests/test_x.py::{name}"
    param = name.split("[")[1][:-1] if "[" in name else None
    return Result(name, fullname, param, params, Samples(device_ms), Samples(wall_ms or device_ms))


def test_grouping_rules():
    a = _result("test_attn[kernl-512]", {"implementation": "kernl", "seq": 512}, [1.0])
    b = _result("test_attn[torch-512]", {"implementation": "torch", "seq": 512}, [2.0])
    c = _result("test_attn[kernl-128]", {"implementation": "kernl", "seq": 128}, [0.5])
    d = _result("test_ln", None, [0.1])
    # a result's own group leaves the implementation out, so implementations meet in one group
    assert a.group == b.group == "{'seq': 512}" and c.group == "{'seq': 128}" and d.group == "{}"
    assert (a.func, a.fullfunc) == ("test_attn", "tests/test_x.py::test_attn")
    assert group_key(a, "func,param:seq") == "test_attn seq=512"
    assert group_key(a, "param") == "kernl-512" and group_key(a, "fullname") == a.fullname
    with pytest.raises(NotImplementedError):
        group_key(a, "colour")
    groups = grouped([b, d, c, a], "group")
    assert list(groups) == ["{'seq': 128}", "{'seq': 512}", "{}"]                # alphabetical
    assert [r.name for r in groups["{'seq': 512}"]] == [a.name, b.name]           # members by name
    assert [len(v) for v in grouped([a, b, c, d], "fullname").values()] == [1, 1, 1, 1]


def test_comparison_table_marks_best_and_worst():
    a = _result("fast", None, [1.0, 1.0, 1.0], [2.0, 2.0, 2.0])
    b = _result("slow", None, [4.0, 4.0, 4.0], [8.0, 8.0, 8.0])
    lines = comparison_table([a, b]).splitlines()
    assert "Median (HIP)" in lines[0] and "Max" in lines[0]
    fast, slow = lines[2], lines[3]
    assert fast.startswith("fast") and fast.count("1.0 (4.0) *") == 4 and fast.count("2.0 (4.0) *") == 4
    assert slow.startswith("slow") and slow.count("4.0 (1.0) !") == 4 and slow.count("8.0 (1.0) !") == 4
    assert "*" not in comparison_table([a]) and "!" not in comparison_table([a])  # nothing to compare with


def test_measure_on_the_host():
    calls = []
    m = measure(lambda x: calls.append(x) or x * 2, 21, warmup_ms=0.5, rep_ms=2.0, max_runs=50)
    assert m.return_value == 42
    assert 1 <= m.wall.rounds <= 50 and m.wall.min > 0.0
    assert len(calls) >= 1 + 5 + 1 + m.wall.rounds            # first run, estimate, warm-up, measured runs


def test_fixture_in_a_pytest_session(tmp_path):
    (tmp_path / "conftest.py").write_text('pytest_plugins = ["kernl_amd.benchmark.plugin"]\n')
    (tmp_path / "test_demo.py").write_text(textwrap.dedent("""
        import pytest

        @pytest.mark.parametrize("size", [10, 1000])
        @pytest.mark.parametrize("implementation", ["builtin", "loop"])
        def test_sum(benchmark, implementation, size):
            data = list(range(size))
            def loop(d):
                t = 0
                for x in d:
                    t += x
                return t
            benchmark.warmup_ms, benchmark.rep_ms = 0.2, 1.0
            assert benchmark(sum if implementation == "builtin" else loop, data) == size * (size - 1) // 2
    """))
    import os

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
    run = subprocess.run([sys.executable, "-m", "pytest", "-q", "-p", "no:cacheprovider", "--benchmark-group-by", "group", str(tmp_path)],
                         capture_output=True, text=True, env=env, cwd=str(tmp_path), timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    out = run.stdout
    assert "{'size': 10}" in out and "{'size': 1000}" in out and "Median (HIP)" in out
    block = out[out.index("{'size': 1000}"):]
    assert "test_sum[builtin-1000]" in block and "test_sum[loop-1000]" in block
