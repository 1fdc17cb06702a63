"""Statistics of one series of timings (reference: src/kernl/benchmark/benchmark_data.py:20-94 — the same figures
under the same names, so result files can be compared)."""
from typing import Dict, Sequence, Tuple

import numpy as np


class Samples:
    """Timings of repeated runs of one function, in milliseconds."""

    def __init__(self, values_ms: Sequence[float]):
        self.values = np.asarray(list(values_ms), dtype=np.float64)
        if self.values.ndim != 1 or self.values.size == 0:
            raise ValueError("Samples needs at least one timing")

    def __len__(self) -> int:
        return int(self.values.size)

    @property
    def rounds(self) -> int:
        return len(self)

    @property
    def total(self) -> float:
        return float(self.values.sum())

    @property
    def min(self) -> float:
        return float(self.values.min())

    @property
    def max(self) -> float:
        return float(self.values.max())

    @property
    def mean(self) -> float:
        return float(self.values.mean())

    @property
    def median(self) -> float:
        # the lower of the two middle values for an even count, as torch.median gives (the reference's choice)
        return float(np.sort(self.values)[(len(self) - 1) // 2])

    @property
    def quartiles(self) -> Tuple[float, float, float]:
        q1, q2, q3 = np.quantile(self.values, [0.25, 0.5, 0.75])
        return float(q1), float(q2), float(q3)

    @property
    def stddev(self) -> float:
        return float(self.values.std(ddof=1)) if len(self) > 1 else 0.0

    @property
    def stddev_outliers(self) -> int:
        """How many timings lie more than one standard deviation away from the mean."""
        lo, hi = self.mean - self.stddev, self.mean + self.stddev
        return int(((self.values < lo) | (self.values > hi)).sum())

    @property
    def ops(self) -> float:
        """Runs per millisecond."""
        return self.rounds / self.total if self.total > 0.0 else 0.0

    def to_dict(self) -> Dict[str, float]:
        q1, _, q3 = self.quartiles
        return {
            "median": self.median, "ops": self.ops, "q1": q1, "q3": q3, "rounds": self.rounds,
            "stddev_outliers": self.stddev_outliers, "stddev": self.stddev, "mean": self.mean, "max": self.max,
            "min": self.min, "total": self.total,
        }
