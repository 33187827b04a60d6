"""``Metric`` / ``AggregationType`` as ``ppo_loss`` returns them (``verl/utils/metric/utils.py:61-160``).

A ``Metric`` is a list of scalar observations (one per micro-batch) with the rule that folds them into one number
(``MEAN`` for statistics a micro-batch normalises by itself, ``SUM`` for losses already divided by a global count).
Unlike the reference, which calls ``.item()`` when a tensor is appended, device scalars are kept as they are and only
read back in ``aggregate()``: appending a metric inside the training step does not synchronise the stream.
"""

from __future__ import annotations

from enum import Enum

import numpy as np
import torch


class AggregationType(Enum):
    MEAN = "mean"
    SUM = "sum"
    MIN = "min"
    MAX = "max"


_FOLD = {AggregationType.MEAN: np.mean, AggregationType.SUM: np.sum, AggregationType.MIN: np.min, AggregationType.MAX: np.max}


def _number(v) -> float:
    if isinstance(v, torch.Tensor):
        return v.detach().item()
    return v


class Metric:
    def __init__(self, aggregation, value=None):
        self.aggregation = AggregationType(aggregation) if isinstance(aggregation, str) else aggregation
        if not isinstance(self.aggregation, AggregationType):
            raise ValueError(f"Unsupported aggregation type: {aggregation}")
        self.values = []
        if value is not None:
            self.append(value)

    def append(self, value) -> None:
        if isinstance(value, Metric):
            self.extend(value)
            return
        if isinstance(value, (list, tuple)):
            self.extend(value)
            return
        if isinstance(value, torch.Tensor):
            if value.numel() != 1:
                raise ValueError("Only scalar tensors can be converted to float")
            value = value.detach()
        elif not isinstance(value, (int, float, np.ndarray, np.generic)):
            raise ValueError(f"Unsupported value type: {type(value)}")
        self.values.append(value)

    def extend(self, values) -> None:
        if isinstance(values, Metric):
            if values.aggregation != self.aggregation:
                raise ValueError(f"Aggregation type mismatch: {self.aggregation} != {values.aggregation}")
            values = values.values
        for v in values:
            self.append(v)

    def numbers(self) -> list:
        """The observations as Python numbers (this is where device scalars are read back)."""
        return [_number(v) for v in self.values]

    def aggregate(self) -> float:
        return _FOLD[self.aggregation](self.numbers())

    @classmethod
    def aggregate_dp(cls, metric_lists: list["Metric"]) -> float:
        """One ``Metric`` per data-parallel rank, each with one value per gradient-accumulation step: SUM and MEAN fold
        the mean over ranks, MIN and MAX fold every value."""
        if not metric_lists:
            raise ValueError("Cannot aggregate an empty list of metrics.")
        rows = [m.numbers() for m in metric_lists]
        if any(len(r) != len(rows[0]) for r in rows):
            raise ValueError(f"All Metric instances must have the same number of values for dp aggregation: {[len(r) for r in rows]}")
        a = np.array(rows, dtype=np.float64)
        kind = metric_lists[0].aggregation
        if kind in (AggregationType.SUM, AggregationType.MEAN):
            return _FOLD[kind](a.mean(axis=0))
        return _FOLD[kind](a.reshape(-1))

    @classmethod
    def from_dict(cls, data: dict, aggregation) -> dict:
        return {k: cls(aggregation, v) for k, v in data.items()}

    def __repr__(self) -> str:
        return f"Metric({self.aggregation.value}, {self.values})"
