"""``Metric`` / ``AggregationType`` as ``ppo_loss`` returns them (``verl/utils/metric/utils.py:61-160``).

A ``Metric`` is a list of scalar observations (one per micro-batch) with the rule that folds them into one number
(``MEAN`` for statistics a micro-batch normalises by itself, ``SUM`` for losses already divided by a global count).
The reference calls ``.item()`` when a tensor is appended (``:103-113``), which synchronises the stream inside the
training step.  Here an appended device scalar is held back until somebody looks: ``values`` (a property), ``aggregate``,
``aggregate_dp``, ``reduce_metrics``, ``repr`` and pickling all read the pending scalars back in ONE batched copy and
from then on the metric holds plain floats, exactly as the reference's ``Metric.values`` does.  Nothing a consumer can
reach is a tensor.
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


def reduce_metrics(metrics: dict) -> dict:
    """``verl/utils/metric/utils.py:25-58``: folds every entry in place: a ``Metric`` by its own rule, a plain list by
    ``np.max`` / ``np.min`` when the key contains "max" / "min", else ``np.mean``."""
    for key, val in metrics.items():
        if isinstance(val, Metric):
            metrics[key] = val.aggregate()
        elif "max" in key:
            metrics[key] = np.max(val)
        elif "min" in key:
            metrics[key] = np.min(val)
        else:
            metrics[key] = np.mean(val)
    return metrics


class Metric:
    def __init__(self, aggregation, value=None):
        self.aggregation = AggregationType(aggregation) if isinstance(aggregation, str) else aggregation
        if not isinstance(self.aggregation, AggregationType):
            raise ValueError(f"Unsupported aggregation type: {aggregation}")
        self._items = []  # floats, and device scalars that nobody has looked at yet
        if value is not None:
            self.append(value)

    @property
    def values(self) -> list:
        """The observations as plain numbers, like the reference's attribute; pending device scalars are read back here,
        all of them in one copy."""
        pending = [i for i, v in enumerate(self._items) if isinstance(v, torch.Tensor)]
        if pending:
            host = torch.stack([self._items[i].reshape(()).float() for i in pending]).cpu().tolist()
            for i, x in zip(pending, host):
                self._items[i] = x
        return self._items

    @values.setter
    def values(self, new) -> None:
        self._items = []
        self.extend(list(new))

    def __getstate__(self):
        return {"aggregation": self.aggregation, "values": list(self.values)}

    def __setstate__(self, state):
        self.aggregation = state["aggregation"]
        self._items = list(state["values"])

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
        self._items.append(value)

    def extend(self, values) -> None:
        if isinstance(values, Metric):
            if values.aggregation != self.aggregation:
                raise ValueError(f"Aggregation type mismatch: {self.aggregation} != {values.aggregation}")
            values = values._items  # (pending scalars stay pending)
        for v in values:
            self.append(v)

    def numbers(self) -> list:
        """The observations as Python numbers (this is where device scalars are read back)."""
        return list(self.values)

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

    def init_list(self) -> "Metric":
        """An empty metric with the same rule (``verl/utils/metric/utils.py:162-163``)."""
        return Metric(aggregation=self.aggregation)

    def __repr__(self) -> str:
        return f"Metric({self.aggregation.value}, {self.values})"
