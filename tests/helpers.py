"""Shared test plumbing: oracle views of packed tensors and error metrics."""

from __future__ import annotations

import numpy as np

from oracle import oracle as O


def rel_l2(actual: np.ndarray, expected: np.ndarray) -> float:
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    denom = np.linalg.norm(expected)
    return float(np.linalg.norm(actual - expected) / (denom if denom > 0 else 1.0))


def bits_equal(a: np.ndarray, b: np.ndarray) -> bool:
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


class OracleMoeTensor:
    """Oracle-side view of one mixed tensor: Projection of any (expert) on demand."""

    def __init__(self, mfe):
        self.mfe = mfe
        self.out = mfe.shape[1]
        self.layouts = [O.runtime_layout(pool.tensor, self.out) for pool in mfe.pools]
        self.where = {}
        for j, pool in enumerate(mfe.pools):
            for local, e in enumerate(np.asarray(pool.expert_ids)):
                self.where[int(e)] = (j, local)
        self._cache = {}

    def projection(self, expert: int) -> O.Projection:
        if expert not in self._cache:
            j, local = self.where[expert]
            self._cache[expert] = O.Projection(O.slice_rows(self.layouts[j], local * self.out, (local + 1) * self.out))
        return self._cache[expert]


def oracle_layer(x_f32, ids, weights, tensors, order=0, swiglu_limit=0.0, activation=0):
    """tensors: (gate, up, down); gate may be None for the gate-less activation (activation=1)."""
    gate, up, down = (OracleMoeTensor(t) if t is not None else None for t in tensors)
    return O.moe_layer(x_f32, ids, weights,
                       lambda e: (gate.projection(e) if gate is not None else None, up.projection(e), down.projection(e)),
                       order, swiglu_limit, activation)
