"""Two mixers side by side: both read the same input, and their results are added.

    y = left(h) + right(h)

Each of the two brings its own constant factor (a mixer's `out_scale`), so the sum needs no
arithmetic of its own: the result is handed on as the pair (left, right), and the norm's kernel that
takes the mixer's result adds the two in 32-bit (`Norm.add_normed(hidden, y, extra)`).  At most one
of the two may keep a per-token cache; the fixed-size states of both lie one behind the other in
one state row of the request, and each mixer sees its own columns of it.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, Optional

import torch

from ..weights.spec import TensorSpec
from .base import BuildContext, CacheSpec, Mixer, StateSpec


class SideBySideMixer(Mixer):
    def __init__(self, left: Mixer, right: Mixer):
        self.left, self.right = left, right
        self.graph_safe = bool(getattr(left, "graph_safe", False) and getattr(right, "graph_safe", False))
        if left.cache_spec() is not None and right.cache_spec() is not None:
            raise ValueError("of two mixers side by side at most one keeps a per-token cache")
        self._columns = []  # per mixer: (first column, columns) of the shared state row, or None
        at = 0
        for m in (left, right):
            spec = m.state_spec()
            if spec is None:
                self._columns.append(None)
                continue
            if len(spec.shape) != 1 or spec.dtype != torch.float32:
                raise ValueError("mixers side by side keep their states as one float32 row each")
            self._columns.append((at, spec.shape[0]))
            at += spec.shape[0]
        self._state_width = at

    def cache_spec(self) -> Optional[CacheSpec]:
        return self.left.cache_spec() or self.right.cache_spec()

    def state_spec(self) -> Optional[StateSpec]:
        return StateSpec((self._state_width,), torch.float32) if self._state_width else None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {**self.left.tensor_specs(), **self.right.tensor_specs()}

    def bind(self, weights, ctx: BuildContext) -> None:
        self.ctx = ctx
        self.left.bind(weights, ctx)
        self.right.bind(weights, ctx)

    def _share(self, cache, which: int):
        columns = self._columns[which]
        state = None if columns is None else cache.state[:, columns[0] : columns[0] + columns[1]]
        return dataclasses.replace(cache, state=state)

    def forward(self, x, step, cache):
        """-> (left's result, right's result): a pair that a norm's kernel adds up."""
        return self.left.forward(x, step, self._share(cache, 0)), self.right.forward(x, step, self._share(cache, 1))
