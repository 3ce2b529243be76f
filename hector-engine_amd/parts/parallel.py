"""Mixers side by side: every branch reads the same input, and the result is the weighted sum
    out = sum_b scale_b * branch_b(n).
At most one branch keeps keys and values in the cache (the layer's cache group is that branch's); the
branches' per-sequence states lie one behind the other in the layer's row of the state area.

branches: a list of {"mixer": PartSpec, "scale": float, "name": suffix of the branch's prefix}."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BuildEnv, LayerCache, Mixer, PartSpec, StepContext, build_part, param, register_part


@register_part("mixer", "parallel")
class ParallelMixers(Mixer):
    accepts_normed_rows = False

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        branches = param(params, "branches", list)
        if not branches:
            raise ValueError("parallel: no branches")
        self.branches: list[Mixer] = []
        self.scales: list[float] = []
        for b in branches:
            spec = b["mixer"]
            if not isinstance(spec, PartSpec):
                raise TypeError("parallel: a branch's mixer must be a PartSpec")
            self.branches.append(build_part("mixer", spec, prefix + b["name"] + ".", env))
            self.scales.append(float(b.get("scale", 1.0)))
        if sum(m.kv_need() is not None for m in self.branches) > 1:
            raise ValueError("parallel: at most one branch may keep keys and values in the cache")
        self.graph_safe = all(m.graph_safe for m in self.branches)
        # each branch's span of the state row, begun on 256 bytes
        self._state_at: list[tuple[int, int]] = []
        at = 0
        for m in self.branches:
            n = m.state_bytes()
            self._state_at.append((at, n))
            at += (n + 255) // 256 * 256 if n else 0
        self._state_bytes = at

    def children(self):
        return list(self.branches)

    def kv_need(self):
        for m in self.branches:
            need = m.kv_need()
            if need is not None:
                return need
        return None

    def state_bytes(self) -> int:
        return self._state_bytes

    def tensor_specs(self):
        specs = {}
        for m in self.branches:
            specs.update(m.tensor_specs())
        return specs

    def bind(self, tensors):
        for m in self.branches:
            m.bind(tensors)

    def forward(self, x, ctx: StepContext, cache: LayerCache):
        rows = ctx.rows
        ctx.sink = None
        total = None
        scale_of_total = 1.0
        for m, scale, (at, n) in zip(self.branches, self.scales, self._state_at):
            state = cache.state[:, at:at + n] if n and cache.state is not None else None
            mine = LayerCache(cache.kpool, cache.vpool, cache.page_table, cache.writes, state) \
                if m.kv_need() is not None else LayerCache(None, None, None, False, state)
            out = m.forward(x, ctx, mine)
            if total is None:
                total, scale_of_total = out, scale
            else:
                joined = ctx.alloc((rows, out.shape[-1]), out.dtype)
                ops.scaled_sum(joined, total, out, rows, scale_of_total, scale)
                total, scale_of_total = joined, 1.0
        if scale_of_total != 1.0:
            joined = ctx.alloc((rows, total.shape[-1]), total.dtype)
            ops.scaled_sum(joined, total, total, rows, scale_of_total, 0.0)
            total = joined
        return total
