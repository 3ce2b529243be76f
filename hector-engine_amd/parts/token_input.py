"""A per-layer input from the token itself, gated by the stream:
    e = table[token][offset : offset + dim];  g = act(W_gate x) * e;  y = W_proj g
where x is the residual stream as it stands (in the activation dtype, no norm in front), `table` a
second embedding table that all layers share (each reads its own stretch of `dim` columns of a token's
row), and y passes an RMS norm with a stored gain before it joins the stream (the block's business:
post_norm() names gain and eps). activation: "gelu_tanh" unless given.

table: the full name of the shared table; names: the suffixes of its own tensors (gate, proj, norm)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BuildEnv, StepContext, TensorSpec, TokenInput, param, register_part, tensor_name
from .linear import Linear


@register_part("token_input", "gated_token_input")
class GatedTokenInput(TokenInput):
    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.hidden = param(params, "hidden_size", int)
        self.vocab = param(params, "vocab_size", int)
        self.dim = param(params, "dim", int)
        self.offset = param(params, "offset", int, 0)
        self.table_width = param(params, "table_width", int, self.offset + self.dim)
        self.eps = param(params, "eps", float)
        self.act = param(params, "activation", str, "gelu_tanh")
        if self.dim <= 0 or self.offset < 0 or self.offset + self.dim > self.table_width:
            raise ValueError(f"gated_token_input: columns {self.offset}..{self.offset + self.dim} do not lie in a "
                             f"table row of {self.table_width}")
        if self.act not in ops.ACT_KINDS:
            raise ValueError(f"gated_token_input: unsupported activation '{self.act}'")
        self._table = param(params, "table", str)
        names = param(params, "names", dict, {})
        self._names = {k: tensor_name(prefix, names, k, d) for k, d in
                       (("gate", "gate.weight"), ("proj", "proj.weight"), ("norm", "norm.weight"))}
        self.table = self.norm = None
        self.gate: Linear | None = None
        self.proj: Linear | None = None

    def tensor_specs(self):
        n = self._names
        return {self._table: TensorSpec((self.vocab, self.table_width), ("normal", 1.0)),
                n["gate"]: TensorSpec((self.dim, self.hidden)),
                n["proj"]: TensorSpec((self.hidden, self.dim)),
                n["norm"]: TensorSpec((self.hidden,), ("gain", 1.0, 0.1))}

    def bind(self, tensors):
        n = self._names
        self.table = tensors[self._table]
        self.gate = Linear(tensors[n["gate"]])
        self.proj = Linear(tensors[n["proj"]])
        self.norm = tensors[n["norm"]]

    def post_norm(self):
        return self.norm, self.eps

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        if ctx.tokens is None:
            raise RuntimeError(f"{self.prefix}: the step's token ids are not at hand")
        rows = ctx.rows
        t = self.gate(x, rows, ctx)
        ops.token_gate(t, t, self.table, ctx.tokens, rows, self.offset, self.act)
        return self.proj(t, rows, ctx)
