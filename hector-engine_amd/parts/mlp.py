"""Dense gated feed-forward: d = (act(x Wg^T) * (x Wu^T)) Wd^T with act = SiLU,
no biases (reference: src/graph_builder.cpp:1415-1428,
kernels/activations.cu:183-198). Gate and up are one product over the
row-concatenated weight gate||up (the reference's optional fusion:
src/graph_builder.cpp:1400-1414).

activation "clamped_swiglu" is the same feed-forward through a bounded gate:
g' = min(g, limit), u' = clamp(u, -limit, limit), act = g' * sigmoid(alpha * g') * (u' + 1), with
the parameters `limit` and `alpha` (1.702 unless given). names: the suffixes of its tensors
(gate, up, down)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import (BuildEnv, FeedForward, NormedRows, PieceRows, StepContext, TensorSpec, param, register_part,
                   tensor_name)
from .linear import Linear

# rows of the intermediate activations held at once in a long prompt step
_ROW_CHUNK = 8192


@register_part("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    accepts_normed_rows = True

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.hidden = param(params, "hidden_size", int)
        self.inter = param(params, "intermediate_size", int)
        act = param(params, "activation", str, "silu")
        if act in ("silu", "swish"):
            self.act = {}                         # SiLU(gate) * up
        elif act == "clamped_swiglu":
            limit = param(params, "limit", float)
            if limit <= 0:
                raise ValueError(f"gated_mlp: limit {limit} must be positive")
            self.act = {"alpha": param(params, "alpha", float, 1.702), "limit": limit, "up_shift": 1.0}
        else:
            raise ValueError(f"gated_mlp: unsupported activation '{act}'")
        names = param(params, "names", dict, {})
        self._names = {k: tensor_name(prefix, names, k, d) for k, d in
                       (("gate", "gate_proj.weight"), ("up", "up_proj.weight"), ("down", "down_proj.weight"))}
        self.gate_up: Linear | None = None
        self.down: Linear | None = None

    def tensor_specs(self):
        n = self._names
        return {
            n["gate"]: TensorSpec((self.inter, self.hidden)),
            n["up"]: TensorSpec((self.inter, self.hidden)),
            n["down"]: TensorSpec((self.hidden, self.inter)),
        }

    def bind(self, tensors):
        p, n = self.prefix, self._names
        g, u = tensors.pop(n["gate"]), tensors.pop(n["up"])
        if g.dtype != u.dtype:
            raise TypeError(f"{p}gate_proj and up_proj are stored in different dtypes")
        # gate and up rows alternate (gate i at row 2i, its up at 2i + 1): the four neighbouring
        # rows whose sums a thread of the MFMA product holds are then two (gate, up) pairs, and
        # the gated activation is that product's epilogue
        w = torch.stack([g, u], 1).reshape(2 * g.shape[0], g.shape[1])
        self.gate_up = Linear(w.contiguous())
        del g, u, w
        self.down = Linear(tensors[n["down"]])

    def forward(self, x, ctx: StepContext):
        rows = ctx.rows
        if rows <= _ROW_CHUNK:
            act = x.scaled.dtype if isinstance(x, NormedRows) else x.dtype
            if self.gate_up.gated_silu_rows(rows, ctx, act):
                # up to 64 rows: the activation is the product's epilogue, and its result goes to the
                # down projection piece-major where that reads it so
                pieces = self.inter % 8 == 0 and self.down.reads_pieces(rows, ctx) and self.gate_up.gated_pieces(rows)
                h = ctx.alloc(ops.pieces_shape(rows, self.inter) if pieces else (rows, self.inter))
                self.gate_up.gated_silu(x, rows, ctx, h, out_pieces=pieces, act=self.act)
                return self.down(PieceRows(h) if pieces else h, rows, ctx, sink=ctx.take_sink())
            h = ctx.alloc((rows, self.inter))
            gu = self.gate_up(x, rows, ctx)
            ops.silu_mul(h, gu, rows, True, **self.act)
            return self.down(h, rows, ctx, sink=ctx.take_sink())
        if not isinstance(x, torch.Tensor):
            x = x.tensor(ctx)
        out = ctx.alloc((rows, self.hidden))
        for r0 in range(0, rows, _ROW_CHUNK):
            n = min(_ROW_CHUNK, rows - r0)
            turn = ctx.scratch.mark()
            h = ctx.alloc((n, self.inter))
            gu = self.gate_up(x[r0:r0 + n], n, ctx)
            ops.silu_mul(h, gu, n, True, **self.act)
            self.down(h, n, ctx, out=out[r0:r0 + n])
            ctx.scratch.release(turn)       # the next turn reuses h and gate||up
        return out


@register_part("feed_forward", "dense_mlp")
class DenseMLP(FeedForward):
    """Feed-forward without a gate: d = act(x Wu^T) Wd^T, no biases. activation: "relu2" (the square of
    relu), "gelu_tanh", "silu" or "relu", element by element; or "polynorm", over a token's whole vector z of
    intermediate values: a N(z) + b N(z^2) + c N(z^3) + e, powers element by element, N the division by the root
    mean square (eps `eps` inside the root), (a, b, c, e) the four stored numbers of the tensor `act`.
    names: the suffixes of its tensors (up, down, act)."""

    accepts_normed_rows = True

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.hidden = param(params, "hidden_size", int)
        self.inter = param(params, "intermediate_size", int)
        self.act = param(params, "activation", str, "relu2")
        if self.act not in ops.ACT_KINDS and self.act != "polynorm":
            raise ValueError(f"dense_mlp: unsupported activation '{self.act}', have {sorted(ops.ACT_KINDS) + ['polynorm']}")
        self.eps = param(params, "eps", float, 1e-6)
        self.numbers = None
        names = param(params, "names", dict, {})
        self._names = {k: tensor_name(prefix, names, k, d) for k, d in
                       (("up", "up_proj.weight"), ("down", "down_proj.weight"), ("act", "act.weight"))}
        self.up: Linear | None = None
        self.down: Linear | None = None

    def tensor_specs(self):
        n = self._names
        specs = {n["up"]: TensorSpec((self.inter, self.hidden)), n["down"]: TensorSpec((self.hidden, self.inter))}
        if self.act == "polynorm":
            specs[n["act"]] = TensorSpec((4,), ("gain", 0.3, 0.2))
        return specs

    def bind(self, tensors):
        n = self._names
        self.up = Linear(tensors[n["up"]])
        self.down = Linear(tensors[n["down"]])
        if self.act == "polynorm":
            self.numbers = tensors[n["act"]]

    def _activate(self, h, rows: int) -> None:
        if self.act == "polynorm":
            ops.polynorm(h, h, self.numbers, rows, self.eps)
        else:
            ops.unary_act(h, h, rows, self.act)

    def forward(self, x, ctx: StepContext):
        rows = ctx.rows
        if rows <= _ROW_CHUNK:
            h = self.up(x, rows, ctx)
            self._activate(h, rows)
            return self.down(h, rows, ctx, sink=ctx.take_sink())
        if not isinstance(x, torch.Tensor):
            x = x.tensor(ctx)
        out = ctx.alloc((rows, self.hidden))
        for r0 in range(0, rows, _ROW_CHUNK):
            n = min(_ROW_CHUNK, rows - r0)
            turn = ctx.scratch.mark()
            h = self.up(x[r0:r0 + n], n, ctx)
            self._activate(h, n)
            self.down(h, n, ctx, out=out[r0:r0 + n])
            ctx.scratch.release(turn)
        return out
