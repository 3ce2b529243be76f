"""A routed feed-forward (mixture of experts): each token uses `top` of its experts.

    z = W_router n                    fp32, E + I outputs: E experts with weights, then I without
    s = softmax(z)                    over all outputs
    c = s + correction                the choice is made on c, the weights on s
    the outputs are cut into `groups` equal runs of neighbours, each run ranked by the largest c it
    holds; outside the `keep` best runs every c is replaced by -inf; the `top` largest c that are left
    are chosen, and a chosen output weighs s * scale (the weights are not made to sum to one)
    expert e: g = min(W_gate n, limit), u = clamp(W_up n, -limit, limit),
              y = g * sigmoid(alpha g) * (u + 1), result W_down y          (no biases)
    the I outputs without weights are identity experts: their result is n itself
    out = sum over the chosen outputs of weight * result

How it runs: one kernel for the router's product in fp32 (its matrix is kept in 32-bit) and the
choice, and then the experts as one feed-forward: all gate and up rows side by side
in one product, the activation kernel multiplies each expert's stretch by the token's weight for
it (an exact 0 where it was not chosen) and appends weight * n for the identity experts, and one
product with the down matrices side by side (and an identity block) adds everything up. Every step
has the same launches whatever the tokens choose, so it replays as a graph, and a token's sums do
not depend on the rest of the batch. A bfloat16 step of so few rows that they cannot choose more than
half of the experts reads only the chosen experts' rows of the same matrices (ops.chosen_experts).
Options: `normalize` divides the chosen outputs' weights by their sum (the softmax over the chosen logits
alone; the choice itself is the same, the softmax being monotone); `shared` = {"feed_forward": PartSpec, "name":
suffix of its prefix, "gate": suffix of a stored vector of hidden_size or None} adds an expert that every token
uses, out += sigmoid(gate . n) * shared(n) (gate None: out += shared(n)), the dot product in fp32.
names: the suffixes of its tensors (router, correction; expert e's are 'e<e>.' + gate / up / down).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BuildEnv, FeedForward, PartSpec, StepContext, TensorSpec, build_part, param, register_part, tensor_name
from .linear import Linear

# rows whose gate and up columns are held at once in a long prompt step
_ROW_CHUNK = 4096


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.hidden = param(params, "hidden_size", int)
        self.inter = param(params, "intermediate_size", int)
        self.real = param(params, "experts", int)
        self.identity = param(params, "identity_experts", int, 0)
        self.top = param(params, "top", int)
        self.scale = param(params, "scale", float, 1.0)
        self.groups = param(params, "groups", int, 1)
        self.keep = param(params, "keep_groups", int, self.groups)
        self.has_correction = param(params, "correction", bool, True)
        self.normalize = param(params, "normalize", bool, False)
        shared = param(params, "shared", dict, None)
        self.shared = self.shared_gate = self._shared_gate = None
        if shared:
            self.shared = build_part("feed_forward", shared["feed_forward"], prefix + shared.get("name", "shared") + ".", env)
            if shared.get("gate"):
                self._shared_gate = prefix + shared.get("name", "shared") + "." + shared["gate"]
        self.limit = param(params, "limit", float, 0.0)
        self.alpha = param(params, "alpha", float, 1.702 if self.limit > 0 else 1.0)
        self.up_shift = param(params, "up_shift", float, 1.0 if self.limit > 0 else 0.0)
        E = self.real + self.identity
        if self.real <= 0 or self.identity < 0 or self.inter <= 0:
            raise ValueError("routed_experts: experts and intermediate_size must be positive, identity_experts not negative")
        if self.groups <= 0 or E % self.groups or not 0 < self.keep <= self.groups:
            raise ValueError(f"routed_experts: {E} router outputs do not form {self.groups} equal groups "
                             f"of which {self.keep} are kept")
        if not 0 < self.top <= self.keep * (E // self.groups):
            raise ValueError(f"routed_experts: top {self.top} exceeds the {self.keep * (E // self.groups)} outputs "
                             "of the kept groups")
        names = param(params, "names", dict, {})
        self._router = tensor_name(prefix, names, "router", "router.weight")
        self._correction = tensor_name(prefix, names, "correction", "router.correction")
        self._expert = names.get("expert", "experts.{e}.")
        self._sub = {k: names.get(k, d) for k, d in (("gate", "gate_proj.weight"), ("up", "up_proj.weight"),
                                                     ("down", "down_proj.weight"))}
        self.router: torch.Tensor | None = None
        self.correction = None
        self.gate_up: Linear | None = None
        self.down: Linear | None = None

    def _name(self, e: int, which: str) -> str:
        return self.prefix + self._expert.format(e=e) + self._sub[which]

    def tensor_specs(self):
        specs = {self._router: TensorSpec((self.real + self.identity, self.hidden))}
        if self.has_correction:
            specs[self._correction] = TensorSpec((self.real + self.identity,))
        for e in range(self.real):
            specs[self._name(e, "gate")] = TensorSpec((self.inter, self.hidden))
            specs[self._name(e, "up")] = TensorSpec((self.inter, self.hidden))
            specs[self._name(e, "down")] = TensorSpec((self.hidden, self.inter))
        if self.shared is not None:
            specs.update(self.shared.tensor_specs())
        if self._shared_gate:
            specs[self._shared_gate] = TensorSpec((1, self.hidden))
        return specs

    def children(self):
        return [self.shared] if self.shared is not None else []

    def bind(self, tensors):
        # the router's sums are 32-bit whatever the run's precision: its matrix is kept in float32
        self.router = tensors[self._router].to(torch.float32).contiguous()
        self.correction = tensors[self._correction] if self.has_correction else None
        gu, downs = [], []
        for e in range(self.real):
            g, u = tensors.pop(self._name(e, "gate")), tensors.pop(self._name(e, "up"))
            # gate i of an expert at row 2i of its stretch, its up at 2i + 1
            gu.append(torch.stack([g, u], 1).reshape(2 * self.inter, self.hidden))
            downs.append(tensors.pop(self._name(e, "down")))
        if self.identity:
            # the identity experts' share rides through the down product on an identity block
            downs.append(torch.eye(self.hidden, dtype=downs[0].dtype, device=downs[0].device))
        self.gate_up = Linear(torch.cat(gu, 0).contiguous())
        self.down = Linear(torch.cat(downs, 1).contiguous())
        if self.shared is not None:
            self.shared.bind(tensors)
        if self._shared_gate:
            self.shared_gate = tensors[self._shared_gate].reshape(-1).contiguous()

    def _few_rows(self, rows: int, x, ctx: StepContext) -> bool:
        """Whether the step runs through the chosen experts alone (kernels.ops.chosen_experts): bfloat16 with the
        fast kernels, sizes in multiples of 8, and so few rows that they cannot choose more than half of the
        experts. (The 32-bit path keeps the products over all experts, whose sums do not depend on the batch.)"""
        return (ctx.env.fast_kernels and x.dtype == torch.bfloat16 and self.gate_up.weight.dtype == torch.bfloat16
                and self.inter % 8 == 0 and self.hidden % 8 == 0 and 2 * rows * self.top <= self.real)

    def forward(self, x, ctx: StepContext):
        if self.shared is None:
            return self._routed(x, ctx, True)
        rows = ctx.rows
        routed = self._routed(x, ctx, False)
        common = self.shared.forward(x, ctx)
        out = ctx.alloc((rows, self.hidden))
        if self.shared_gate is not None:
            ops.gated_add(out, routed, common, x, self.shared_gate, rows)
        else:
            ops.scaled_sum(out, routed, common, rows, 1.0, 1.0)
        return out

    def _routed(self, x, ctx: StepContext, may_sink: bool):
        rows, real, I = ctx.rows, self.real, self.inter
        dense = ctx.alloc((rows, real + 1), torch.float32)
        ids = ctx.alloc((rows, self.top), torch.int32)
        weights = ctx.alloc((rows, self.top), torch.float32)
        # the router's product (fp32 sums over the rows as they are) and the choice, one launch
        ops.route_tokens(dense, ids, weights, None, self.correction, rows, real, self.groups, self.keep,
                         self.top, self.scale, x=x, router=self.router, normalize=self.normalize)
        cols = real * I + (self.hidden if self.identity else 0)
        act = {"alpha": self.alpha, "limit": self.limit, "up_shift": self.up_shift}
        if self._few_rows(rows, x, ctx):
            # the rows of the step choose at most half of the experts: only those experts' weights are read
            h = ctx.alloc((rows * self.top, I))
            out = ctx.alloc((rows, self.hidden))
            ops.chosen_experts(out, h, x, self.gate_up.weight, self.down.weight, ids, weights, dense, rows, real, I, **act)
            return out
        if rows <= _ROW_CHUNK:
            gu = self.gate_up(x, rows, ctx)
            h = ctx.alloc((rows, cols))
            ops.routed_act(h, gu, dense, x if self.identity else None, rows, real, I, **act)
            return self.down(h, rows, ctx, sink=ctx.take_sink() if may_sink else None)
        out = ctx.alloc((rows, self.hidden))
        for r0 in range(0, rows, _ROW_CHUNK):
            n = min(_ROW_CHUNK, rows - r0)
            turn = ctx.scratch.mark()
            gu = self.gate_up(x[r0:r0 + n], n, ctx)
            h = ctx.alloc((n, cols))
            ops.routed_act(h, gu, dense[r0:r0 + n], x[r0:r0 + n] if self.identity else None, n, real, I, **act)
            self.down(h, n, ctx, out=out[r0:r0 + n])
            ctx.scratch.release(turn)
        return out
