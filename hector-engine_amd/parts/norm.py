"""RMS normalisation: y = x * rsqrt(mean(x^2) + eps) * weight, the weight
multiplying directly (reference: kernels/normalization.cu:36-63). Applied to the
fp32 residual stream, fused with the pending residual add
(kernels/fused_add_rmsnorm.cu:47-81)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BuildEnv, Norm, StepContext, TensorSpec, param, register_part, tensor_name


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.size = param(params, "size", int)
        self.eps = param(params, "eps", float)
        # names: the suffix of its tensor (weight)
        self._name = tensor_name(prefix, param(params, "names", dict, {}), "weight", "weight")
        self.weight: torch.Tensor | None = None

    def tensor_specs(self):
        return {self._name: TensorSpec((self.size,), ("gain", 1.0, 0.1))}

    def bind(self, tensors):
        self.weight = tensors[self._name]

    def carried(self):
        return self.weight, self.eps

    def add_norm(self, resid, delta, rows, ctx: StepContext, want_out: bool = True, delta_scale: float = 1.0):
        out = ctx.alloc((rows, self.size)) if want_out else None
        if delta is not None and delta_scale != 1.0:
            ops.residual_add(resid, delta, rows, delta_scale)
            delta = None
        ops.add_rmsnorm(resid, delta, self.weight, out, rows, self.eps)
        return out


@register_part("norm", "dynamic_tanh")
class DynamicTanh(Norm):
    """y = tanh(alpha * x) * weight + bias with a stored scalar alpha and vectors weight, bias: it
    stands where a norm would and computes neither a mean nor a variance, so no row is reduced and no
    pair of products has a row scale to carry; where a product adds into the stream itself (steps of
    up to 64 rows), its epilogue computes this norm in full. Computed in fp32 on the fp32 residual stream, fused with the
    pending (scaled) residual add. names: suffixes of its tensors (weight, bias, alpha)."""

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.size = param(params, "size", int)
        names = param(params, "names", dict, {})
        self._names = {k: tensor_name(prefix, names, k, k) for k in ("weight", "bias", "alpha")}
        self.weight = self.bias = self.alpha = None

    def tensor_specs(self):
        n = self._names
        return {n["weight"]: TensorSpec((self.size,), ("gain", 1.0, 0.1)),
                n["bias"]: TensorSpec((self.size,), ("normal", 0.02)),
                n["alpha"]: TensorSpec((), ("gain", 0.5, 0.05))}

    def bind(self, tensors):
        n = self._names
        self.weight, self.bias, self.alpha = tensors[n["weight"]], tensors[n["bias"]], tensors[n["alpha"]]
        if not (self.weight.dtype == self.bias.dtype == self.alpha.dtype):
            raise TypeError(f"{self.prefix}: weight, bias and alpha are stored in different dtypes")

    def carried(self):
        return self.weight, 1.0, self.bias, self.alpha

    def add_norm(self, resid, delta, rows, ctx: StepContext, want_out: bool = True, delta_scale: float = 1.0):
        out = ctx.alloc((rows, self.size)) if want_out else None
        ops.add_dyt(resid, delta, self.weight, self.bias, self.alpha, out, rows, delta_scale)
        return out


@register_part("norm", "group_rmsnorm")
class GroupRMSNorm(Norm):
    """RMS norm in groups: the vector is cut into `groups` equal consecutive parts, each is divided by its own
    sqrt(mean(part^2) + eps), and the whole is multiplied by weight. No pair of products carries it (a row has
    several scales). names: the suffix of its tensor (weight)."""

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.size = param(params, "size", int)
        self.groups = param(params, "groups", int, 1)
        self.eps = param(params, "eps", float)
        if self.groups <= 0 or self.size % self.groups:
            raise ValueError(f"group_rmsnorm: {self.groups} groups do not divide the size {self.size}")
        self._name = tensor_name(prefix, param(params, "names", dict, {}), "weight", "weight")
        self.weight: torch.Tensor | None = None

    def tensor_specs(self):
        return {self._name: TensorSpec((self.size,), ("gain", 1.0, 0.1))}

    def bind(self, tensors):
        self.weight = tensors[self._name]

    def add_norm(self, resid, delta, rows, ctx: StepContext, want_out: bool = True, delta_scale: float = 1.0):
        if delta is not None:
            ops.residual_add(resid, delta, rows, delta_scale)
        if not want_out:
            return None
        out = ctx.alloc((rows, self.size))
        ops.add_group_normed(resid, None, None, 1, 0.0, 1.0, out, rows, next_weight=self.weight,
                             next_groups=self.groups, next_eps=self.eps)
        return out

    def add_normed_delta(self, resid, delta, rows: int, scale: float, out) -> None:
        """resid += scale * norm(delta); out (or None) receives the new rows of resid in its own dtype."""
        ops.add_group_normed(resid, delta, self.weight, self.groups, self.eps, scale, out, rows)
