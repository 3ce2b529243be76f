"""A gated delta rule mixer: a matrix per head that is carried from token to token; no keys and values
in the cache, but a state of fixed size per sequence.

With H heads over G groups of queries and keys (head h reads the q and k of group h // (H / G)), keys of
d and values of e dims, all from n, the mixer's input:
    q = W_q n, k = W_k n (G x d), v = W_v n (H x e); each through a causal convolution per channel over the
    last K inputs and SiLU; q and k to unit length per head, x / sqrt(sum(x^2) + unit_eps), q times d^-1/2
    beta = sigmoid(W_b n),   g = exp(-exp(A_log) softplus(W_a n + dt_bias))        per head, fp32
    S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q                   (S [d, e], fp32)
    out = W_o (rms over each head of o * norm * silu(W_g n))                         (norm [e], shared by the heads)
A sequence carries the last K - 1 inputs of the convolution and S (zeros at its start) in its row of the
cache's state area, which the kernels address on the device through the step's slots: prompt steps,
one-token steps, mixed steps and replayed graphs run the same launches, and a token's sums do not depend
on how the rows were cut into steps. The product of the two gates' rows has 32-bit sums and a 32-bit
result also under bfloat16: what enters the sigmoid, the softplus and the exponentials is never rounded
to 16 bits.

names: the suffixes of its tensors (q, k, v, q_conv, k_conv, v_conv, b, a, A_log, dt_bias, g, norm, o)."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.random_init import register_init
from .base import BuildEnv, LayerCache, Mixer, StepContext, TensorSpec, param, register_part, tensor_name
from .linear import Linear

_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "q_conv": "q_conv.weight",
          "k_conv": "k_conv.weight", "v_conv": "v_conv.weight", "b": "b_proj.weight", "a": "a_proj.weight",
          "A_log": "A_log", "dt_bias": "dt_bias", "g": "g_proj.weight", "norm": "norm.weight", "o": "o_proj.weight"}

# random values for the tests' and the benchmark's models: decay rates exp(A_log) around 1 and decay inputs
# around -1, so that a head forgets over tens of tokens
register_init("delta_a_log", lambda init: (0.0, 0.5))
register_init("delta_dt_bias", lambda init: (-1.0, 0.5))


def state_floats(H: int, d: int, e: int) -> int:
    """Floats of the heads' matrices as the scan kernel keeps them (the rule of csrc/delta_rule.hip, kept here
    so that the cache can be sized where no kernel library is loaded): a value dim's column is held by a power
    of two of lanes with 8 to 32 key dims each, in steps of 8, the fewest dims in all."""
    padded = [g * per for g in (1, 2, 4, 8, 16, 32, 64) for per in [(-(-d // g) + 7) // 8 * 8] if per <= 32]
    if not padded:
        raise ValueError(f"gated_delta: key width {d} above 2048")
    return H * e * min(padded)


@register_part("mixer", "gated_delta")
class GatedDeltaRule(Mixer):
    accepts_normed_rows = False

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.hidden = param(params, "hidden_size", int)
        self.H = param(params, "num_heads", int)
        self.G = param(params, "num_kv_heads", int, self.H)
        self.d = param(params, "head_dim", int)
        self.e = param(params, "value_dim", int, self.d)
        self.K = param(params, "conv_taps", int)
        self.eps = param(params, "eps", float)
        self.unit_eps = param(params, "unit_eps", float, 1e-6)
        self.q_scale = param(params, "q_scale", float, self.d ** -0.5)
        if min(self.H, self.G, self.d, self.e, self.K) <= 0 or self.H % self.G:
            raise ValueError("gated_delta: sizes must be positive and the heads a multiple of the q/k groups")
        self.C = 2 * self.G * self.d + self.H * self.e          # channels of the convolution: q | k | v
        state_floats(self.H, self.d, self.e)
        names = param(params, "names", dict, {})
        self._names = {k: tensor_name(prefix, names, k, v) for k, v in _NAMES.items()}
        self.qkvg: Linear | None = None
        self.gates: Linear | None = None
        self.o_proj: Linear | None = None
        self.taps = self.a_log = self.dt_bias = self.norm = None

    # bytes of the carried convolution inputs, rounded so that the matrices start on 16 bytes
    def _conv_bytes(self) -> int:
        return (4 * (self.K - 1) * self.C + 15) // 16 * 16

    def state_bytes(self) -> int:
        return self._conv_bytes() + 4 * state_floats(self.H, self.d, self.e)

    def tensor_specs(self):
        n, H, G, d, e, D, K = self._names, self.H, self.G, self.d, self.e, self.hidden, self.K
        return {n["q"]: TensorSpec((G * d, D)), n["k"]: TensorSpec((G * d, D)), n["v"]: TensorSpec((H * e, D)),
                n["q_conv"]: TensorSpec((G * d, K), ("normal", 0.4)), n["k_conv"]: TensorSpec((G * d, K), ("normal", 0.4)),
                n["v_conv"]: TensorSpec((H * e, K), ("normal", 0.4)),
                n["b"]: TensorSpec((H, D)), n["a"]: TensorSpec((H, D)),
                n["A_log"]: TensorSpec((H,), ("delta_a_log",)), n["dt_bias"]: TensorSpec((H,), ("delta_dt_bias",)),
                n["g"]: TensorSpec((H * e, D)), n["norm"]: TensorSpec((e,), ("gain", 1.0, 0.1)),
                n["o"]: TensorSpec((D, H * e))}

    def bind(self, tensors):
        n = self._names
        ws = [tensors.pop(n[x]) for x in ("q", "k", "v", "g")]
        if len({w.dtype for w in ws}) != 1:
            raise TypeError(f"{self.prefix}: the projections are stored in different dtypes")
        self.qkvg = Linear(torch.cat(ws, 0).contiguous())
        del ws
        # the gates' rows stay in the stored dtype: the products are exact in 32 bits, and the sums and the result
        # are 32-bit (out_dtype below)
        self.gates = Linear(torch.cat([tensors[n["b"]], tensors[n["a"]]], 0).contiguous())
        self.taps = torch.cat([tensors[n[x]] for x in ("q_conv", "k_conv", "v_conv")], 0).contiguous()
        self.a_log, self.dt_bias = tensors[n["A_log"]], tensors[n["dt_bias"]]
        if self.a_log.dtype != self.dt_bias.dtype:
            raise TypeError(f"{self.prefix}: A_log and dt_bias are stored in different dtypes")
        self.norm = tensors[n["norm"]].repeat(self.H).contiguous()     # one gain vector for every head
        self.o_proj = Linear(tensors[n["o"]])

    def forward(self, x, ctx: StepContext, cache: LayerCache):
        if cache.state is None:
            raise RuntimeError(f"{self.prefix}: a delta-rule mixer needs its row of the state area")
        rows, H, G, d, e, C = ctx.rows, self.H, self.G, self.d, self.e, self.C
        if ops.delta_state_floats(H, d, e) != state_floats(H, d, e):
            raise RuntimeError(f"{self.prefix}: the scan kernel's state layout differs from the cache's")
        proj = self.qkvg(x, rows, ctx)                                   # [rows, q | k | v | g]
        ba = self.gates(x, rows, ctx, out_dtype=torch.float32)           # [rows, b | a], 32-bit
        qkv = ctx.alloc((rows, C))
        ops.conv_state(qkv, proj[:, :C], self.taps, None, cache.state, ctx.positions, ctx.row_seq, ctx.seq_slot,
                       ctx.seq_start, ctx.cu_seqlens, rows, ctx.num_seqs, ctx.all_single, act=True)
        y = ctx.alloc((rows, H * e), torch.float32)
        if ctx.padded:
            y.zero_()           # the scan writes the rows of sequences only
        ws = ctx.alloc((max(4, ops.delta_workspace_floats(rows, H, G, d)),), torch.float32)
        ops.delta_scan(y, qkv[:, :G * d], qkv[:, G * d:2 * G * d], qkv[:, 2 * G * d:], ba, self.a_log, self.dt_bias,
                       cache.state, self._conv_bytes(), ctx.cu_seqlens, ctx.seq_slot, rows, ctx.num_seqs, H, G, d, e,
                       self.q_scale, self.unit_eps, workspace=ws)
        out = ctx.alloc((rows, H * e))
        ops.gated_group_norm(out, y, proj[:, C:], self.norm, rows, H, self.eps, gate_after="silu")
        return self.o_proj(out, rows, ctx, sink=ctx.take_sink())
