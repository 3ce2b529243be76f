"""A matrix memory per head that is carried from token to token (the mLSTM recurrence): no keys and
values in the cache, but a state of fixed size per sequence.

With H heads, keys of dk and values of dv dims (all from n, the mixer's input):
    q = W_q n * q_scale,  k = W_k n,  v = W_v n,  g = W_g n          (q_scale: dk^-1/2 unless given)
    i = cap tanh((W_i n + b_i) / cap),   f = logsigmoid(cap tanh((W_f n + b_f) / cap))    per head, fp32
    m_t = max(f + m_(t-1), i)
    S_t = exp(f + m_(t-1) - m_t) S_(t-1) + exp(i - m_t) k v^T;   n_t likewise with k alone
    y = S_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6)
    out = W_o (rms over each head of y * norm * sigmoid(g))
S, n and m start at zero and live in 32-bit floats in the sequence's row of the cache's state area,
which the kernel addresses on the device through the step's slots: prompt steps, one-token steps, mixed
steps and replayed graphs run the same launches. The two gates' product has 32-bit sums and a 32-bit
result also under bfloat16 activations and weights: what enters the recurrence's exponentials is never
rounded to 16 bits.

names: the suffixes of its tensors (q, k, v, g, o, norm, i, f, i_bias, f_bias)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import BuildEnv, LayerCache, Mixer, StepContext, TensorSpec, param, register_part, tensor_name
from .linear import Linear

_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "g": "gate.weight", "o": "out_proj.weight",
          "norm": "norm.weight", "i": "igate.weight", "f": "fgate.weight", "i_bias": "igate.bias", "f_bias": "fgate.bias"}


@register_part("mixer", "mlstm")
class MatrixMemory(Mixer):
    accepts_normed_rows = False

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.hidden = param(params, "hidden_size", int)
        self.H = param(params, "num_heads", int)
        self.dk = param(params, "head_dim", int)
        self.dv = param(params, "value_dim", int, self.dk)
        self.cap = param(params, "gate_cap", float, 0.0)
        self.eps = param(params, "eps", float)
        self.q_scale = param(params, "q_scale", float, self.dk ** -0.5)
        self.out_scale = param(params, "out_scale", float, 1.0)
        if min(self.H, self.dk, self.dv) <= 0:
            raise ValueError("mlstm: heads, head_dim and value_dim must be positive")
        if self.dk > 512:
            raise ValueError(f"mlstm: head_dim {self.dk} above 512")
        names = param(params, "names", dict, {})
        self._names = {k: tensor_name(prefix, names, k, d) for k, d in _NAMES.items()}
        self.qkvg: Linear | None = None
        self.gates: Linear | None = None
        self.o_proj: Linear | None = None
        self.norm = None

    def _state_floats(self) -> int:
        # the rule of csrc/matrix_memory.hip, kept here so that the cache can be sized where no kernel
        # library is loaded: 8 key dims a thread, a power of two of threads a value dim, workgroups of
        # up to 256 threads, and n and m once a workgroup
        ng = 1
        while ng * 8 < self.dk:
            ng *= 2
        pb = max(1, min(self.dv, 256 // ng))
        tiles = -(-self.dv // pb)
        return self.H * self.dv * ng * 8 + self.H * tiles * (ng * 8 + 4)

    def state_bytes(self) -> int:
        return 4 * self._state_floats()

    def tensor_specs(self):
        n, H, dk, dv, D = self._names, self.H, self.dk, self.dv, self.hidden
        return {n["q"]: TensorSpec((H * dk, D)), n["k"]: TensorSpec((H * dk, D)), n["v"]: TensorSpec((H * dv, D)),
                n["g"]: TensorSpec((H * dv, D)), n["o"]: TensorSpec((D, H * dv)),
                n["norm"]: TensorSpec((H * dv,), ("gain", 1.0, 0.1)),
                n["i"]: TensorSpec((H, D)), n["f"]: TensorSpec((H, D)),
                n["i_bias"]: TensorSpec((H,), ("gain", -1.0, 0.5)), n["f_bias"]: TensorSpec((H,), ("gain", 3.0, 1.0))}

    def bind(self, tensors):
        n = self._names
        ws = [tensors.pop(n[x]) for x in ("q", "k", "v", "g")]
        if len({w.dtype for w in ws}) != 1:
            raise TypeError(f"{self.prefix}: the projections are stored in different dtypes")
        self.qkvg = Linear(torch.cat(ws, 0).contiguous())
        del ws
        f32 = torch.float32
        # the gates' rows stay in the stored dtype: products of bfloat16 numbers are exact in 32 bits, and the sums
        # and the result are 32-bit (out_dtype below), so nothing that enters the exponentials is rounded to 16 bits
        self.gates = Linear(torch.cat([tensors[n["i"]], tensors[n["f"]]], 0).contiguous())
        self.gate_bias = torch.cat([tensors[n["i_bias"]].to(f32), tensors[n["f_bias"]].to(f32)], 0).contiguous()
        self.o_proj = Linear(tensors[n["o"]])
        self.norm = tensors[n["norm"]]

    def forward(self, x, ctx: StepContext, cache: LayerCache, out_scale: float = 1.0):
        if cache.state is None:
            raise RuntimeError(f"{self.prefix}: a matrix memory needs its row of the state area")
        rows, H, dk, dv = ctx.rows, self.H, self.dk, self.dv
        if ops.mlstm_state_floats(H, dk, dv) != self._state_floats():
            raise RuntimeError(f"{self.prefix}: the kernel's state layout differs from the cache's")
        proj = self.qkvg(x, rows, ctx)                                   # [rows, q | k | v | g]
        pre = self.gates(x, rows, ctx, out_dtype=torch.float32)          # [rows, i | f], 32-bit; the scan bounds them
        y = ctx.alloc((rows, H * dv), torch.float32)
        if ctx.padded:
            y.zero_()           # the scan writes the rows of sequences only
        ops.mlstm_scan(y, proj[:, :H * dk], proj[:, H * dk:2 * H * dk], proj[:, 2 * H * dk:2 * H * dk + H * dv], pre,
                       cache.state, 0, ctx.cu_seqlens, ctx.seq_slot, rows, ctx.num_seqs, H, dk, dv, self.q_scale,
                       raw_gates=True, gate_bias=self.gate_bias, cap=self.cap)
        g = ctx.alloc((rows, H * dv))
        ops.gated_group_norm(g, y, proj[:, 2 * H * dk + H * dv:], self.norm, rows, H, self.eps, gate_after=True,
                             out_scale=self.out_scale * out_scale)
        return self.o_proj(g, rows, ctx)
