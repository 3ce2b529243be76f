"""Attention whose keys and values are one latent vector a token.

With H heads, d unrotated and r rotated query/key dims a head, values of e dims, a query latent of
q_rank and a key/value latent of `rank` dims, all from n, the mixer's input:
    c_q = rms(W_dq n) * g_q,   q = W_uq c_q                 a head's q is [d unrotated | r rotated]
    [c' | k_r] = W_dkv n,      c = rms(c') * g_kv           k_r: r dims, one rotated key part for all heads
    head h: key [W_uk,h c | rot(k_r)], value W_uv,h c, score (q_h . key) * scale
    causal, the last `window` positions (0: all), softmax with exp(sink_h) more in its denominator
    out = W_o (heads' results side by side)
The cache keeps c and rot(k_r) per token and nothing per head. Since q . (W_uk,h c) = (W_uk,h^T q) . c, the
step takes each head's unrotated query through W_uk,h^T and then runs the shared attention kernels as H
query heads over ONE key/value head whose key is [rot(k_r) | c] (r + rank wide, the rotated dims first, where
the rotation kernel turns them) and whose value is c; a head's result over the latents goes through W_uv,h
before the output product. The rotation is the position part's (half-split pairs, optional YaRN scaling,
whose factor on cos and sin rides along); the scale is taken as given.

Everything else (cache pages, window, sinks, the routes to the plain / MFMA kernels) is the attention part's.
names: the suffixes of its tensors (dq, dq_norm, uq, dkv, dkv_norm, uk, uv, sinks, o)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .attention import Attention
from .base import BuildEnv, LayerCache, PartSpec, StepContext, TensorSpec, param, register_part, tensor_name
from .linear import Linear

_NAMES = {"dq": "q_a_proj.weight", "dq_norm": "q_a_norm.weight", "uq": "q_b_proj.weight", "dkv": "kv_a_proj.weight",
          "dkv_norm": "kv_a_norm.weight", "uk": "k_b_proj.weight", "uv": "v_b_proj.weight", "sinks": "sinks",
          "o": "o_proj.weight"}


@register_part("mixer", "latent_attention")
class LatentAttention(Attention):
    accepts_normed_rows = False

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        self.d = param(params, "head_dim", int)            # unrotated dims of a head's query and key
        self.r = param(params, "rotary_dim", int, 0)        # rotated dims
        self.e = param(params, "value_dim", int, self.d)
        self.rank = param(params, "kv_rank", int)
        self.q_rank = param(params, "q_rank", int)
        self.norm_eps = param(params, "eps", float)
        heads = param(params, "num_heads", int)
        if min(self.d, self.e, self.rank, self.q_rank, heads) <= 0 or self.r < 0 or self.r % 2:
            raise ValueError("latent_attention: sizes must be positive and the rotated dims even")
        inner = {"hidden_size": param(params, "hidden_size", int), "num_heads": heads, "num_kv_heads": 1,
                 "head_dim": self.r + self.rank, "value_dim": self.rank, "window": param(params, "window", int, 0),
                 "scale": param(params, "scale", float), "sinks": param(params, "sinks", bool, False),
                 "position": param(params, "position", PartSpec, PartSpec("none"))}
        super().__init__(inner, prefix, env)
        rot = self.position.rotary()
        if self.position.custom or self.position.interleaved or (rot[1] if rot else 0) != self.r:
            raise ValueError("latent_attention: the position part must be a half-split rotation of exactly the rotated dims")
        names = param(params, "names", dict, {})
        self._lnames = {k: tensor_name(prefix, names, k, v) for k, v in _NAMES.items()}
        self.dq = self.dkv = self.uq = None
        self.dq_norm = self.dkv_norm = self.w_keys = self.w_values = None

    def tensor_specs(self):
        n, H, D = self._lnames, self.H, self.hidden
        specs = {n["dq"]: TensorSpec((self.q_rank, D)), n["dq_norm"]: TensorSpec((self.q_rank,), ("gain", 1.0, 0.1)),
                 n["uq"]: TensorSpec((H * (self.d + self.r), self.q_rank), ("normal", 0.1)),
                 n["dkv"]: TensorSpec((self.rank + self.r, D)), n["dkv_norm"]: TensorSpec((self.rank,), ("gain", 1.0, 0.1)),
                 n["uk"]: TensorSpec((H * self.d, self.rank), ("normal", 0.1)),
                 n["uv"]: TensorSpec((H * self.e, self.rank), ("normal", 0.1)),
                 n["o"]: TensorSpec((D, H * self.e))}
        if self.has_sinks:
            specs[n["sinks"]] = TensorSpec((H,), ("normal", 1.0))
        specs.update(self.position.tensor_specs())
        return specs

    def bind(self, tensors):
        n, H = self._lnames, self.H
        self.dq, self.dkv, self.uq = Linear(tensors[n["dq"]]), Linear(tensors[n["dkv"]]), Linear(tensors[n["uq"]])
        self.dq_norm, self.dkv_norm = tensors[n["dq_norm"]], tensors[n["dkv_norm"]]
        # a head's matrices as [head][in][out]: W_uk,h^T takes d to rank as it is stored, W_uv,h takes rank to e
        self.w_keys = tensors[n["uk"]].view(H, self.d, self.rank).contiguous()
        self.w_values = tensors[n["uv"]].view(H, self.e, self.rank).transpose(1, 2).contiguous()
        self.o_proj = Linear(tensors[n["o"]])
        if self.has_sinks:
            self.sinks = tensors[n["sinks"]]
        self.position.bind(tensors)

    def _encoded_q(self, x, ctx: StepContext, cache: LayerCache):
        if not cache.writes:
            raise RuntimeError(f"{self.prefix}: a latent attention keeps a cache of its own")
        rows, H, d, r, rank = ctx.rows, self.H, self.d, self.r, self.rank
        hd = r + rank
        cq = self.dq(x, rows, ctx)                                   # [rows, q_rank]
        down = self.dkv(x, rows, ctx)                                # [rows, rank | r]
        ops.rmsnorm_rows(cq, cq, self.dq_norm, rows, self.q_rank, self.q_rank, self.q_rank, self.norm_eps)
        ops.rmsnorm_rows(down, down, self.dkv_norm, rows, rank, rank + r, rank + r, self.norm_eps)
        q = self.uq(cq, rows, ctx)                                   # [rows, H (d | r)]
        qkv = ctx.alloc((rows, (H + 1) * hd + rank))                 # [H heads of (r | rank) | key (r | rank) | value rank]
        ops.head_product(qkv[:, :H * hd].unflatten(1, (H, hd))[:, :, r:], q.unflatten(1, (H, d + r))[:, :, :d],
                         self.w_keys, rows)
        ops.latent_pack(qkv, q, down, rows, H, d, r, rank)
        out = ctx.alloc((rows, H * self.pd))
        rot = self.position.rotary()
        ops.qkv_rope_cache(out, cache.kpool, cache.vpool, qkv, H * hd, hd, None, ctx.positions, ctx.row_seq,
                           ctx.seq_slot, cache.page_table, rot[0] if rot else None, r, rows, H, 1, self.pd, True,
                           key_dim=hd, value_dim=rank, interleaved=False, mscale=self.position.mscale)
        return out, None

    def _project(self, out, rows: int, ctx: StepContext, gate=None):
        H = self.H
        values = ctx.alloc((rows, H * self.e))
        ops.head_product(values.unflatten(1, (H, self.e)), out.unflatten(1, (H, self.pd))[:, :, :self.rank],
                         self.w_values, rows)
        return self.o_proj(values, rows, ctx, sink=ctx.take_sink())
