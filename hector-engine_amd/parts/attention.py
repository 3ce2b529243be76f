"""Grouped-query attention over the paged cache.

q = n Wq^T + bq, k = n Wk^T + bk, v = n Wv^T + bv (one product over q||k||v, the
reference's optional fusion: src/graph_builder.cpp:1543-1670); q and k are
encoded by the position part after the bias and before the cache write, v is
not (src/graph_builder.cpp:1213-1326); the new keys and values are written
before attention so that a query sees its own key (:1318-1326); the query at
position p attends the keys (p - window, p], all of [0, p] without a window
(kernels/attention.cu:60, :196, :696); kv head = h // (H / KVH) (:180);
scale 1/sqrt(head_dim) (src/graph_builder.cpp:1328); then o = a Wo^T.

Options of the same part, each off unless its parameter says otherwise:
  value_dim   the values of a head are that wide (the keys stay head_dim wide). Keys, values and
              the rotated q then live in heads of one padded size (the wider of the two, in steps
              of 16 where the MFMA kernels run): the padding is zeros, the output matrix gets zero
              columns for it, and every attention kernel sees one head size.
  scale       the factor on q . k (default 1/sqrt(head_dim)).
  chunk       position i sees j <= i only when floor(i / chunk) = floor(j / chunk); chunks are
              counted from position 0 of the sequence.
  sinks       a stored number per head joins the softmax's denominator as exp(sink_h); it has no
              key and no value, is not scaled and counts once.
  sink_value  a constant in place of the stored sinks: every head's softmax has exp(sink_value) more in its
              denominator (0.0: one is added), and no tensor is read.
  head_gate   head h's output is multiplied by sigmoid(g_h), g = Wg n with one row of Wg a head;
              the rows of Wg ride behind q||k||v in the one product.
  out_gate    the concatenated heads are multiplied element by element by sigmoid(Wg n), Wg with a row for
              every value of every head (tensor `gate`); its rows ride behind q||k||v likewise.
  qk_norm     "projection": q (all heads' rows of a token at once) is divided by its root mean square
              (eps `qk_norm_eps`) and multiplied by a stored vector of that size, k likewise; after the
              bias and before the position encoding. "head": every head of q is divided by its own root
              mean square and multiplied by one stored vector of head_dim that all heads share, every
              head of k likewise with a second vector.
  conv_taps   K > 0: q and k pass a causal convolution per channel over the last K projected rows of the
              sequence (tensors `q_conv`, `k_conv`, [channels, K], the last column on the row's own
              input, zeros before the sequence's start, no bias), directly behind the projection and
              before the norm; the sequence carries the last K - 1 projected rows in its state.
  values      "keys": there is no value projection; a kv head's value is its key as it stands before
              the q/k norm (behind the convolution). value_dim must equal head_dim.
  distance_slope_span  s > 0: the score of key j for the query at position i loses slope_h * (i - j), with
              slope_h = 2^(-s (h + 1) / H) for head h.
  q_temp      {coef, every}: the q of position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1).
  score_maps  2: differential attention. A head has two queries and a kv head two keys (in the q and k
              matrices a head's rows for map 1 stand in front of its rows for map 2); the two maps are
              separate softmax attentions that share the head's values, with results a1 and a2, and the head's output is
              rms(a1 - lambda * a2) * (1 - diff) over its value_dim values (no gain, eps `diff_eps`), with
              lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff from four stored vectors of head_dim and the
              constant `diff`. The kernels see 2 H heads over 2 KVH kv heads: the rows of q are reordered
              so that the heads of one (kv head, map) are neighbours, and the value rows of a kv head
              stand once for each of its maps; ops.diff_heads then joins the pairs.
  names       the suffixes of its tensors (q, k, v, o, q_bias, k_bias, v_bias, o_bias, sinks, gate,
              lq1, lk1, lq2, lk2, q_norm, k_norm, q_conv, k_conv).
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch

from ..kernels import kv_layout, ops, routes
from .base import (BuildEnv, KVNeed, LayerCache, Mixer, PartSpec, PieceRows, StepContext, TensorSpec,
                   build_part, param, register_part, tensor_name)

_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
          "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias", "o_bias": "o_proj.bias",
          "sinks": "sinks", "gate": "gate.weight", "lq1": "lambda_q1", "lk1": "lambda_k1", "lq2": "lambda_q2",
          "lk2": "lambda_k2", "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", "q_conv": "q_conv.weight", "k_conv": "k_conv.weight"}
from .linear import Linear


@dataclass(frozen=True)
class AttentionCase:
    """What a route of "attention" decides by."""
    all_single: bool    # every sequence of the step brings one token
    fast: bool          # sizes and environment allow the MFMA kernels
    fusable: bool       # head size and position encoding are ones the fused one-token kernel takes


def keys_uneven(lengths: list[int], before=None) -> bool:
    """Whether one sequence of a one-token step has several times the keys of the others (and
    thousands of them): the one-token attention then cuts every sequence's keys across more
    workgroups, or the long sequence would be left to a few of them. Once up (`before`), the flag
    stays up until the longest sequence has fewer than three times the mean (four to raise it), so
    that a batch at the edge does not go back and forth between two graphs."""
    longest = max(lengths)
    return longest >= 4096 and longest * len(lengths) >= (3 if before else 4) * sum(lengths)


@register_part("mixer", "attention")
class Attention(Mixer):
    accepts_normed_rows = True
    step_hint = staticmethod(keys_uneven)

    def __init__(self, params: dict, prefix: str, env: BuildEnv):
        super().__init__(prefix, env)
        self.hidden = param(params, "hidden_size", int)
        self.H = param(params, "num_heads", int)
        self.KVH = param(params, "num_kv_heads", int)
        self.hd = param(params, "head_dim", int)
        self.qkv_bias = param(params, "qkv_bias", bool, False)
        self.out_bias = param(params, "out_bias", bool, False)
        self.window = param(params, "window", int, 0)
        self.kv_projection = param(params, "kv_projection", bool, True)
        self.scale = param(params, "scale", float, 1.0 / math.sqrt(self.hd))
        self.vd = param(params, "value_dim", int, self.hd)
        self.chunk = param(params, "chunk", int, 0)
        self.has_sinks = param(params, "sinks", bool, False)
        self.head_gate = param(params, "head_gate", bool, False)
        self.out_gate = param(params, "out_gate", bool, False)
        self.sink_value = param(params, "sink_value", float, None)
        self.qk_norm = param(params, "qk_norm", str, "")
        self.qk_norm_eps = param(params, "qk_norm_eps", float, 1e-6)
        self.q_norm_w = self.k_norm_w = None
        self.conv_taps = param(params, "conv_taps", int, 0)
        self.values_are_keys = param(params, "values", str, "projection") == "keys"
        self.slope_span = param(params, "distance_slope_span", float, 0.0)
        self.slopes: torch.Tensor | None = None
        self.taps = None
        self.maps = param(params, "score_maps", int, 1)
        self.diff = param(params, "diff", float, 0.0)
        self.diff_eps = param(params, "diff_eps", float, 1e-6)
        self.lam = 0.0                      # lambda of a differential attention, from its four vectors (bind)
        qt = param(params, "q_temp", dict, None)
        self.q_temp = None if not qt else (float(qt["coef"]), int(qt["every"]))
        if self.maps not in (1, 2) or (self.maps == 2 and (self.head_gate or self.out_gate or self.qk_norm)):
            raise ValueError(f"attention: score_maps {self.maps} must be 1 or 2 (and 2 goes without gates and q/k norms)")
        if self.head_gate and self.out_gate:
            raise ValueError("attention: head_gate and out_gate exclude each other")
        if self.qk_norm not in ("", "projection", "head"):
            raise ValueError(f"attention: unknown qk_norm '{self.qk_norm}'")
        if param(params, "values", str, "projection") not in ("projection", "keys"):
            raise ValueError(f"attention: unknown values '{params['values']}'")
        if self.conv_taps < 0 or self.slope_span < 0:
            raise ValueError("attention: conv_taps and distance_slope_span must not be negative")
        if (self.conv_taps or self.values_are_keys) and (self.qkv_bias or self.maps > 1 or self.head_gate or self.out_gate
                                                         or not self.kv_projection):
            raise ValueError("attention: conv_taps and values 'keys' go without biases, gates, score maps and shared caches")
        if self.values_are_keys and self.vd != self.hd:
            raise ValueError(f"attention: values that are the keys are head_dim {self.hd} wide, not {self.vd}")
        if self.has_sinks and self.sink_value is not None:
            raise ValueError("attention: stored sinks and sink_value exclude each other")
        if self.q_temp is not None and self.q_temp[1] <= 0:
            raise ValueError(f"attention: q_temp.every {self.q_temp[1]} must be positive")
        # the heads as the kernels count them: a differential head is two, one a score map
        self.Hk, self.KVHk = self.H * self.maps, self.KVH * self.maps
        names = param(params, "names", dict, {})
        self._names = {k: tensor_name(prefix, names, k, d) for k, d in _NAMES.items()}
        if self.H % self.KVH:
            raise ValueError(f"attention: {self.H} heads are not a multiple of {self.KVH} kv heads")
        if self.vd <= 0 or self.chunk < 0:
            raise ValueError(f"attention: value_dim {self.vd} must be positive, chunk {self.chunk} not negative")
        # the one head size of the cache pages, of the rotated q and of the attention's output
        self.pd = max(self.hd, self.vd)
        mfma = env.dtype == torch.bfloat16 and getattr(env, "fast_kernels", True)
        if mfma and (self.hd != self.vd or self.pd % 16) and self.pd <= 256:
            self.pd = (self.pd + 15) // 16 * 16
        self.sinks: torch.Tensor | None = None
        self.position = build_part("position", param(params, "position", PartSpec, PartSpec("none")),
                                   prefix, env)
        self.qkv: Linear | None = None
        self.q_only: Linear | None = None
        self.o_proj: Linear | None = None
        self._chosen: dict[tuple, routes.Route] = {}      # (all one-token, dtype) -> route, for one version of the table
        self._chosen_version = -1
        self.fast = mfma and self.pd % 16 == 0 and self.pd <= 256 and self.scale > 0   # else the plain kernel
        # what the fused one-token kernel and the kernels without these options do not take
        self.extras = self.chunk > 0 or self.has_sinks or self.head_gate or self.maps > 1 or self.q_temp is not None \
            or self.out_gate or self.sink_value is not None or bool(self.qk_norm) or self.conv_taps > 0 \
            or self.values_are_keys or self.slope_span > 0
        # rows of the gate's matrix behind q||k||v: one a head, or one for every value of every head
        self.gate_rows = self.H if self.head_gate else self.H * self.vd if self.out_gate else 0

    def children(self):
        return [self.position]

    def state_bytes(self) -> int:
        # the last K - 1 projected q and k rows of the sequence, fp32
        return 4 * (self.conv_taps - 1) * (self.Hk + self.KVHk) * self.hd if self.conv_taps > 1 else 0

    def kv_need(self):
        # pages in the order the attention kernels read their operands
        return KVNeed(self.KVHk, self.pd, self.window, k_page_elems=kv_layout.k_page_elems(self.pd),
                      v_page_elems=kv_layout.v_page_elems(self.pd), chunk=self.chunk)

    def tensor_specs(self):
        n, hd, vd = self._names, self.hd, self.vd
        specs = {n["q"]: TensorSpec((self.Hk * hd, self.hidden)),
                 n["o"]: TensorSpec((self.hidden, self.H * vd))}
        if self.kv_projection:
            specs[n["k"]] = TensorSpec((self.KVHk * hd, self.hidden))
            if not self.values_are_keys:
                specs[n["v"]] = TensorSpec((self.KVH * vd, self.hidden))
        if self.conv_taps:
            specs[n["q_conv"]] = TensorSpec((self.H * hd, self.conv_taps), ("normal", 0.4))
            specs[n["k_conv"]] = TensorSpec((self.KVH * hd, self.conv_taps), ("normal", 0.4))
        if self.qkv_bias:
            specs[n["q_bias"]] = TensorSpec((self.Hk * hd,))
            if self.kv_projection:
                specs[n["k_bias"]] = TensorSpec((self.KVHk * hd,))
                specs[n["v_bias"]] = TensorSpec((self.KVH * vd,))
        if self.maps == 2:
            for key in ("lq1", "lk1", "lq2", "lk2"):
                specs[n[key]] = TensorSpec((hd,), ("normal", 0.1))
        if self.out_bias:
            specs[n["o_bias"]] = TensorSpec((self.hidden,))
        if self.has_sinks:
            specs[n["sinks"]] = TensorSpec((self.H,), ("normal", 1.0))
        if self.gate_rows:
            specs[n["gate"]] = TensorSpec((self.gate_rows, self.hidden))
        if self.qk_norm:
            per_head = self.qk_norm == "head"
            specs[n["q_norm"]] = TensorSpec((hd if per_head else self.H * hd,), ("gain", 1.0, 0.1))
            if self.kv_projection:
                specs[n["k_norm"]] = TensorSpec((hd if per_head else self.KVH * hd,), ("gain", 1.0, 0.1))
        specs.update(self.position.tensor_specs())
        return specs

    def bind(self, tensors):
        p, n = self.prefix, self._names
        names = ["q"] + ((["k"] if self.values_are_keys else ["k", "v"]) if self.kv_projection else [])
        ws = [self._by_map(x, tensors.pop(n[x])) for x in names]
        gate_w = tensors.pop(n["gate"]) if self.gate_rows else None
        if gate_w is not None:
            ws.append(gate_w)          # the gate's rows ride behind q||k||v: one product
            spare = -sum(w.shape[0] for w in ws) % 8
            if spare:                  # rows of zeros, so that the product's rows stay a multiple of 8 wide
                ws.append(torch.zeros((spare, gate_w.shape[1]), dtype=gate_w.dtype, device=gate_w.device))
        if len({w.dtype for w in ws}) != 1:
            raise TypeError(f"{p}q/k/v projections are stored in different dtypes")
        w = torch.cat(ws, 0).contiguous() if len(ws) > 1 else ws[0]
        b = None
        if self.qkv_bias:
            bs = [self._by_map(x, tensors.pop(n[x + "_bias"])) for x in names]
            if len({x.dtype for x in bs}) != 1:
                raise TypeError(f"{p}q/k/v biases are stored in different dtypes")
            b = torch.cat(bs, 0).contiguous() if len(bs) > 1 else bs[0]
        def bias_for(bias, rows):
            """The bias, with zeros for the rows behind q||k||v (the gates and the spare rows)."""
            if bias is None or bias.numel() == rows:
                return bias
            return torch.cat([bias, torch.zeros(rows - bias.numel(), dtype=bias.dtype, device=bias.device)])

        self.qkv = Linear(w, bias_for(b, w.shape[0]))
        q_rows = self.Hk * self.hd
        if gate_w is not None and self.kv_projection:
            spare = -(q_rows + self.gate_rows) % 8
            self.q_only = Linear(torch.cat([ws[0], gate_w, torch.zeros((spare, gate_w.shape[1]), dtype=gate_w.dtype,
                                                                       device=gate_w.device)], 0).contiguous(),
                                 None if b is None else bias_for(b[:q_rows], q_rows + self.gate_rows + spare))
        else:
            self.q_only = Linear(w if gate_w is not None else w[:q_rows],
                                 None if b is None else bias_for(b[:q_rows], w.shape[0] if gate_w is not None else q_rows))
        del ws
        wo = tensors[n["o"]]
        if self.maps == 2:
            f = lambda key: tensors[n[key]].to(device="cpu", dtype=torch.float32)
            self.lam = float(torch.exp((f("lq1") * f("lk1")).sum()) - torch.exp((f("lq2") * f("lk2")).sum())) + self.diff
        if self.pd != self.vd and self.maps == 1:
            # zero columns where the attention's output holds the padding of a head
            padded = torch.zeros((self.hidden, self.H, self.pd), dtype=wo.dtype, device=wo.device)
            padded[:, :, :self.vd] = wo.view(self.hidden, self.H, self.vd)
            wo = padded.view(self.hidden, self.H * self.pd)
        self.o_proj = Linear(wo, tensors.get(n["o_bias"]))
        if self.has_sinks:
            self.sinks = tensors[n["sinks"]]
        elif self.sink_value is not None:
            self.sinks = torch.full((self.H,), self.sink_value, dtype=torch.float32, device=wo.device)
        if self.qk_norm:
            self.q_norm_w = tensors[n["q_norm"]]
            self.k_norm_w = tensors[n["k_norm"]] if self.kv_projection else None
        if self.conv_taps:
            self.taps = torch.cat([tensors[n["q_conv"]], tensors[n["k_conv"]]], 0).contiguous()
            self._no_state = torch.zeros((1, 16), dtype=torch.uint8, device=wo.device)
        if self.slope_span:
            h = torch.arange(1, self.H + 1, dtype=torch.float64)
            self.slopes = torch.exp2(-self.slope_span * h / self.H).to(torch.float32).to(wo.device)
        self.position.bind(tensors)

    def _by_map(self, which: str, t: torch.Tensor) -> torch.Tensor:
        """A differential attention's stored rows (or bias) as the kernels' heads read them: q from
        [head][map] to [kv head][map][head of the group]; k is stored [kv head][map] already; the
        value rows of a kv head once for each of its two maps."""
        if self.maps == 1 or which == "k":
            return t
        rest = t.shape[1:]
        if which == "q":
            G, R = self.KVH, self.H // self.KVH
            return t.reshape(G, R, 2, self.hd, *rest).transpose(1, 2).reshape(t.shape).contiguous()
        return t.reshape(self.KVH, 1, self.vd, *rest).expand(self.KVH, 2, self.vd, *rest).reshape(
            2 * t.shape[0], *rest).contiguous()

    def _project(self, out, rows: int, ctx: StepContext, gate=None):
        """The output product behind the attention kernels (a differential attention joins its pairs
        of heads first)."""
        if self.maps == 2:
            mixed = ctx.alloc((rows, self.H * self.vd))
            ops.diff_heads(mixed, out, rows, self.H, self.KVH, self.pd, self.vd, self.lam, 1.0 - self.diff,
                           self.diff_eps)
            out = mixed
        if self.out_gate:
            ops.sigmoid_gate(out, gate, rows, self.H, self.pd, self.vd)
        return self.o_proj(out, rows, ctx, sink=ctx.take_sink())

    def forward(self, x, ctx: StepContext, cache: LayerCache):
        if cache.writes and not self.kv_projection:
            raise RuntimeError(f"{self.prefix}: a mixer without k/v projections must read another run's cache")
        if self._chosen_version != routes.version():
            self._chosen.clear()
            self._chosen_version = routes.version()
        key = (ctx.all_single, ctx.env.dtype)
        route = self._chosen.get(key)
        if route is None:
            rot = self.position.rotary()
            case = AttentionCase(
                all_single=ctx.all_single, fast=self.fast,
                fusable=not self.position.custom and rot is not None and not self.extras
                and self.hd == self.vd == self.pd
                and not self.position.interleaved and self.position.mscale == 1.0
                and ops.attention_decode_fused_ok(self.H, self.KVH, self.hd, rot[1]))
            route = self._chosen[key] = routes.choose("attention", (ctx.env.dtype,), case)
        return route.run(self, x, ctx, cache)

    # ---- the routes' bodies ----

    def _run_fused_one_token(self, x, ctx: StepContext, cache: LayerCache):
        """One-token steps: bias, rotation, cache write and attention in one launch."""
        rows, H, KVH, hd = ctx.rows, self.H, self.KVH, self.hd
        proj = self.qkv if cache.writes else self.q_only
        rot = self.position.rotary()
        # where the projection is cut along K (17 to 64 rows), the kernel below adds the slices
        # itself: the same bits, and the launch that would add them is not needed
        qkv = proj.k_slices(x, rows, ctx)
        if qkv is None:
            qkv = proj(x, rows, ctx, use_bias=False)
        pieces = self.o_proj.reads_pieces(rows, ctx)       # the layout the output product reads best
        out = ctx.alloc(ops.pieces_shape(rows, H * hd) if pieces else (rows, H * hd))
        uneven = bool(ctx.hints.get(keys_uneven, False))
        floats = ops.attention_decode_fused_workspace_floats(rows, H, KVH, hd, ctx.max_keys, uneven)
        ws = ctx.alloc((floats,), torch.float32) if floats else None
        # the page numbers of the step's rows, where the host has put them beside the step's metadata
        by_row = ctx.row_tables.get(cache.page_table.data_ptr())
        ops.attention_decode_fused(out, qkv, proj.bias, cache.kpool, cache.vpool, ctx.positions,
                                   ctx.row_seq, None if by_row is not None else ctx.seq_slot,
                                   by_row if by_row is not None else cache.page_table, rot[0], rot[1],
                                   rows, H, KVH, hd, self.window, self.scale, ctx.max_keys,
                                   cache.writes, ws, out_pieces=pieces, spread=uneven)
        return self.o_proj(PieceRows(out) if pieces else out, rows, ctx, sink=ctx.take_sink())

    def _encoded_q(self, x, ctx: StepContext, cache: LayerCache):
        """(q with bias and position encoding, after the new keys and values went into the cache;
        the heads' gates as a view of the projection's rows, or None)."""
        rows, H, KVH, hd = ctx.rows, self.Hk, self.KVHk, self.hd
        writes = cache.writes
        proj = self.qkv if writes else self.q_only
        rot = self.position.rotary()
        # With a rotation (or no encoding) the bias is added inside the fused kernel;
        # any other encoding sees q and k with their bias already added.
        fused_bias = not self.position.custom and not self.qk_norm
        qkv = proj(x, rows, ctx, use_bias=not fused_bias)
        if self.conv_taps or self.values_are_keys:
            qkv = self._conv_norm_rows(qkv, ctx, cache)
        elif self.qk_norm == "head":
            ops.qk_head_norm(qkv, qkv, self.q_norm_w, self.k_norm_w if writes else self.q_norm_w, H, KVH if writes else 0,
                             hd, self.qk_norm_eps, rows)
        elif self.qk_norm:
            # each token's q (all heads at once), and its k, by a root mean square of their own, in place
            wide = qkv.stride(0)
            if writes:
                ops.rmsnorm_row_pair(qkv, self.q_norm_w, H * hd, self.k_norm_w, KVH * hd, H * hd, rows, self.qk_norm_eps)
            else:
                ops.rmsnorm_rows(qkv, qkv, self.q_norm_w, rows, H * hd, wide, wide, self.qk_norm_eps)
        if not fused_bias:
            q_cols, kv_cols = H * hd, KVH * hd
            qv = qkv[:, :q_cols].unflatten(1, (H, hd))
            kv = qkv[:, q_cols:q_cols + kv_cols].unflatten(1, (KVH, hd)) if writes else None
            self.position.apply(qv, kv, ctx)
        q = ctx.alloc((rows, H * self.pd))
        inv_freq, r = rot if rot is not None else (None, 0)
        ops.qkv_rope_cache(q, cache.kpool, cache.vpool, qkv, H * hd, KVH * hd,
                           proj.bias if fused_bias else None, ctx.positions, ctx.row_seq,
                           ctx.seq_slot, cache.page_table, inv_freq, r, rows, H, KVH, self.pd, writes,
                           key_dim=hd, value_dim=self.vd, interleaved=self.position.interleaved,
                           mscale=self.position.mscale, q_temp=self.q_temp)
        gate = None
        if self.gate_rows:
            at = H * hd + (KVH * (hd + self.vd) if writes else 0)
            gate = qkv[:rows, at:at + self.gate_rows]
        return q, gate

    def _conv_norm_rows(self, qk, ctx: StepContext, cache: LayerCache):
        """The rows [q | k | v] the cache-write kernel reads, from the projected [q | k]: the convolution over
        each sequence's rows (with the rows it carries), then the heads' norm; the keys as they leave the
        convolution are the values."""
        rows, H, KVH, hd = ctx.rows, self.H, self.KVH, self.hd
        C = (H + KVH) * hd
        if self.conv_taps:
            if self.conv_taps > 1 and cache.state is None:
                raise RuntimeError(f"{self.prefix}: a convolution over the rows needs its row of the state area")
            conv = ctx.alloc((rows, C))
            state = cache.state if cache.state is not None else self._no_state     # one tap carries nothing
            ops.conv_state(conv, qk[:, :C], self.taps, None, state, ctx.positions, ctx.row_seq, ctx.seq_slot,
                           ctx.seq_start, ctx.cu_seqlens, rows, ctx.num_seqs, ctx.all_single, act=False)
            qk = conv
        if not self.values_are_keys:
            if self.qk_norm == "head":
                ops.qk_head_norm(qk, qk, self.q_norm_w, self.k_norm_w, H, KVH, hd, self.qk_norm_eps, rows)
            elif self.qk_norm:
                raise ValueError(f"{self.prefix}: a convolution goes with the heads' own norm or none")
            return qk
        out = ctx.alloc((rows, C + KVH * hd))
        if self.qk_norm == "head":
            ops.qk_head_norm(out, qk, self.q_norm_w, self.k_norm_w, H, KVH, hd, self.qk_norm_eps, rows, copy_v=True)
        else:
            out[:rows, :C].copy_(qk[:rows, :C])
            out[:rows, C:].copy_(qk[:rows, H * hd:C])
        return out

    def _run_plain(self, x, ctx: StepContext, cache: LayerCache):
        """The plain kernel: one fixed order per (query, head), in the precision of the cache."""
        rows, H, KVH, hd = ctx.rows, self.Hk, self.KVHk, self.pd
        q, gate = self._encoded_q(x, ctx, cache)
        out = ctx.alloc((rows, H * hd))
        floats = ops.attention_plain_workspace_floats(rows, H, hd, ctx.most_keys, self.window, self.chunk)
        ws = ctx.alloc((floats,), torch.float32) if floats else None
        ops.attention_plain(out, q, cache.kpool, cache.vpool, ctx.positions, ctx.row_seq,
                            ctx.seq_slot, cache.page_table, rows, H, KVH, hd, self.window,
                            self.scale, ctx.most_keys, ws, chunk=self.chunk, sinks=self.sinks,
                            gate=gate if self.head_gate else None, slopes=self.slopes)
        return self._project(out, rows, ctx, gate)

    def _run_mfma_one_token(self, x, ctx: StepContext, cache: LayerCache):
        """One-token steps of the head sizes and encodings the fused kernel does not take."""
        rows, H, KVH, hd = ctx.rows, self.Hk, self.KVHk, self.pd
        q, gate = self._encoded_q(x, ctx, cache)
        out = ctx.alloc((rows, H * hd))
        floats = ops.attention_decode_workspace_floats(rows, H, KVH, hd, ctx.max_keys)
        ws = ctx.alloc((max(floats, 1),), torch.float32)
        ops.attention_decode(out, q, cache.kpool, cache.vpool, ctx.positions, ctx.row_seq,
                             ctx.seq_slot, cache.page_table, rows, H, KVH, hd, self.window,
                             self.scale, ctx.max_keys, ws, chunk=self.chunk, sinks=self.sinks,
                             gate=gate if self.head_gate else None, slopes=self.slopes)
        return self._project(out, rows, ctx, gate)

    def _run_mfma_prompt(self, x, ctx: StepContext, cache: LayerCache):
        """Prompt steps and mixed steps."""
        rows, H, KVH, hd = ctx.rows, self.Hk, self.KVHk, self.pd
        q, gate = self._encoded_q(x, ctx, cache)
        out = ctx.alloc((rows, H * hd))
        # few queries against many keys (a continuation of a long sequence): the keys in parts
        most = ctx.most_keys
        if self.window > 0:
            most = min(most, self.window + ctx.max_q_len)
        if self.chunk > 0:
            most = min(most, self.chunk + ctx.max_q_len)
        parts = ops.attention_prefill_parts(ctx.num_seqs, ctx.max_q_len, H, hd, most)
        ws = ctx.alloc((ops.attention_prefill_workspace_floats(rows, H, hd, parts),), torch.float32) \
            if parts > 1 else None
        if ctx.padded:
            # the prompt kernels write the rows of sequences only: padding rows hold zeros (their
            # parts too, whose join then gives zeros), never what the buffer held before
            (ws if ws is not None else out).zero_()
        ops.attention_prefill(out, q, cache.kpool, cache.vpool, ctx.cu_seqlens, ctx.seq_slot,
                              ctx.seq_start, cache.page_table, ctx.num_seqs, ctx.max_q_len,
                              rows, H, KVH, hd, self.window, self.scale, parts=parts, workspace=ws,
                              chunk=self.chunk, sinks=self.sinks, gate=gate if self.head_gate else None,
                              slopes=self.slopes)
        return self._project(out, rows, ctx, gate)


_BF16 = (torch.bfloat16,)
routes.register_route("attention", _BF16, "fused_one_token",
                      lambda c: c.fast and c.all_single and c.fusable, Attention._run_fused_one_token)
routes.register_route("attention", _BF16, "plain", lambda c: not c.fast, Attention._run_plain)
routes.register_route("attention", _BF16, "mfma_one_token", lambda c: c.all_single, Attention._run_mfma_one_token)
routes.register_route("attention", _BF16, "mfma_prompt", lambda c: True, Attention._run_mfma_prompt)
routes.register_route("attention", (torch.float32,), "plain", lambda c: True, Attention._run_plain)
