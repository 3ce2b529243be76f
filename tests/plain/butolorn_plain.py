"""A plain, slow Butolorn in float64 torch on the CPU, one function per mechanism, written from
the design's equations and sharing nothing with the library. It reads config.json with `json`
and model.safetensors with the safetensors package.

Notation: x the residual stream [T, D]; p the position of a token in its sequence (from 0).
Attention: H query heads, G key/value heads, key width d, value width e, r rotated dims.
Matrix memory: H heads, a memory S [d, e], a key sum n [d] and a running maximum m per head.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


def read_model(folder: str):
    """(config dict, {name: float64 tensor})."""
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    w = {k: (v.to(F64) if v.is_floating_point() else v) for k, v in
         load_file(os.path.join(folder, "model.safetensors")).items()}
    return cfg, w


# ---- small functions -------------------------------------------------------------

def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def relu_squared(z):
    return torch.clamp(z, min=0.0) ** 2


def log_sigmoid(z):
    return -torch.logaddexp(-z, torch.zeros_like(z))


# ---- rotation ---------------------------------------------------------------------

def rotate(x, positions, r: int, base: float, interleaved: bool):
    """x [T, heads, d]; the first r dims of every head turn by p * base^(-2i/r), pair i being
    dims (2i, 2i+1) when interleaved and (i, i + r/2) otherwise; the other dims stay."""
    out = x.clone()
    for i in range(r // 2):
        a, b = (2 * i, 2 * i + 1) if interleaved else (i, i + r // 2)
        freq = base ** (-2.0 * i / r)
        for t, p in enumerate(positions):
            c, s = math.cos(p * freq), math.sin(p * freq)
            out[t, :, a] = x[t, :, a] * c - x[t, :, b] * s
            out[t, :, b] = x[t, :, b] * c + x[t, :, a] * s
    return out


# ---- attention ---------------------------------------------------------------------

def softmax_attention(q, k, v, scale, first_pos: int, one_more: bool):
    """q [T, d] at positions first_pos.., k [S, d], v [S, e] at positions 0..: causal. With
    one_more the denominator holds one more than the keys' exponentials."""
    T = q.shape[0]
    out = torch.zeros((T, v.shape[1]), dtype=F64)
    for t in range(T):
        last = first_pos + t
        s = (k[:last + 1] @ q[t]) * scale
        top = max(s.max().item(), 0.0) if one_more else s.max().item()
        e = torch.exp(s - top)
        den = e.sum() + (math.exp(-top) if one_more else 0.0)
        out[t] = (e / den) @ v[:last + 1]
    return out


def attention_mixer(h, w, pre, m, eps, side: bool, carry=None):
    """h [T, D] -> [T, D]; carry = (k [S, G, d], v [S, G, e]) of the tokens before. side: the
    attention that stands beside a matrix memory (no biases, q and k normed over the whole
    projection, interleaved rotation, one more in the denominator, a gate on the heads' outputs);
    otherwise the attention that stands alone (biases, half-split rotation)."""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ w[pre + "q"].T, h @ w[pre + "k"].T, h @ w[pre + "v"].T
    if side:
        q = rms(q, eps) * w[pre + "q.norm"]
        k = rms(k, eps) * w[pre + "k.norm"]
    else:
        q, k, v = q + w[pre + "q.b"], k + w[pre + "k.b"], v + w[pre + "v.b"]
    q, k, v = q.reshape(T, H, d), k.reshape(T, G, d), v.reshape(T, G, e)
    first = 0 if carry is None else carry[0].shape[0]
    rot = m.get("rot")
    if rot:
        positions = range(first, first + T)
        q = rotate(q, positions, rot["dims"], rot["base"], side)
        k = rotate(k, positions, rot["dims"], rot["base"], side)
    if carry is not None:
        k, v = torch.cat([carry[0], k]), torch.cat([carry[1], v])
    heads = [softmax_attention(q[:, a], k[:, a // (H // G)], v[:, a // (H // G)], m["scale"], first, side)
             for a in range(H)]
    y = torch.cat(heads, -1)
    if side:
        y = y * torch.sigmoid(h @ w[pre + "g"].T)
    return y @ w[pre + "o"].T, (k, v)


# ---- matrix memory -----------------------------------------------------------------

def bounded(z, cap: float):
    return cap * torch.tanh(z / cap)


def memory_scan(q, k, v, log_in, log_keep, state=None):
    """q, k [T, H, d] (q already scaled), v [T, H, e], the logarithms of the two gates [T, H];
    state (S [H, d, e], n [H, d], m [H]) or None for zeros. Returns (y [T, H, e], state)."""
    T, H, d = q.shape
    e = v.shape[2]
    if state is None:
        state = (torch.zeros((H, d, e), dtype=F64), torch.zeros((H, d), dtype=F64), torch.zeros(H, dtype=F64))
    S, n, m = (s.clone() for s in state)
    y = torch.zeros((T, H, e), dtype=F64)
    for t in range(T):
        for a in range(H):
            top = max(log_keep[t, a].item() + m[a].item(), log_in[t, a].item())
            keep = math.exp(log_keep[t, a].item() + m[a].item() - top)
            take = math.exp(log_in[t, a].item() - top)
            S[a] = keep * S[a] + take * torch.outer(k[t, a], v[t, a])
            n[a] = keep * n[a] + take * k[t, a]
            m[a] = top
            y[t, a] = (S[a].T @ q[t, a]) / (max(abs(torch.dot(n[a], q[t, a]).item()), math.exp(-top)) + 1e-6)
    return y, (S, n, m)


def memory_mixer(h, w, pre, m, eps, carry=None):
    """h [T, D] -> [T, D]; carry = the memory's state of the tokens before."""
    T = h.shape[0]
    H, d, e, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[pre + "q"].T).reshape(T, H, d) * d ** -0.5
    k = (h @ w[pre + "k"].T).reshape(T, H, d)
    v = (h @ w[pre + "v"].T).reshape(T, H, e)
    log_in = bounded(h @ w[pre + "i"].T + w[pre + "i.b"], cap)
    log_keep = log_sigmoid(bounded(h @ w[pre + "f"].T + w[pre + "f.b"], cap))
    y, state = memory_scan(q, k, v, log_in, log_keep, carry)
    y = rms(y, eps).reshape(T, H * e) * w[pre + "norm"] * torch.sigmoid(h @ w[pre + "g"].T)
    return y @ w[pre + "o"].T, state


def side_by_side(h, w, pre, m, eps, carry=None):
    left, c_left = attention_mixer(h, w, pre + "left.", m["left"], eps, True, None if carry is None else carry[0])
    right, c_right = memory_mixer(h, w, pre + "right.", m["right"], eps, None if carry is None else carry[1])
    return m["left_scale"] * left + m["right_scale"] * right, (c_left, c_right)


# ---- feed-forward and token input --------------------------------------------------

def dense_ff(h, w, pre):
    return relu_squared(h @ w[pre + "up"].T) @ w[pre + "down"].T


def token_input(x, tokens, w, pre, layer: int, dim: int, eps):
    """What layer `layer` adds for its tokens: its `dim` columns of the second table, gated by the stream."""
    e = w["side.embed"][torch.tensor(tokens)][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ w[pre + "gate"].T) * e) @ w[pre + "proj"].T
    return rms(y, eps) * w[pre + "norm"]


# ---- the model -----------------------------------------------------------------------

def order_of_runs(cfg):
    """[(layer, the embedding is added again before it)] in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    runs = [(l, False) for l in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(l, t > 0 and l == loop["start"]) for l in range(loop["start"], loop["stop"])]
    return runs + [(l, False) for l in range(loop["stop"], n)]


def forward(cfg, w, tokens, carry=None, layers_out=None):
    """Logits [T, vocab] of `tokens` that continue the sequence `carry` describes (None: its
    start), and the new carry: one entry for every run of a layer."""
    eps = cfg["norm"]["eps"]
    side = (cfg.get("token_side") or {}).get("dim", 0)
    runs = order_of_runs(cfg)
    x0 = w["embed"][torch.tensor(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    x = x0.clone()
    new_carry = []
    for j, (l, again) in enumerate(runs):
        if again:
            x = x + x0
        layer, pre = cfg["layers"][l], f"l{l}."
        h = rms(x, eps) * w[pre + "norm1"]
        c = None if carry is None else carry[j]
        if layer["type"] == "attention":
            y, c = attention_mixer(h, w, pre + "mix.", layer["mixer"], eps, False, c)
        else:
            y, c = side_by_side(h, w, pre + "mix.", layer["mixer"], eps, c)
        new_carry.append(c)
        x = x + rms(y, eps) * w[pre + "norm1b"]
        if layer.get("mlp") is not None:
            y = dense_ff(rms(x, eps) * w[pre + "norm2"], w, pre + "mlp.")
            x = x + rms(y, eps) * w[pre + "norm2b"]
        if side:
            x = x + token_input(x, tokens, w, pre + "side.", l, side, eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return (rms(x, eps) * w["final.norm"]) @ w["embed"].T, new_carry


def greedy(cfg, w, prompt, steps: int) -> list[int]:
    """`steps` tokens after `prompt`, each the argmax of the last logits (lowest id on ties)."""
    logits, carry = forward(cfg, w, list(prompt))
    out = []
    for _ in range(steps):
        out.append(int(torch.argmax(logits[-1]).item()))
        logits, carry = forward(cfg, w, [out[-1]], carry)
    return out
