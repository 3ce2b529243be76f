"""A plain, slow Domorax in float64 torch on the CPU, one function per mechanism, written from the
design's equations and sharing nothing with the library. It reads config.json with `json` and
model.safetensors with the safetensors package.

Notation: x the residual stream [T, D]; p the position of a token in its sequence (from 0); h the
input of a mixer or feed-forward (the stream itself: this design norms what a branch returns, not
what it reads).
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


def group_norm(x, weight, groups: int, eps: float):
    """The last axis in `groups` equal consecutive parts, each divided by its own root mean
    square; the whole times weight."""
    shape = x.shape
    parts = x.reshape(*shape[:-1], groups, shape[-1] // groups)
    return rms(parts, eps).reshape(shape) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.logaddexp(z, torch.zeros_like(z))


def short_conv(u, taps, before=None):
    """u [T, C], taps [C, K]: y[t] = sum over j < K of taps[:, j] * u[t - (K - 1 - j)] (the last column weighs
    the row's own input), with zeros (or the rows of `before`, the K - 1 inputs ahead of u) in front of the sequence."""
    T, C = u.shape
    K = taps.shape[1]
    front = torch.zeros((K - 1, C), dtype=u.dtype) if before is None else before
    padded = torch.cat([front, u], 0)
    y = torch.zeros_like(u)
    for j in range(K):
        y = y + taps[:, j] * padded[j:j + T]
    return y


# ---- rotation ---------------------------------------------------------------------

def rotary_frequencies(r: int, base: float, scaling: dict | None):
    """(frequency of pair i for i < r/2, factor on cos and sin)."""
    f = [base ** (-2.0 * i / r) for i in range(r // 2)]
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns):
        return r * math.log(original / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), r - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate_half(x, positions, r: int, freqs, mult: float):
    """x [T, heads, d]: the first r dims of every head, dim i paired with dim i + r/2, turn by
    p * freqs[i]; cos and sin are multiplied by mult; the other dims stay."""
    out = x.clone()
    for i in range(r // 2):
        a, b = i, i + r // 2
        for t, p in enumerate(positions):
            c, s = math.cos(p * freqs[i]) * mult, math.sin(p * freqs[i]) * mult
            out[t, :, a] = x[t, :, a] * c - x[t, :, b] * s
            out[t, :, b] = x[t, :, b] * c + x[t, :, a] * s
    return out


# ---- mixers -----------------------------------------------------------------------

def latent_attention(h, w, pre, m, eps, positions):
    """Queries and keys/values through latents; every head's key is [its own unrotated part, one
    rotated part shared by all heads]; a window; a learned number per head in the softmax's
    denominator."""
    T = h.shape[0]
    H, d, r, e, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    cq = rms(h @ w[pre + "dq"].T, eps) * w[pre + "dq.norm"]
    q = (cq @ w[pre + "uq"].T).reshape(T, H, d + r)
    down = h @ w[pre + "dkv"].T
    c = rms(down[:, :rank], eps) * w[pre + "dkv.norm"]
    k_rot = down[:, rank:].reshape(T, 1, r)
    k_plain = (c @ w[pre + "uk"].T).reshape(T, H, d)
    v = (c @ w[pre + "uv"].T).reshape(T, H, e)
    rot = m.get("rot") or {}
    dims = rot.get("dims", r)
    freqs, mult = rotary_frequencies(dims, rot["base"], rot.get("scaling")) if dims else ([], 1.0)
    q_rot = rotate_half(q[:, :, d:], positions, dims, freqs, mult)
    k_rot = rotate_half(k_rot, positions, dims, freqs, mult)
    window = (m.get("mask") or {}).get("size", 0)
    out = torch.zeros((T, H, e), dtype=F64)
    for t in range(T):
        first = 0 if not window else max(0, t - window + 1)
        for head in range(H):
            s = (k_plain[first:t + 1, head] @ q[t, head, :d] + k_rot[first:t + 1, 0] @ q_rot[t, head]) * m["scale"]
            sink = w[pre + "sink"][head]
            top = torch.maximum(s.max(), sink)
            p = torch.exp(s - top)
            out[t, head] = (p[:, None] * v[first:t + 1, head]).sum(0) / (p.sum() + torch.exp(sink - top))
    return out.reshape(T, H * e) @ w[pre + "o"].T


def head_slopes(H: int):
    """slope_h = 2^(-8 (h + 1) / H) for head h."""
    return [2.0 ** (-8.0 * (h + 1) / H) for h in range(H)]


def distance_attention(q, k, v, scale, slopes, first_position=0):
    """q [Tq, H, d] at the positions first_position.., k and v [Tk, G, d] at the positions 0..: causal softmax
    attention whose score for key j and the query at position i is (q . k) * scale - slope_h * (i - j)."""
    Tq, H, d = q.shape
    G = k.shape[1]
    out = torch.zeros((Tq, H, v.shape[2]), dtype=F64)
    ahead = torch.arange(k.shape[0], dtype=F64)
    for head in range(H):
        g = head // (H // G)
        for t in range(Tq):
            i = first_position + t
            s = (k[:i + 1, g] @ q[t, head]) * scale - slopes[head] * (i - ahead[:i + 1])
            p = torch.softmax(s, 0)
            out[t, head] = (p[:, None] * v[:i + 1, g]).sum(0)
    return out


def conv_attention(h, w, pre, m, eps):
    """Grouped-query attention whose q and k pass a short convolution and a per-head norm, whose
    values are the keys as they leave the convolution, and whose scores lose slope_h * distance."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    q = short_conv(h @ w[pre + "q"].T, w[pre + "q.conv"]).reshape(T, H, d)
    k = short_conv(h @ w[pre + "k"].T, w[pre + "k.conv"]).reshape(T, G, d)
    v = k
    q = rms(q, eps) * w[pre + "q.norm"]
    k = rms(k, eps) * w[pre + "k.norm"]
    out = distance_attention(q, k, v, m["scale"], head_slopes(H))
    return out.reshape(T, H * d) @ w[pre + "o"].T


def delta_rule(q, k, v, beta, g, S=None):
    """One head. q, k [T, d] (unit vectors, q times d^-1/2), v [T, e], beta and g [T]. Per token:
    S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q. Returns (o [T, e], S)."""
    T, d = q.shape
    e = v.shape[1]
    S = torch.zeros((d, e), dtype=F64) if S is None else S.clone()
    o = torch.zeros((T, e), dtype=F64)
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o, S


def unit(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def delta_mixer(h, w, pre, m, eps):
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ w[pre + "q"].T, w[pre + "q.conv"])).reshape(T, G, d)
    k = silu(short_conv(h @ w[pre + "k"].T, w[pre + "k.conv"])).reshape(T, G, d)
    v = silu(short_conv(h @ w[pre + "v"].T, w[pre + "v.conv"])).reshape(T, H, e)
    q = unit(q) * d ** -0.5
    k = unit(k)
    beta = torch.sigmoid(h @ w[pre + "b"].T)
    g = torch.exp(-torch.exp(w[pre + "A_log"]) * softplus(h @ w[pre + "a"].T + w[pre + "dt_bias"]))
    gate = silu(h @ w[pre + "g"].T).reshape(T, H, e)
    out = torch.zeros((T, H, e), dtype=F64)
    for head in range(H):
        j = head // (H // G)
        o, _ = delta_rule(q[:, j], k[:, j], v[:, head], beta[:, head], g[:, head])
        out[:, head] = rms(o, eps) * w[pre + "norm"] * gate[:, head]
    return out.reshape(T, H * e) @ w[pre + "o"].T


# ---- feed-forwards ----------------------------------------------------------------

def poly_norm(z, numbers, eps):
    a, b, c, e = [float(x) for x in numbers]
    return a * rms(z, eps) + b * rms(z * z, eps) + c * rms(z * z * z, eps) + e


def dense_ff(h, w, pre, eps):
    return poly_norm(h @ w[pre + "up"].T, w[pre + "act"], eps) @ w[pre + "down"].T


def gated_expert(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def routed_ff(h, w, pre, mlp):
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ w[pre + "router"].T
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = torch.topk(z[t], top).indices
        share = torch.softmax(z[t][chosen], 0)
        for s, e in zip(share, chosen.tolist()):
            out[t] = out[t] + s * gated_expert(h[t:t + 1], w, f"{pre}e{e}.")[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ w[pre + "shared.sg"].T) * gated_expert(h, w, pre + "shared.")
    return out


# ---- the model --------------------------------------------------------------------

def forward(cfg, w, tokens, streams=None):
    """Logits [T, vocab] of one sequence from its first token on. streams: a list that receives
    what each layer hands on (after the depth average)."""
    eps, groups, mult = cfg["norm"]["eps"], cfg["norm"]["groups"], cfg["residual_mult"]
    positions = list(range(len(tokens)))
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)]
    kept = [x]
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.mix.", layer["mixer"]
        if layer["type"] == "latent_attention":
            y = latent_attention(x, w, pre, m, eps, positions)
        elif layer["type"] == "attention":
            y = conv_attention(x, w, pre, m, eps)
        elif layer["type"] == "delta":
            y = delta_mixer(x, w, pre, m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + mult * group_norm(y, w[f"l{i}.norm1"], groups, eps)
        mlp = layer.get("mlp")
        if mlp:
            y = dense_ff(x, w, f"l{i}.mlp.", eps) if mlp["kind"] == "dense" else routed_ff(x, w, f"l{i}.mlp.", mlp)
            x = x + mult * group_norm(y, w[f"l{i}.norm2"], groups, eps)
        kept.append(x)
        x = sum(w[f"l{i}.dwa"][j] * kept[j] for j in range(i + 2))
        if streams is not None:
            streams.append(x)
    return group_norm(x, w["final.norm"], groups, eps) @ w["head"].T


def greedy(cfg, w, prompt, new_tokens: int):
    tokens = list(prompt)
    for _ in range(new_tokens):
        tokens.append(int(forward(cfg, w, tokens)[-1].argmax()))
    return tokens[len(prompt):]
