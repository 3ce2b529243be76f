"""Domorax as data: a decoder whose layers each name their kind and sizes.

Token embedding; per layer a block that norms what a branch returns and nothing it reads,
x += m * norm1(mixer(x)) and, where the layer has one, x += m * norm2(ff(x)), the norms RMS norms in
groups (the row in equal consecutive parts, each by its own root mean square) with a gain; after every
layer the stream that goes on is a weighted sum of the embedding's output and of all layers' results so
far (the layer's own numbers 'dwa'). The mixer is one of three: an attention through latents
(parts/latent_attention.py: a rotated key part shared by the heads, YaRN-scaled rotation, a window, sinks);
a grouped-query attention whose q and k pass a short convolution and a per-head norm, whose values are the
keys, and whose scores fall with the distance by a slope a head (options of parts/attention.py); a gated
delta rule (parts/delta_rule.py). The feed-forward is dense with a PolyNorm activation, or routed: the `top`
experts by the router's logits, weighted by the softmax over the chosen logits alone, plus a shared expert
behind a sigmoid gate. Final grouped norm, then the output matrix.

Tensor names: 'embed', 'final.norm', 'head', and per layer i 'l<i>.norm1', 'l<i>.norm2', 'l<i>.dwa',
'l<i>.mix.*' (latent: dq, dq.norm, uq, dkv, dkv.norm, uk, uv, sink, o; attention: q, k, q.conv, k.conv, q.norm,
k.norm, o; delta: q, k, v, q.conv, k.conv, v.conv, b, a, A_log, dt_bias, g, norm, o) and 'l<i>.mlp.*' (dense: up,
down, act; routed: router, e<j>.{gate,up,down}, shared.{gate,up,down,sg}).
"""
from __future__ import annotations

from ..config.domorax import DomoraxConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from ..registry import register_architecture

# positions are exact in the fp32 angles up to 2^24; the configuration names no bound of its own
_MAX_POSITIONS = 1 << 22
# the distance slopes of the convolved attention: slope_h = 2^(-8 (h + 1) / H)
_SLOPE_SPAN = 8.0


def _mixer(cfg: DomoraxConfig, kind: str, m) -> PartSpec:
    if kind == "latent_attention":
        position = PartSpec("none")
        if m.rot_dim:
            rot = {"head_dim": m.rot_dim + m.kv_rank, "rotary_dim": m.rot_dim, "theta": m.rot_base}
            if m.rot_scaling:
                rot["scaling"] = {"kind": "yarn", **m.rot_scaling}
            position = PartSpec("rotary", rot)
        return PartSpec("latent_attention", {
            "hidden_size": cfg.width, "num_heads": m.heads, "head_dim": m.dim, "rotary_dim": m.rot_dim, "value_dim": m.vdim,
            "kv_rank": m.kv_rank, "q_rank": m.q_rank, "scale": m.scale, "window": m.window, "sinks": True,
            "eps": cfg.norm_eps, "position": position,
            "names": {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk",
                      "uv": "uv", "sinks": "sink", "o": "o"}})
    if kind == "attention":
        return PartSpec("attention", {
            "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
            "value_dim": m.vdim, "scale": m.scale, "conv_taps": m.conv, "values": "keys", "qk_norm": "head",
            "qk_norm_eps": cfg.norm_eps, "distance_slope_span": _SLOPE_SPAN,
            "names": {"q": "q", "k": "k", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm", "q_conv": "q.conv",
                      "k_conv": "k.conv"}})
    return PartSpec("gated_delta", {
        "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim, "value_dim": m.vdim,
        "conv_taps": m.conv, "eps": cfg.norm_eps,
        "names": {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "b": "b",
                  "a": "a", "A_log": "A_log", "dt_bias": "dt_bias", "g": "g", "norm": "norm", "o": "o"}})


def _feed_forward(cfg: DomoraxConfig, mlp) -> PartSpec:
    gated = {"gate": "gate", "up": "up", "down": "down"}
    if mlp.kind == "dense":
        return PartSpec("dense_mlp", {"hidden_size": cfg.width, "intermediate_size": mlp.ff, "activation": "polynorm",
                                      "eps": cfg.norm_eps, "names": {"up": "up", "down": "down", "act": "act"}})
    params = {"hidden_size": cfg.width, "intermediate_size": mlp.ff, "experts": mlp.experts, "top": mlp.top,
              "correction": False, "normalize": True, "names": {"router": "router", "expert": "e{e}.", **gated}}
    if mlp.shared_ff:
        params["shared"] = {"name": "shared", "gate": "sg", "feed_forward": PartSpec("gated_mlp", {
            "hidden_size": cfg.width, "intermediate_size": mlp.shared_ff, "activation": "silu", "names": gated})}
    return PartSpec("routed_experts", params)


def domorax_spec(cfg: DomoraxConfig) -> ModelSpec:
    norm = PartSpec("group_rmsnorm", {"size": cfg.width, "groups": cfg.norm_groups, "eps": cfg.norm_eps,
                                      "names": {"weight": ""}})
    layers = []
    for l, layer in enumerate(cfg.layers):
        params = {"mixer_norm": norm, "mixer": _mixer(cfg, layer.type, layer.mixer), "residual_scale": cfg.residual_mult,
                  "names": {"mixer_norm": "norm1", "mixer": "mix", "feed_forward_norm": "norm2", "feed_forward": "mlp"}}
        if layer.mlp is not None:
            params["feed_forward_norm"] = norm
            params["feed_forward"] = _feed_forward(cfg, layer.mlp)
        layers.append(LayerSpec(f"l{l}.", PartSpec("post_norm", params)))
    return ModelSpec(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "names": {"weight": ""}}),
        embedding_prefix="embed.",
        layers=layers,
        schedule=[ScheduleEntry(l) for l in range(len(layers))],
        final_norm=norm,
        final_norm_prefix="final.norm.",
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "names": {"weight": ""}}),
        head_prefix="head.",
        max_positions=_MAX_POSITIONS,
        depth_mix=[f"l{l}.dwa" for l in range(len(layers))],
    )


register_architecture("Domorax", DomoraxConfig, domorax_spec)
