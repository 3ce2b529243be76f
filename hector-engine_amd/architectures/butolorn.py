"""Butolorn as data: a decoder whose layers each name their kind and sizes.

Token embedding times a constant; per layer a block with norms on both sides of each branch,
x += norm1b(mixer(norm1(x))) and, where the layer has one, x += norm2b(ff(norm2(x))), all RMS norms
with a gain; then a token input, x += rms(proj(gelu_tanh(gate x) * e)) * gain with e the layer's
stretch of the token's row of a second embedding table. The mixer is either a grouped-query
attention with biases and a half-split partial rotation, or two mixers side by side on the same
input, weighted and summed: an attention without biases whose q and k are RMS-normed over the whole
projection, with an interleaved partial rotation, one more in the softmax's denominator and an
element-wise sigmoid gate on its heads' outputs; and a matrix memory carried from token to token
(parts/matrix_memory.py). The feed-forward is dense with the square of relu. A stretch of layers
may run several times in a row with the same weights, each pass with a cache and state of its own,
the embedding's output added again before every pass but the first. Final RMS norm, then the
embedding matrix once more as the output matrix.

Tensor names: 'embed', 'side.embed', 'final.norm', and per layer i 'l<i>.norm1', 'l<i>.norm1b',
'l<i>.norm2', 'l<i>.norm2b', 'l<i>.mix.{q,k,v,o}' (+ '.b') or 'l<i>.mix.left.{q,k,v,g,o,q.norm,k.norm}'
with 'l<i>.mix.right.{q,k,v,g,o,norm,i,i.b,f,f.b}', 'l<i>.mlp.{up,down}', 'l<i>.side.{gate,proj,norm}'.
"""
from __future__ import annotations

from ..config.butolorn import ButolornAttention, ButolornConfig
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from ..registry import register_architecture

# positions are exact in the fp32 angles up to 2^24; the configuration names no bound of its own
_MAX_POSITIONS = 1 << 22


def _attention(cfg: ButolornConfig, a: ButolornAttention, side_by_side: bool) -> PartSpec:
    position = PartSpec("none")
    if a.rot_dims:
        position = PartSpec("rotary", {"head_dim": a.dim, "rotary_dim": a.rot_dims, "theta": a.rot_base,
                                       "interleaved": side_by_side})
    params = {"hidden_size": cfg.width, "num_heads": a.heads, "num_kv_heads": a.kv_heads, "head_dim": a.dim,
              "value_dim": a.vdim, "scale": a.scale, "out_bias": False, "position": position}
    if side_by_side:
        params.update({"qkv_bias": False, "qk_norm": "projection", "qk_norm_eps": cfg.norm_eps, "sink_value": 0.0,
                       "out_gate": True,
                       "names": {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g", "q_norm": "q.norm",
                                 "k_norm": "k.norm"}})
    else:
        params.update({"qkv_bias": True,
                       "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b",
                                 "v_bias": "v.b"}})
    return PartSpec("attention", params)


def butolorn_spec(cfg: ButolornConfig) -> ModelSpec:
    norm = PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.norm_eps, "names": {"weight": ""}})
    layers = []
    for l, layer in enumerate(cfg.layers):
        m = layer.mixer
        if layer.type == "attention":
            mixer = _attention(cfg, m, False)
        else:
            r = m.right
            memory = PartSpec("mlstm", {
                "hidden_size": cfg.width, "num_heads": r.heads, "head_dim": r.dim, "value_dim": r.vdim,
                "gate_cap": r.gate_cap, "eps": cfg.norm_eps,
                "names": {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "i": "i", "f": "f",
                          "i_bias": "i.b", "f_bias": "f.b"}})
            mixer = PartSpec("parallel", {"branches": [
                {"name": "left", "scale": m.left_scale, "mixer": _attention(cfg, m.left, True)},
                {"name": "right", "scale": m.right_scale, "mixer": memory}]})
        params = {"mixer_norm": norm, "mixer_post_norm": norm, "mixer": mixer,
                  "names": {"mixer_norm": "norm1", "mixer_post_norm": "norm1b", "mixer": "mix",
                            "feed_forward_norm": "norm2", "feed_forward_post_norm": "norm2b", "feed_forward": "mlp",
                            "token_input": "side"}}
        if layer.mlp is not None:
            params["feed_forward_norm"] = params["feed_forward_post_norm"] = norm
            params["feed_forward"] = PartSpec("dense_mlp", {
                "hidden_size": cfg.width, "intermediate_size": layer.mlp.ff, "activation": "relu2",
                "names": {"up": "up", "down": "down"}})
        if cfg.side_dim:
            params["token_input"] = PartSpec("gated_token_input", {
                "hidden_size": cfg.width, "vocab_size": cfg.vocab, "dim": cfg.side_dim, "offset": l * cfg.side_dim,
                "table_width": len(cfg.layers) * cfg.side_dim, "table": "side.embed", "eps": cfg.norm_eps,
                "activation": "gelu_tanh", "names": {"gate": "gate", "proj": "proj", "norm": "norm"}})
        layers.append(LayerSpec(f"l{l}.", PartSpec("sandwich_norm", params)))
    return ModelSpec(
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "hidden_size": cfg.width,
                                               "scale": cfg.embedding_scale, "names": {"weight": ""}}),
        embedding_prefix="embed.",
        layers=layers,
        schedule=[ScheduleEntry(l, add_embedding=again) for l, again in cfg.runs()],
        final_norm=norm,
        final_norm_prefix="final.norm.",
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "hidden_size": cfg.width, "tied_to": "embed"}),
        head_prefix="head.",
        max_positions=_MAX_POSITIONS,
    )


register_architecture("Butolorn", ButolornConfig, butolorn_spec)
