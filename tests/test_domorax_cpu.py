"""Domorax without a GPU: its configuration (round trip, defaults, errors that name the key), the tensors
and states its parts ask for, and the plain implementation against itself (a recurrence carried in
portions, a convolution with carried inputs, the scaled rotation, the routed weights)."""
import json
import math

import pytest
import torch

from tests.plain import domorax_plain as P

F64 = torch.float64


# ---- configurations as the tests write them ----------------------------------------
def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, window=0, base=10000.0, scaling=None):
    m = {"dim": dim, "heads": heads, "kv_rank": kv_rank, "q_rank": q_rank, "rot": {"base": base, "dims": rot_dim},
         "rot_dim": rot_dim, "scale": scale, "vdim": vdim}
    if scaling:
        m["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    if window:
        m["mask"] = {"size": window}
    return m


def conv_attn(heads, kv_heads, dim, conv, scale):
    return {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv_heads, "scale": scale, "vdim": dim}


def delta(heads, kv_heads, dim, vdim, conv):
    return {"conv": conv, "dim": dim, "heads": heads, "kv_heads": kv_heads, "vdim": vdim}


def dense(ff):
    return {"ff": ff, "kind": "dense"}


def moe(ff, experts, top, shared=0):
    m = {"expert": {"ff": ff}, "kind": "moe", "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def layer(kind, mixer, mlp):
    return {"mixer": mixer, "mlp": mlp, "type": kind}


def model(layers, vocab, width, groups, mult, eps=1e-6):
    return {"architecture": "Domorax", "layers": layers, "norm": {"eps": eps, "groups": groups}, "residual_mult": mult,
            "torch_dtype": "bfloat16", "vocab": vocab, "width": width}


# A: every kind of layer and feed-forward; B: what A makes equal differs (key and value widths, heads and groups, one
# norm group, no window, no scaling, one expert a token, no shared expert, a layer without a feed-forward, one tap);
# C: sizes that are no multiple of 8
MODELS = {
    "A": model([layer("delta", delta(4, 2, 16, 24, 3), dense(96)),
                layer("latent_attention", latent(4, 16, 8, 24, 40, 32, 0.2, window=37, scaling=(4.0, 64, 16.0, 1.0)),
                      moe(32, 6, 2, shared=48)),
                layer("attention", conv_attn(6, 2, 32, 4, 0.15), moe(32, 6, 2, shared=48)),
                layer("latent_attention", latent(2, 24, 16, 8, 32, 24, 0.25, window=70), dense(64))],
               vocab=200, width=64, groups=4, mult=0.5),
    "B": model([layer("attention", conv_attn(3, 3, 16, 1, 0.3), None),
                layer("delta", delta(3, 3, 8, 8, 2), moe(16, 5, 1)),
                layer("latent_attention", latent(3, 8, 4, 8, 16, 16, 0.3, base=100.0), moe(24, 4, 3, shared=8)),
                layer("delta", delta(2, 1, 40, 12, 4), None),
                layer("attention", conv_attn(2, 1, 48, 2, 0.1), dense(40))],
               vocab=131, width=48, groups=1, mult=1.0, eps=1e-5),
    "C": model([layer("latent_attention", latent(5, 6, 2, 10, 12, 10, 0.35, window=5), moe(10, 3, 2, shared=6)),
                layer("delta", delta(6, 2, 5, 7, 3), dense(22)),
                layer("attention", conv_attn(3, 1, 20, 3, 0.2), dense(14))],
               vocab=77, width=30, groups=3, mult=0.7),
}


def config_of(data):
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.registry import config_from_dict
    return config_from_dict(json.loads(json.dumps(data)))


@pytest.mark.parametrize("name", list(MODELS))
def test_configuration_round_trip(name):
    cfg = config_of(MODELS[name])
    assert cfg.to_dict() == MODELS[name]
    assert config_of(cfg.to_dict()).to_dict() == MODELS[name]


def test_defaults_of_what_a_layer_leaves_out():
    cfg = config_of(MODELS["B"])
    lat = cfg.layers[2].mixer
    assert lat.window == 0 and lat.rot_scaling is None and lat.rot_dims == lat.rot_dim == 4
    assert cfg.layers[0].mlp is None and cfg.layers[1].mlp.shared_ff == 0 and cfg.layers[2].mlp.shared_ff == 8
    data = json.loads(json.dumps(MODELS["B"]))
    del data["residual_mult"], data["norm"]["groups"]
    cfg = config_of(data)
    assert cfg.residual_mult == 1.0 and cfg.norm_groups == 1


@pytest.mark.parametrize("change,key", [
    (lambda d: d["layers"][0].update(type="mamba"), "layers[0].type"),
    (lambda d: d["layers"][1]["mixer"].pop("conv"), "conv"),
    (lambda d: d["layers"][1]["mixer"].update(heads=4), "layers[1].mixer.heads"),
    (lambda d: d["layers"][2]["mixer"].update(rot_dim=3), "layers[2].mixer.rot_dim"),
    (lambda d: d["layers"][2]["mlp"]["router"].update(top=9), "layers[2].mlp.router.top"),
    (lambda d: d["layers"][4]["mixer"].update(vdim=8), "layers[4].mixer.vdim"),
    (lambda d: d["layers"][4]["mlp"].update(kind="glu"), "layers[4].mlp.kind"),
    (lambda d: d["norm"].update(groups=5), "norm.groups"),
    (lambda d: d.pop("vocab"), "vocab"),
    (lambda d: d.update(layers=[]), "layers"),
])
def test_errors_name_the_key(change, key):
    from hector_engine_amd.config.base import ConfigError
    data = json.loads(json.dumps(MODELS["B"]))
    change(data)
    with pytest.raises(ConfigError) as err:
        config_of(data)
    assert key in str(err.value)


def test_tensors_and_states_the_parts_ask_for():
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.parts.base import BuildEnv
    from hector_engine_amd.parts.delta_rule import state_floats
    from hector_engine_amd.registry import build_model
    m = build_model(config_of(MODELS["A"]), BuildEnv(torch.device("cpu"), torch.bfloat16))
    specs = {k: tuple(v.shape) for k, v in m.tensor_specs().items()}
    assert specs["embed"] == (200, 64) and specs["head"] == (200, 64) and specs["final.norm"] == (64,)
    assert specs["l0.mix.q"] == (32, 64) and specs["l0.mix.v.conv"] == (96, 3) and specs["l0.mix.norm"] == (24,)
    assert specs["l0.mix.A_log"] == (4,) and specs["l0.mlp.act"] == (4,) and specs["l0.dwa"] == (2,) and specs["l3.dwa"] == (5,)
    assert specs["l1.mix.uq"] == (4 * 24, 32) and specs["l1.mix.dkv"] == (48, 64) and specs["l1.mix.uk"] == (64, 40)
    assert specs["l1.mix.uv"] == (96, 40) and specs["l1.mix.sink"] == (4,) and specs["l1.mix.o"] == (64, 96)
    assert specs["l2.mix.k"] == (64, 64) and specs["l2.mix.q.norm"] == (32,) and specs["l2.mix.k.conv"] == (64, 4)
    assert "l2.mix.v" not in specs and "l1.mlp.correction" not in specs
    assert specs["l1.mlp.router"] == (6, 64) and specs["l1.mlp.e5.down"] == (64, 32) and specs["l1.mlp.shared.sg"] == (1, 64)
    plans = m.run_plans()
    # the delta layer carries 2 inputs of 160 channels and its matrices; the latent layers one key head of rot + rank
    # dims and a window; the convolved attention 3 inputs of its q and k channels
    assert plans[0].kv is None and plans[0].state_bytes == 4 * 2 * 160 + 4 * state_floats(4, 16, 24)
    assert (plans[1].kv.kv_heads, plans[1].kv.window, plans[1].state_bytes) == (1, 37, 0) and plans[1].kv.head_dim >= 48
    assert plans[2].kv.kv_heads == 2 and plans[2].kv.window == 0 and plans[2].state_bytes == 4 * 3 * (6 + 2) * 32
    assert state_floats(1, 32, 1) == 32 and state_floats(2, 96, 3) == 2 * 3 * 96 and state_floats(1, 5, 2) == 16
    assert state_floats(1, 130, 1) == 8 * 24


# ---- the plain implementation against itself --------------------------------------------
def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=F64) * scale


def test_the_recurrence_in_portions_is_the_recurrence():
    T, d, e = 50, 6, 4
    q, k, v = P.unit(rnd(T, d, seed=1)) * d ** -0.5, P.unit(rnd(T, d, seed=2)), rnd(T, e, seed=3)
    beta, g = torch.sigmoid(rnd(T, seed=4)), torch.exp(-torch.exp(rnd(T, seed=5)) * 0.3)
    whole, S = P.delta_rule(q, k, v, beta, g)
    parts, carry = [], None
    for a, b in ((0, 1), (1, 3), (3, 30), (30, 50)):
        o, carry = P.delta_rule(q[a:b], k[a:b], v[a:b], beta[a:b], g[a:b], carry)
        parts.append(o)
    assert torch.allclose(torch.cat(parts), whole, atol=1e-12) and torch.allclose(carry, S, atol=1e-12)
    # written once with full strength and never decayed, a value is read back exactly by its own key
    S0 = torch.zeros(d, e, dtype=F64)
    o, S1 = P.delta_rule(k[:1], k[:1], v[:1], torch.ones(1, dtype=F64), torch.ones(1, dtype=F64), S0)
    assert torch.allclose(o[0], v[0] * (k[0] @ k[0]), atol=1e-12)


def test_the_convolution_with_carried_inputs():
    u, taps = rnd(20, 5, seed=6), rnd(5, 4, seed=7)
    whole = P.short_conv(u, taps)
    tail = P.short_conv(u[8:], taps, before=u[5:8])
    assert torch.allclose(tail, whole[8:], atol=1e-12)
    assert torch.allclose(whole[0], taps[:, 3] * u[0], atol=1e-12)         # the last column is the current token's
    assert torch.allclose(whole[1], taps[:, 3] * u[1] + taps[:, 2] * u[0], atol=1e-12)


def test_the_scaled_rotation():
    plain, one = P.rotary_frequencies(8, 10000.0, None)
    assert one == 1.0 and plain == [10000.0 ** (-2 * i / 8) for i in range(4)]
    f, mult = P.rotary_frequencies(8, 10000.0, {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 1.0})
    assert abs(mult - (0.1 * math.log(4.0) + 1)) < 1e-12
    assert f[0] == plain[0] and abs(f[3] - plain[3] / 4.0) < 1e-15 and all(a <= b for a, b in zip(f, plain))
    x = rnd(3, 2, 12, seed=8)
    y = P.rotate_half(x, [0, 5, 9], 8, f, mult)
    assert torch.allclose(y[0, :, :8], x[0, :, :8] * mult) and torch.equal(y[:, :, 8:], x[:, :, 8:])
    norm = lambda t: (t[:, :, :8] ** 2).sum(-1)
    assert torch.allclose(norm(y), norm(x) * mult ** 2)


def test_the_routed_weights_and_the_group_norm():
    h = rnd(7, 10, seed=9)
    w = {"r.router": rnd(5, 10, seed=10)}
    for e in range(5):
        w[f"r.e{e}.gate"], w[f"r.e{e}.up"], w[f"r.e{e}.down"] = rnd(6, 10, seed=20 + e), rnd(6, 10, seed=30 + e), rnd(10, 6, seed=40 + e)
    every = P.routed_ff(h, w, "r.", {"router": {"experts": 5, "top": 5}})
    z = torch.softmax(h @ w["r.router"].T, -1)
    want = sum(z[:, e:e + 1] * P.gated_expert(h, w, f"r.e{e}.") for e in range(5))
    assert torch.allclose(every, want, atol=1e-12)          # all experts chosen: the softmax over all logits
    one = P.routed_ff(h, w, "r.", {"router": {"experts": 5, "top": 1}})
    best = (h @ w["r.router"].T).argmax(-1)
    assert torch.allclose(one[2], P.gated_expert(h[2:3], w, f"r.e{int(best[2])}.")[0], atol=1e-12)   # one expert: weight 1
    x, g = rnd(4, 12, seed=11), rnd(12, seed=12)
    assert torch.allclose(P.group_norm(x, g, 1, 1e-6), P.rms(x, 1e-6) * g)
    parts = P.group_norm(x, g, 3, 1e-6)
    assert torch.allclose(parts[:, 4:8], P.rms(x[:, 4:8], 1e-6) * g[4:8])


def test_prefix_logits_do_not_depend_on_what_follows():
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.parts.base import BuildEnv
    from hector_engine_amd.registry import build_model
    from hector_engine_amd.weights.random_init import random_tensors
    cfg = config_of(MODELS["C"])
    specs = build_model(cfg, BuildEnv(torch.device("cpu"), torch.bfloat16)).tensor_specs()
    w = {k: v.to(F64) for k, v in random_tensors(specs, 5, torch.bfloat16, "cpu").items()}
    ids = [3, 70, 12, 12, 5, 44, 9, 1, 30, 2, 61]
    whole = P.forward(MODELS["C"], w, ids)
    assert torch.allclose(P.forward(MODELS["C"], w, ids[:6]), whole[:6], atol=1e-9)
    assert P.greedy(MODELS["C"], w, ids[:4], 3) == P.greedy(MODELS["C"], w, ids[:4], 5)[:3]
