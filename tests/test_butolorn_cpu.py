"""Butolorn without a GPU: its configuration (every size from the file, defaults for what a layer
leaves out, errors that name the key), the order its layers run in, the tensors its parts ask for,
the state a sequence carries, and the plain implementation against itself (a prompt at once equals
the same tokens one by one and in portions, through what it carries)."""
import copy
import math

import pytest
import torch

import hector_engine_amd  # noqa: F401
from hector_engine_amd.config.base import ConfigError
from hector_engine_amd.parts.base import BuildEnv
from hector_engine_amd.registry import build_model, config_from_dict
from tests.plain import butolorn_plain as P


def attn(heads, kv, dim, vdim, scale, rot_dims, base=10000.0):
    return {"dim": dim, "heads": heads, "kv_heads": kv, "rot": {"base": base, "dims": rot_dims}, "scale": scale,
            "vdim": vdim}


def memory(heads, dim, vdim, cap):
    return {"dim": dim, "gate_cap": cap, "heads": heads, "vdim": vdim}


def pair(left, right, left_scale=1.0, right_scale=1.0):
    return {"left": left, "left_scale": left_scale, "right": right, "right_scale": right_scale}


def layer(kind, mixer, ff=None):
    return {"mixer": mixer, "mlp": None if ff is None else {"ff": ff, "kind": "dense"}, "type": kind}


def model(layers, vocab, width, side, loop=(0, 0, 1), eps=1e-6, scale=1.0):
    d = {"architecture": "Butolorn", "embedding": {"scale": scale}, "layers": layers,
         "loop": {"start": loop[0], "stop": loop[1], "times": loop[2]}, "norm": {"eps": eps}, "vocab": vocab,
         "width": width}
    if side:
        d["token_side"] = {"dim": side}
    return d


SMALL = model([layer("parallel", pair(attn(4, 2, 8, 12, 0.3, 4, 500.0), memory(3, 6, 10, 9.0), 0.7, 1.3), 20),
               layer("attention", attn(3, 1, 10, 6, 0.25, 10)),
               layer("parallel", pair(attn(2, 2, 16, 16, 0.2, 16), memory(1, 20, 4, 15.0)), 12)],
              vocab=53, width=24, side=5, loop=(1, 3, 2), eps=1e-5, scale=3.0)


def test_configuration_reads_back_and_every_size_comes_from_the_file():
    cfg = config_from_dict(copy.deepcopy(SMALL))
    assert cfg.to_dict() == SMALL
    assert [l.type for l in cfg.layers] == ["parallel", "attention", "parallel"]
    a, p = cfg.layers[1].mixer, cfg.layers[0].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.rot_dims, a.rot_base) == (3, 1, 10, 6, 0.25, 10, 10000.0)
    assert (p.left.heads, p.left.kv_heads, p.left.dim, p.left.vdim, p.left.rot_dims, p.left.rot_base) == (4, 2, 8, 12, 4, 500.0)
    assert (p.right.heads, p.right.dim, p.right.vdim, p.right.gate_cap) == (3, 6, 10, 9.0)
    assert (p.left_scale, p.right_scale) == (0.7, 1.3)
    assert cfg.layers[0].mlp.ff == 20 and cfg.layers[1].mlp is None
    assert (cfg.vocab, cfg.width, cfg.side_dim, cfg.norm_eps, cfg.embedding_scale) == (53, 24, 5, 1e-5, 3.0)


def test_the_order_of_runs():
    cfg = config_from_dict(copy.deepcopy(SMALL))
    assert cfg.runs() == [(0, False), (1, False), (2, False), (1, True), (2, False)] == P.order_of_runs(SMALL)
    d = copy.deepcopy(SMALL)
    d["loop"] = {"start": 0, "stop": 2, "times": 3}
    assert config_from_dict(d).runs() == [(0, False), (1, False), (0, True), (1, False), (0, True), (1, False), (2, False)] \
        == P.order_of_runs(d)
    d["loop"] = {"start": 2, "stop": 3, "times": 1}
    assert config_from_dict(d).runs() == [(0, False), (1, False), (2, False)] == P.order_of_runs(d)
    del d["loop"]
    assert config_from_dict(d).runs() == [(0, False), (1, False), (2, False)] == P.order_of_runs(d)


def test_defaults_for_what_a_layer_leaves_out():
    d = copy.deepcopy(SMALL)
    del d["layers"][1]["mixer"]["kv_heads"], d["layers"][1]["mixer"]["vdim"], d["layers"][1]["mixer"]["rot"]
    del d["layers"][0]["mixer"]["left_scale"], d["token_side"], d["embedding"]
    cfg = config_from_dict(d)
    a = cfg.layers[1].mixer
    assert (a.kv_heads, a.vdim, a.rot_dims) == (3, 10, 0)
    assert cfg.layers[0].mixer.left_scale == 1.0 and cfg.side_dim == 0 and cfg.embedding_scale == 1.0
    spec = build_model(cfg, BuildEnv(torch.device("cpu"), torch.float32)).tensor_specs()
    assert "side.embed" not in spec and "l0.side.gate" not in spec
    d["layers"][2]["mixer"]["left"]["rot"]["dims"] = 0                 # no dimension rotated: the same as no 'rot'
    assert config_from_dict(d).layers[2].mixer.left.rot_dims == 0


@pytest.mark.parametrize("path,value,word", [
    (("layers", 0, "type"), "conv", "unknown mixer type"),
    (("layers", 1, "mixer", "kv_heads"), 2, "kv_heads"),
    (("layers", 1, "mixer", "rot", "dims"), 7, "rot.dims"),
    (("layers", 1, "mixer", "rot", "dims"), 12, "rot.dims"),
    (("layers", 0, "mixer", "right", "gate_cap"), 0.0, "gate_cap"),
    (("layers", 0, "mlp", "kind"), "moe", "unknown kind"),
    (("loop", "stop"), 4, "loop"),
    (("loop", "times"), 0, "loop.times"),
    (("width",), 0, "width"),
])
def test_errors_name_the_key(path, value, word):
    d = copy.deepcopy(SMALL)
    at = d
    for k in path[:-1]:
        at = at[k]
    at[path[-1]] = value
    with pytest.raises(ConfigError, match=word):
        config_from_dict(d)


def test_tensors_the_parts_ask_for_and_the_state_a_sequence_carries():
    m = build_model(config_from_dict(copy.deepcopy(SMALL)), BuildEnv(torch.device("cpu"), torch.float32))
    specs = {k: tuple(v.shape) for k, v in m.tensor_specs().items()}
    assert specs["embed"] == (53, 24) and specs["final.norm"] == (24,) and specs["side.embed"] == (53, 15)
    assert "head" not in specs and "l1.norm2" not in specs and "l1.mlp.up" not in specs
    for l in range(3):
        assert specs[f"l{l}.norm1"] == specs[f"l{l}.norm1b"] == specs[f"l{l}.side.norm"] == (24,)
        assert specs[f"l{l}.side.gate"] == (5, 24) and specs[f"l{l}.side.proj"] == (24, 5)
    assert specs["l0.norm2"] == specs["l0.norm2b"] == (24,)
    assert specs["l0.mlp.up"] == (20, 24) and specs["l0.mlp.down"] == (24, 20)
    assert specs["l1.mix.q"] == (30, 24) and specs["l1.mix.k"] == (10, 24) and specs["l1.mix.v"] == (6, 24)
    assert specs["l1.mix.q.b"] == (30,) and specs["l1.mix.k.b"] == (10,) and specs["l1.mix.v.b"] == (6,)
    assert specs["l1.mix.o"] == (24, 18) and "l1.mix.o.b" not in specs and "l1.mix.g" not in specs
    assert specs["l0.mix.left.q"] == (32, 24) and specs["l0.mix.left.k"] == (16, 24) and specs["l0.mix.left.v"] == (24, 24)
    assert specs["l0.mix.left.q.norm"] == (32,) and specs["l0.mix.left.k.norm"] == (16,)
    assert specs["l0.mix.left.g"] == (48, 24) and specs["l0.mix.left.o"] == (24, 48) and "l0.mix.left.q.b" not in specs
    assert specs["l0.mix.right.q"] == specs["l0.mix.right.k"] == (18, 24)
    assert specs["l0.mix.right.v"] == specs["l0.mix.right.g"] == (30, 24) and specs["l0.mix.right.o"] == (24, 30)
    assert specs["l0.mix.right.norm"] == (30,)
    assert specs["l0.mix.right.i"] == specs["l0.mix.right.f"] == (3, 24)
    assert specs["l0.mix.right.i.b"] == specs["l0.mix.right.f.b"] == (3,)
    plans = m.run_plans()
    assert len(plans) == 5                                   # one a run: a repeated layer has a cache and a state a pass
    assert plans[1].state_bytes == 0 and plans[1].kv is not None and plans[0].kv is not None
    # every run of a side-by-side layer carries a memory of at least heads * dim * vdim floats, a key sum and a maximum
    assert plans[0].state_bytes >= 4 * (3 * 6 * 10 + 3 * 6 + 3)
    assert plans[2].state_bytes == plans[4].state_bytes >= 4 * (20 * 4 + 20 + 1)
    assert plans[0].kv.kv_heads == 2 and plans[2].kv.kv_heads == 2 and plans[1].kv.kv_heads == 1


def random_weights(cfg_dict, seed):
    m = build_model(config_from_dict(copy.deepcopy(cfg_dict)), BuildEnv(torch.device("cpu"), torch.float32))
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, spec in m.tensor_specs().items():
        t = torch.randn(tuple(spec.shape), generator=g, dtype=torch.float64)
        w[name] = t * (0.3 if len(spec.shape) == 2 else 0.5)
    return w


def test_plain_prompt_equals_plain_token_by_token_and_portions():
    w = random_weights(SMALL, 3)
    ids = torch.randint(0, 53, (23,), generator=torch.Generator().manual_seed(5)).tolist()
    whole, _ = P.forward(SMALL, w, ids)
    carry, rows = None, []
    for t in ids:
        out, carry = P.forward(SMALL, w, [t], carry)
        rows.append(out)
    assert torch.allclose(torch.cat(rows), whole, rtol=1e-9, atol=1e-9)
    carry, rows, at = None, [], 0
    for c in (2, 1, 7, 2, 11):
        out, carry = P.forward(SMALL, w, ids[at:at + c], carry)
        rows.append(out)
        at += c
    assert torch.allclose(torch.cat(rows), whole, rtol=1e-9, atol=1e-9)


def test_plain_memory_equals_its_sum_form():
    """The recurrence with a running maximum equals the direct sums it stands for:
    y_t = sum_s w_ts (k_s . q_t) v_s / (max(|sum_s w_ts k_s . q_t|, exp(-m_t)) + 1e-6), with
    w_ts = exp(i_s + f_(s+1) + .. + f_t - m_t) and m_t = max(0 + f_1 + .. + f_t, max_s (i_s + f_(s+1) + .. + f_t))."""
    g = torch.Generator().manual_seed(1)
    T, H, d, e = 9, 2, 3, 4
    q, k = torch.randn(T, H, d, generator=g, dtype=torch.float64), torch.randn(T, H, d, generator=g, dtype=torch.float64)
    v = torch.randn(T, H, e, generator=g, dtype=torch.float64)
    log_in = 2 * torch.randn(T, H, generator=g, dtype=torch.float64)
    log_keep = P.log_sigmoid(2 * torch.randn(T, H, generator=g, dtype=torch.float64))
    y, (S, n, m) = P.memory_scan(q, k, v, log_in, log_keep)
    for a in range(H):
        for t in range(T):
            tail = [log_keep[s + 1:t + 1, a].sum().item() for s in range(t + 1)]
            logs = [log_in[s, a].item() + tail[s] for s in range(t + 1)]
            top = max([log_keep[:t + 1, a].sum().item()] + logs)
            wts = [math.exp(x - top) for x in logs]
            num = sum(wt * torch.dot(k[s, a], q[t, a]) * v[s, a] for s, wt in enumerate(wts))
            den = sum(wt * torch.dot(k[s, a], q[t, a]) for s, wt in enumerate(wts))
            want = num / (max(abs(den.item()), math.exp(-top)) + 1e-6)
            assert torch.allclose(y[t, a], want, rtol=1e-10, atol=1e-12)
        assert abs(m[a].item() - top) < 1e-12


def test_plain_rotation_layouts_and_the_added_one():
    x = torch.arange(12, dtype=torch.float64).reshape(1, 1, 12) + 1
    for inter, (a, b) in ((True, (2, 3)), (False, (1, 5))):
        y = P.rotate(x, [7], 8, 100.0, inter)
        ang = 7 * 100.0 ** (-2.0 / 8)                     # pair 1
        assert abs(y[0, 0, a].item() - (x[0, 0, a] * math.cos(ang) - x[0, 0, b] * math.sin(ang)).item()) < 1e-12
        assert abs(y[0, 0, b].item() - (x[0, 0, b] * math.cos(ang) + x[0, 0, a] * math.sin(ang)).item()) < 1e-12
        assert torch.equal(y[..., 8:], x[..., 8:])        # what lies behind the rotated dims stays
    q, k, v = torch.ones(1, 2, dtype=torch.float64), torch.zeros(3, 2, dtype=torch.float64), torch.eye(3, dtype=torch.float64)
    # three keys of score 0: a third each, and a quarter each with one more in the denominator
    assert torch.allclose(P.softmax_attention(q, k, v, 1.0, 2, False), torch.full((1, 3), 1 / 3, dtype=torch.float64))
    assert torch.allclose(P.softmax_attention(q, k, v, 1.0, 2, True), torch.full((1, 3), 0.25, dtype=torch.float64))
