"""Domorax on the GPU against the plain implementation (tests/plain/domorax_plain.py): each new kernel
alone, fed in portions and in batches through slots that are used again, with inputs planted so that a
lost state, a window that is one token off, a left-out sink or a forgotten distance slope shows; then whole
models of several shapes and layer orders through the engine's step function, cut and batched in many ways,
in 32-bit and in bfloat16; and greedy generation through the library's own entry point, its command line
and the trace replay."""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

from tests.helpers import argmax_agrees_where_clear, rand_ids
from tests.plain import domorax_plain as P
from tests.test_domorax_cpu import MODELS, conv_attn, delta, dense, latent, layer, model, moe
from tests.test_kernels_gpu import dev, rnd

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64


@pytest.fixture(scope="module")
def ops():
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.kernels import ops as o
    return o


def i32(values):
    return torch.tensor(values, dtype=torch.int32, device="cuda")


# a schedule of steps over three sequences: (sequence, new tokens) per step; lengths 71, 9 and 140
SCHEDULE = [[(0, 3), (1, 1), (2, 64)], [(0, 1), (1, 1), (2, 1)], [(0, 2), (2, 2)], [(1, 7), (2, 70)],
            [(0, 64)], [(0, 1), (2, 1)], [(2, 2)]]
LENGTHS = [71, 9, 140]


def run_schedule(slots, per_step):
    done = [0, 0, 0]
    for step in SCHEDULE:
        seqs = [s for s, _ in step]
        q_lens = [n for _, n in step]
        per_step(seqs, q_lens, [done[s] for s in seqs], [slots[s] for s in seqs])
        for s, n in step:
            done[s] += n
    assert done == LENGTHS


def cu_of(q_lens):
    cu = [0]
    for n in q_lens:
        cu.append(cu[-1] + n)
    return i32(cu)


def rows_meta(q_lens, starts):
    positions, row_seq = [], []
    for i, (n, st) in enumerate(zip(q_lens, starts)):
        positions += list(range(st, st + n))
        row_seq += [i] * n
    return i32(positions), i32(row_seq)


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == "float32" else dict(rtol=2e-2, atol=2e-2)


# ------------------------------------------------------------------ the delta rule
def plain_delta(x, ba, a_log, dt_bias, H, G, d, e, q_scale):
    T = x.shape[0]
    q = P.unit(x[:, :G * d].double().reshape(T, G, d)) * q_scale
    k = P.unit(x[:, G * d:2 * G * d].double().reshape(T, G, d))
    v = x[:, 2 * G * d:2 * G * d + H * e].double().reshape(T, H, e)
    beta = torch.sigmoid(ba[:, :H].double())
    g = torch.exp(-torch.exp(a_log.double()) * P.softplus(ba[:, H:].double() + dt_bias.double()))
    out = torch.zeros(T, H, e, dtype=F64)
    for h in range(H):
        out[:, h], _ = P.delta_rule(q[:, h // (H // G)], k[:, h // (H // G)], v[:, h], beta[:, h], g[:, h])
    return out.reshape(T, H * e)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,d,e", [(4, 2, 16, 24), (3, 3, 8, 8), (2, 1, 40, 12), (6, 2, 5, 7), (1, 1, 1, 1), (2, 2, 130, 3),
                                     (2, 1, 96, 64), (1, 1, 32, 70), (1, 1, 300, 5)])
def test_delta_rule_in_portions_and_batches_equals_the_whole(ops, dtype, H, G, d, e):
    tdt = TORCH[dtype]
    wide = 2 * G * d + H * e + 8                                  # q | k | v inside wider rows, as behind a convolution
    xs = [rnd(n, wide, seed=10 + i).to(tdt) for i, n in enumerate(LENGTHS)]
    bas = [rnd(n, 2 * H, seed=20 + i, scale=2.0) for i, n in enumerate(LENGTHS)]
    a_log, dt_bias = rnd(H, seed=30, scale=0.5), rnd(H, seed=31) - 1.0
    q_scale = d ** -0.5
    want = [plain_delta(x.float(), ba, a_log, dt_bias, H, G, d, e, q_scale) for x, ba in zip(xs, bas)]
    offset = 256
    nbytes = 4 * ops.delta_state_floats(H, d, e)
    assert nbytes >= 4 * H * d * e
    state = torch.zeros(6, offset + nbytes + 64, dtype=torch.uint8, device="cuda")
    state[:, :offset] = 55
    state[:, offset + nbytes:] = 77                               # what lies around the matrices is not touched
    slots = [4, 0, 2]
    got = [torch.zeros(n, H * e, dtype=F64) for n in LENGTHS]

    def per_step(seqs, q_lens, starts, sl):
        x = dev(torch.cat([xs[s][at:at + n] for s, n, at in zip(seqs, q_lens, starts)]))
        ba = dev(torch.cat([bas[s][at:at + n] for s, n, at in zip(seqs, q_lens, starts)]))
        rows = x.shape[0]
        y = torch.full((rows, H * e), float("nan"), device="cuda")
        ops.delta_scan(y, x[:, :G * d], x[:, G * d:2 * G * d], x[:, 2 * G * d:2 * G * d + H * e], ba, dev(a_log), dev(dt_bias),
                       state, offset, cu_of(q_lens), i32(sl), rows, len(seqs), H, G, d, e, q_scale, 1e-6)
        at = 0
        for s, n, st in zip(seqs, q_lens, starts):
            got[s][st:st + n] = y[at:at + n].cpu().double()
            at += n

    run_schedule(slots, per_step)
    for g, w in zip(got, want):
        assert torch.allclose(g, w, rtol=1e-4, atol=2e-5 * max(1.0, w.abs().max().item()))
    assert bool((state[:, :offset] == 55).all()) and bool((state[:, offset + nbytes:] == 77).all())
    assert bool((state[[1, 3, 5]][:, offset:offset + nbytes] == 0).all())          # other slots' matrices stay zero


@pytest.mark.parametrize("feed", ["whole", "ones", "pairs"])
def test_a_value_written_early_is_read_back_far_later(ops, feed):
    """Token 3 writes a large value under a key of its own with full strength; no later token's key meets it and
    nothing decays. The query at the last of 400 tokens is that key: the output is the value, however the rows
    were fed. A state that is lost, begun again or moved to another slot gives zero instead."""
    H, G, d, e, T = 2, 1, 16, 8, 400
    x = torch.zeros(T, 2 * d + H * e)
    x[:, d + 1] = 1.0                                     # every token's key: unit vector 1
    x[:, 0] = 1.0                                         # every token's query: unit vector 0
    x[3, d:2 * d] = 0.0
    x[3, d + 5] = 1.0                                     # token 3's key: unit vector 5
    x[3, 2 * d:] = 7.0
    x[T - 1, :d] = 0.0
    x[T - 1, 5] = 1.0                                     # the last query asks for unit vector 5
    ba = torch.zeros(T, 2 * H)
    ba[:, :H] = 30.0                                      # beta = 1
    ba[:, H:] = -40.0                                     # softplus -> 0: no decay
    state = torch.zeros(3, 4 * ops.delta_state_floats(H, d, e), dtype=torch.uint8, device="cuda")
    y = torch.zeros(T, H * e, device="cuda")
    cuts = {"whole": [T], "ones": [1] * T, "pairs": [2] * (T // 2)}[feed]
    at = 0
    for n in cuts:
        xs, bs = dev(x[at:at + n]), dev(ba[at:at + n])
        out = torch.zeros(n, H * e, device="cuda")
        ops.delta_scan(out, xs[:, :d], xs[:, d:2 * d], xs[:, 2 * d:], bs, dev(torch.zeros(H)), dev(torch.zeros(H)), state, 0,
                       cu_of([n]), i32([1]), n, 1, H, G, d, e, 1.0, 0.0)
        y[at:at + n] = out
        at += n
    assert torch.allclose(y[T - 1].cpu(), torch.full((H * e,), 7.0), atol=1e-5)
    assert float(y[T - 2].abs().max()) < 1e-6 and float(y[3].abs().max()) < 1e-6


# ------------------------------------------------------------------ norms and small operations
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,D,groups", [(1, 8, 1), (5, 320, 4), (70, 30, 3), (3, 2048, 8), (2, 1030, 5)])
def test_a_branch_normed_in_groups_into_the_stream(ops, dtype, rows, D, groups):
    tdt = TORCH[dtype]
    resid, delta, w = rnd(rows, D, seed=1), rnd(rows, D, seed=2, scale=3.0).to(tdt), (rnd(D, seed=3) + 1).to(tdt)
    r = dev(resid.clone())
    out = torch.empty(rows, D, dtype=tdt, device="cuda")
    ops.add_group_normed(r, dev(delta), dev(w), groups, 1e-5, 0.5, out, rows)
    want = resid.double() + 0.5 * P.group_norm(delta.double(), w.double(), groups, 1e-5)
    assert torch.allclose(r.cpu().double(), want, rtol=1e-6, atol=1e-5)             # the stream itself stays in 32 bits
    assert torch.allclose(out.cpu().double(), want, **tol(dtype))
    normed = torch.empty(rows, D, dtype=tdt, device="cuda")
    ops.add_group_normed(r, None, None, 1, 0.0, 1.0, normed, rows, next_weight=dev(w), next_groups=groups, next_eps=1e-6)
    assert torch.allclose(normed.cpu().double(), P.group_norm(r.cpu().double(), w.double(), groups, 1e-6), **tol(dtype))
    before = r.clone()
    ops.add_group_normed(r, dev(delta), dev(w), groups, 1e-5, -0.5, None, rows)       # and taken out again
    assert torch.allclose(r.cpu(), resid, atol=1e-5) and not torch.equal(r, before)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,W", [(1, 4), (9, 384), (70, 22), (2, 3000)])
def test_polynorm(ops, dtype, rows, W):
    tdt = TORCH[dtype]
    z, numbers = rnd(rows, W, seed=4, scale=2.0).to(tdt), torch.tensor([0.7, -0.4, 0.25, 0.1]).to(tdt)
    out = dev(z.clone())
    ops.polynorm(out, out, dev(numbers), rows, 1e-6)
    want = P.poly_norm(z.double(), numbers.double(), 1e-6)
    assert torch.allclose(out.cpu().double(), want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,H,G,d", [(1, 1, 1, 4), (70, 6, 2, 32), (5, 3, 1, 20), (9, 2, 2, 96)])
def test_heads_normed_with_the_raw_keys_as_values(ops, dtype, rows, H, G, d):
    tdt = TORCH[dtype]
    x = rnd(rows, (H + G) * d + 3, seed=5, scale=2.0).to(tdt)
    qw, kw = (rnd(d, seed=6) + 1).to(tdt), (rnd(d, seed=7) + 1).to(tdt)
    out = torch.full((rows, (H + 2 * G) * d + 5), 9.0, dtype=tdt, device="cuda")
    ops.qk_head_norm(out, dev(x), dev(qw), dev(kw), H, G, d, 1e-5, rows, copy_v=True)
    q = P.rms(x[:, :H * d].double().reshape(rows, H, d), 1e-5) * qw.double()
    k = P.rms(x[:, H * d:(H + G) * d].double().reshape(rows, G, d), 1e-5) * kw.double()
    got = out.cpu().double()
    assert torch.allclose(got[:, :H * d], q.reshape(rows, -1), **tol(dtype))
    assert torch.allclose(got[:, H * d:(H + G) * d], k.reshape(rows, -1), **tol(dtype))
    assert torch.equal(out[:, (H + G) * d:(H + 2 * G) * d].cpu(), x[:, H * d:(H + G) * d])       # the values: the keys as they were
    assert bool((out[:, (H + 2 * G) * d:] == 9.0).all())
    same_place = dev(x.clone())
    ops.qk_head_norm(same_place, same_place, dev(qw), dev(kw), H, G, d, 1e-5, rows)
    assert torch.equal(same_place[:, :(H + G) * d], out[:, :(H + G) * d]) and torch.equal(same_place[:, (H + G) * d:].cpu(), x[:, (H + G) * d:])


def test_the_mix_over_all_results_so_far(ops):
    rows, D, n = 7, 30, 4
    kept = torch.zeros(n + 1, rows, D, device="cuda")
    planes = [rnd(rows, D, seed=40 + j) for j in range(n)]
    for j in range(n - 1):
        kept[j] = dev(planes[j])
    kept[n:] = 5.0
    resid = dev(planes[n - 1].clone())
    c = torch.tensor([0.5, -0.25, 2.0, 0.75]).to(torch.bfloat16)
    ops.depth_mix(resid, kept, dev(c), n, rows)
    want = sum(c[j].double() * planes[j].double() for j in range(n))
    assert torch.allclose(resid.cpu().double(), want, atol=1e-5)
    assert torch.equal(kept[n - 1].cpu(), planes[n - 1]) and bool((kept[n:] == 5.0).all())


@pytest.mark.parametrize("dtype", DTYPES)
def test_the_gate_of_a_shared_expert(ops, dtype):
    tdt = TORCH[dtype]
    rows, D = 9, 50
    a, b, x = (rnd(rows, D, seed=s).to(tdt) for s in (50, 51, 52))
    g = rnd(D, seed=53, scale=0.3).to(tdt)
    out = torch.empty(rows, D, dtype=tdt, device="cuda")
    ops.gated_add(out, dev(a), dev(b), dev(x), dev(g), rows)
    want = a.double() + torch.sigmoid(x.double() @ g.double())[:, None] * b.double()
    assert torch.allclose(out.cpu().double(), want, **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,H,K,N", [(1, 1, 1, 1), (9, 4, 16, 40), (70, 3, 300, 70), (130, 2, 40, 24)])
def test_a_product_per_head_on_strided_views(ops, dtype, rows, H, K, N):
    tdt = TORCH[dtype]
    x = rnd(rows, H, K + 5, seed=60).to(tdt)
    w = rnd(H, K, N, seed=61, scale=K ** -0.5).to(tdt)
    out = torch.full((rows, H, N + 3), 4.0, dtype=tdt, device="cuda")
    ops.head_product(out[:, :, 2:2 + N], dev(x)[:, :, 5:], dev(w), rows)
    want = torch.einsum("rhk,hkn->rhn", x[:, :, 5:].double(), w.double())
    assert torch.allclose(out[:, :, 2:2 + N].cpu().double(), want, **tol(dtype))
    assert bool((out[:, :, :2] == 4.0).all()) and bool((out[:, :, 2 + N:] == 4.0).all())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("K", [1, 2, 4])
def test_a_convolution_without_bias_and_activation_in_portions(ops, dtype, K):
    tdt = TORCH[dtype]
    C = 20
    us = [rnd(n, C + 4, seed=70 + i).to(tdt) for i, n in enumerate(LENGTHS)]
    taps = rnd(C, K, seed=80, scale=0.5).to(tdt)
    want = [P.short_conv(u[:, :C].double(), taps.double()) for u in us]
    state = torch.zeros(6, max(16, 4 * (K - 1) * C) + 32, dtype=torch.uint8, device="cuda")
    got = [torch.zeros(n, C, dtype=F64) for n in LENGTHS]

    def per_step(seqs, q_lens, starts, sl):
        x = dev(torch.cat([us[s][at:at + n] for s, n, at in zip(seqs, q_lens, starts)]))
        rows = x.shape[0]
        positions, row_seq = rows_meta(q_lens, starts)
        out = torch.empty(rows, C, dtype=tdt, device="cuda")
        ops.conv_state(out, x[:, :C], dev(taps), None, state, positions, row_seq, i32(sl), i32(starts), cu_of(q_lens), rows,
                       len(seqs), all(n == 1 for n in q_lens), act=False)
        at = 0
        for s, n, st in zip(seqs, q_lens, starts):
            got[s][st:st + n] = out[at:at + n].cpu().double()
            at += n

    run_schedule([4, 0, 2], per_step)
    for g, w in zip(got, want):
        assert torch.allclose(g, w, **tol(dtype))


@pytest.mark.parametrize("E,top", [(12, 2), (5, 1), (4, 4), (33, 7)])
def test_weights_that_are_the_softmax_over_the_chosen_logits(ops, E, top):
    rows, D = 40, 24
    x, router = rnd(rows, D, seed=90), rnd(E, D, seed=91)
    dense_w = torch.empty(rows, E + 1, device="cuda")
    ids = torch.empty(rows, top, dtype=torch.int32, device="cuda")
    weights = torch.empty(rows, top, device="cuda")
    ops.route_tokens(dense_w, ids, weights, None, None, rows, E, 1, 1, top, 1.0, x=dev(x), router=dev(router), normalize=True)
    z = x.double() @ router.double().T
    best = z.topk(top, -1)
    assert torch.equal(ids.cpu().long().sort(-1).values, best.indices.sort(-1).values)
    want = torch.zeros(rows, E, dtype=F64).scatter(1, best.indices, torch.softmax(best.values, -1))
    assert torch.allclose(dense_w[:, :E].cpu().double(), want, atol=1e-6) and float(dense_w[:, E].abs().max()) == 0.0
    assert torch.allclose(weights.cpu().double().sum(-1), torch.ones(rows, dtype=F64), atol=1e-6)
    assert torch.allclose(torch.gather(want, 1, ids.cpu().long()), weights.cpu().double(), atol=1e-6)


# ------------------------------------------------------------------ attention with distance slopes
@pytest.mark.parametrize("kind,dtype", [("plain", "float32"), ("plain", "bfloat16"), ("decode", "bfloat16"), ("prefill", "bfloat16"),
                                        ("prefill_without_lds", "bfloat16"), ("prefill_in_parts", "bfloat16")])
@pytest.mark.parametrize("H,KVH,hd", [(6, 2, 32), (4, 1, 96), (3, 3, 16), (20, 1, 48), (2, 1, 160)])
def test_scores_that_fall_with_the_distance(ops, kind, dtype, H, KVH, hd):
    """Every attention kernel with a slope a head, against the direct sums: prompts, a continuation and single tokens
    over page edges. One early key of every sequence is made to match the last query, with a score that equals what
    the slope takes off at that distance: without the slope it would take most of the weight; with it, it is one key
    among the near ones."""
    from tests.test_kernels_gpu import fill_cache, paged_setup
    tdt = TORCH[dtype]
    lengths, q_lens = ([300, 1, 64, 65, 131], [1, 1, 1, 1, 1]) if kind == "decode" else ([150, 237, 3, 66], [150, 37, 3, 1])
    slots, table, kpool, vpool = paged_setup(lengths, KVH, hd, tdt, 90)
    ks = [rnd(n, KVH, hd, seed=100 + i).to(tdt) for i, n in enumerate(lengths)]
    vs = [rnd(n, KVH, hd, seed=110 + i).to(tdt) for i, n in enumerate(lengths)]
    qs = [rnd(m, H, hd, seed=120 + i, scale=2.0).to(tdt) for i, m in enumerate(q_lens)]
    slopes = torch.tensor(P.head_slopes(H), dtype=torch.float32)
    scale = hd ** -0.5
    for k, q in zip(ks, qs):
        n = k.shape[0]
        if n > 8:
            first = q[-1, ::H // KVH].float()                        # the last query of each group's first head
            much = slopes[::H // KVH, None] * (n - 3) / (first.pow(2).sum(-1, keepdim=True) * scale)
            k[2] = (first * much).to(tdt)                            # key 2 points where that query points
    fill_cache(table, slots, kpool, vpool, ks, vs)
    rows = sum(q_lens)
    q = torch.cat(qs).reshape(rows, H * hd)
    positions = torch.cat([torch.arange(n - m, n) for n, m in zip(lengths, q_lens)]).int()
    row_seq = torch.cat([torch.full((m,), i) for i, m in enumerate(q_lens)]).int()
    cu, starts = cu_of(q_lens), i32([n - m for n, m in zip(lengths, q_lens)])
    out = torch.full((rows, H * hd), 7.0, dtype=tdt, device="cuda")
    pools = (dev(kpool), dev(vpool))
    if kind == "plain":
        ops.attention_plain(out, dev(q), *pools, dev(positions), dev(row_seq), i32(slots), dev(table), rows, H, KVH, hd, 0,
                            scale, slopes=dev(slopes))
    elif kind == "decode":
        ws = torch.empty(ops.attention_decode_workspace_floats(rows, H, KVH, hd, 4096), device="cuda")
        ops.attention_decode(out, dev(q), *pools, dev(positions), dev(row_seq), i32(slots), dev(table), rows, H, KVH, hd, 0,
                             scale, 4096, ws, slopes=dev(slopes))
    elif kind == "prefill_in_parts":
        if hd > 128:
            pytest.skip("keys in parts are for head sizes up to 128")
        ws = torch.empty(ops.attention_prefill_workspace_floats(rows, H, hd, 3), device="cuda")
        ops.attention_prefill(out, dev(q), *pools, cu, i32(slots), starts, dev(table), len(lengths), max(q_lens), rows, H, KVH,
                              hd, 0, scale, kernel=2, parts=3, workspace=ws, slopes=dev(slopes))
    else:
        # the library's choice (32 queries a wavefront with pages shared through LDS up to a head size of 128), or
        # the kernel of 16 queries a wavefront named outright
        ops.attention_prefill(out, dev(q), *pools, cu, i32(slots), starts, dev(table), len(lengths), max(q_lens), rows, H, KVH,
                              hd, 0, scale, kernel=1 if kind == "prefill_without_lds" else 0, slopes=dev(slopes))
    r, moved = 0, 0.0
    for i, (n, m) in enumerate(zip(lengths, q_lens)):
        want = P.distance_attention(qs[i].double(), ks[i].double(), vs[i].double(), scale, slopes.double().tolist(), n - m)
        flat = P.distance_attention(qs[i].double(), ks[i].double(), vs[i].double(), scale, [0.0] * H, n - m)
        got = out[r:r + m].cpu().double().reshape(want.shape)
        bound = 3e-5 if dtype == "float32" else 2 ** -6          # scores of a hundred, known to 32 bits, under an exponential
        assert torch.allclose(got, want, rtol=bound, atol=bound)
        moved = max(moved, (want[-1] - flat[-1]).abs().max().item())
        r += m
    assert moved > 0.3          # the slope decides here


# ------------------------------------------------------------------ whole models through the engine
SHARP = (".mix.q", ".mix.k", ".mix.uq", ".mix.uk", ".mix.dkv")


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    """name -> model folder. In the sharp variant the matrices are made larger than the random default, those in front
    of queries and keys most, so that attention weights are far from uniform and a key that is wrongly seen or missed,
    a sink or a slope matters; the calm variant (name + '_calm') keeps them nearer their random size."""
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.registry import config_from_dict
    from hector_engine_amd.weights import write_random_model
    from hector_engine_amd.weights.safetensors_io import write_safetensors
    from safetensors.torch import load_file
    out = {}
    for i, (name, cfg) in enumerate(MODELS.items()):
        for calm in (False, True):
            folder = str(tmp_path_factory.mktemp(f"domorax_{name}"))
            write_random_model(config_from_dict(json.loads(json.dumps(cfg))), 80 + i, folder, "bfloat16")
            path = folder + "/model.safetensors"
            tensors = load_file(path)
            for k in tensors:
                if k.endswith(SHARP):
                    tensors[k] = (tensors[k].float() * (2 if calm else 6)).to(torch.bfloat16)
                elif k.endswith((".router", ".mix.a", ".mix.b")):
                    tensors[k] = (tensors[k].float() * 8).to(torch.bfloat16)
                elif tensors[k].dim() == 2 and k != "embed" and not calm:
                    tensors[k] = (tensors[k].float() * 2).to(torch.bfloat16)
            write_safetensors(path, tensors, {"format": "pt"})
            out[name + "_calm" if calm else name] = folder
    return out


def variant(name, dtype):
    """The folder a precision is tested on: the sharp one in 32-bit; under bfloat16 the rounding of q and k times large
    scores moves single attention weights by tenths and the plain implementation in float64 is no measure, so the calm one."""
    return name if dtype == "float32" else name + "_calm"


@pytest.fixture(scope="module")
def plain(folders):
    return {name: P.read_model(f) for name, f in folders.items()}


@pytest.fixture(scope="module")
def engines(folders):
    import hector_engine_amd as he
    cache = {}

    def get(name, dtype, **kw):
        key = (name, dtype, tuple(sorted(kw.items())))
        if key not in cache:
            opts = dict(max_tokens=4096, max_slots=8, max_seq_len=1024)
            opts.update(kw)
            cache[key] = he.Engine(folders[variant(name, dtype)], dtype=dtype, **opts)
        return cache[key]

    return get


def same(got, want, dtype, tol32=2e-5):
    """float32: every logit within tol32 of the logits' size (or of 1). bfloat16: per position the root mean square of
    the logits' error (mean taken off) against that of the logits; the bound is on the bulk: a median of 3 % at most,
    5 % at most but for a tenth of the positions (or one), and never over 20 %."""
    got, want = got.detach().cpu().double(), want.double()
    assert got.shape == want.shape, (got.shape, want.shape)
    if dtype == "float32":
        scale = want.abs().max().item()
        err = (got - want).abs().max().item()
        assert err <= tol32 * max(scale, 1.0), f"max error {err:.3g} above {tol32 * max(scale, 1.0):.3g} (logit scale {scale:.3g})"
        return
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    r = d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt()
    assert bool(torch.isfinite(r).all())
    assert r.max().item() <= 0.2, r
    assert (r > 0.05).sum().item() <= max(1, len(r) // 10), r
    if len(r) >= 8:
        assert r.median().item() <= 0.03, r


def entry(slot, tokens, want):
    from hector_engine_amd.engine.engine import StepEntry
    return StepEntry(slot, list(tokens), list(want))


def test_the_folder_written_from_a_configuration_reads_back(folders):
    from hector_engine_amd.registry import load_config
    for name, folder in folders.items():
        assert load_config(folder).to_dict() == json.load(open(folder + "/config.json")) == MODELS[name.split("_")[0]]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_each_request_alone_and_whole(engines, plain, name, dtype):
    eng = engines(name, dtype)
    cfg, w = plain[variant(name, dtype)]
    for seed, n in enumerate([1, 2, 23, 64, 65, 150]):
        ids = rand_ids(cfg["vocab"], n, seed)
        s = eng.acquire()
        got = eng.step([entry(s, ids, range(n))])
        want = P.forward(cfg, w, ids)
        same(got, want, dtype)
        if dtype == "float32":
            argmax_agrees_where_clear(got, want, 0.05 * want.abs().max().item())
        eng.release(s)


def test_every_mechanism_matters_to_the_logits(plain, monkeypatch):
    """The models are such that leaving a mechanism out moves the logits by far more than the tests' bounds."""
    cfg, w = plain["A"]
    ids = rand_ids(cfg["vocab"], 90, 3)
    want = P.forward(cfg, w, ids)
    scale = want.abs().max().item()

    def moved(changed_cfg=None, changed_w=None, **patches):
        with monkeypatch.context() as mp:
            for k, v in patches.items():
                mp.setattr(P, k, v)
            return (P.forward(changed_cfg or cfg, changed_w or w, ids) - want).abs().max().item() / scale

    def with_mixer(i, **kw):
        c = json.loads(json.dumps(cfg))
        c["layers"][i]["mixer"].update(kw)
        return c

    assert moved(with_mixer(1, mask={"size": 36})) > 1e-3                   # a window one token shorter
    assert moved(with_mixer(1, mask={"size": 38})) > 1e-3                   # and one longer
    assert moved(with_mixer(3, mask=None)) > 1e-3
    no_scaling = with_mixer(1)
    no_scaling["layers"][1]["mixer"]["rot"].pop("scaling")
    assert moved(no_scaling) > 1e-3
    assert moved(changed_w={**w, "l1.mix.sink": w["l1.mix.sink"] - 30.0}) > 1e-3      # the sink left out
    assert moved(changed_w={**w, "l2.mix.k.conv": torch.roll(w["l2.mix.k.conv"], 1, 1)}) > 1e-3
    assert moved(changed_w={**w, "l3.dwa": torch.flip(w["l3.dwa"], [0])}) > 1e-2
    assert moved(group_norm=lambda x, g, n, eps: P.rms(x, eps) * g) > 1e-3
    assert moved(unit=lambda x: x) > 1e-3
    assert moved(poly_norm=lambda z, n, eps: P.silu(z)) > 1e-3
    assert moved(softplus=lambda z: z) > 1e-4
    c = json.loads(json.dumps(cfg))
    c["residual_mult"] = 1.0
    assert moved(c) > 1e-2


@pytest.mark.parametrize("name", list(MODELS))
def test_the_stream_after_every_layer(engines, plain, name, monkeypatch):
    eng = engines(name, "float32", use_graphs=False)
    cfg, w = plain[name]
    ids = rand_ids(cfg["vocab"], 70, 9)
    want = []
    P.forward(cfg, w, ids, want)
    seen = []
    import hector_engine_amd.engine.model as M
    mix = M.ops.depth_mix

    def watched(resid, kept, coeffs, n, rows):
        mix(resid, kept, coeffs, n, rows)
        seen.append(resid[:rows].clone())

    monkeypatch.setattr(M.ops, "depth_mix", watched)
    s = eng.acquire()
    eng.step([entry(s, ids, [69])])
    eng.release(s)
    assert len(seen) == len(want) == len(cfg["layers"])
    for got, ref in zip(seen, want):
        assert torch.allclose(got.cpu().double(), ref, rtol=2e-5, atol=2e-5 * ref.abs().max().item())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_prompt_then_token_by_token_over_page_edges(engines, plain, name, dtype):
    eng = engines(name, dtype)
    cfg, w = plain[variant(name, dtype)]
    n, tail = 210, 150                  # the decoded positions 60..209 cross two page edges and every window's edge
    ids = rand_ids(cfg["vocab"], n, 11)
    want = P.forward(cfg, w, ids)
    s = eng.acquire()
    whole = eng.step([entry(s, ids, range(n))]).clone()
    eng.release(s)
    s = eng.acquire()
    assert eng.step([entry(s, ids[:n - tail], [])]) is None
    dec = torch.cat([eng.step([entry(s, [t], [0])]).clone() for t in ids[n - tail:]])
    eng.release(s)
    same(dec, want[n - tail:], dtype)
    if dtype == "float32":
        assert torch.equal(dec, whole[n - tail:])        # the 32-bit path does not depend on the cut
    else:
        same(dec, whole[n - tail:].cpu(), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
@pytest.mark.parametrize("cuts", [[2] * 40, [3, 2, 61, 17, 64, 2, 70], [1, 1, 2, 1, 25, 47, 48, 2], [128, 2, 2, 65]])
def test_prompts_fed_in_portions(engines, plain, name, dtype, cuts):
    eng = engines(name, dtype)
    cfg, w = plain[variant(name, dtype)]
    n = sum(cuts)
    ids = rand_ids(cfg["vocab"], n, 12)
    want = P.forward(cfg, w, ids)
    s = eng.acquire()
    whole = eng.step([entry(s, ids, range(n))]).clone()
    eng.release(s)
    s = eng.acquire()
    parts, at = [], 0
    for c in cuts:
        parts.append(eng.step([entry(s, ids[at:at + c], range(c))]).clone())
        at += c
    eng.release(s)
    got = torch.cat(parts)
    same(got, want, dtype)
    if dtype == "float32":
        assert torch.equal(got, whole)
    else:
        same(got, whole.cpu(), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(MODELS))
def test_unequal_batches_equal_each_request_alone_and_slots_are_used_again(engines, plain, name, dtype):
    eng = engines(name, dtype, max_slots=4)
    cfg, w = plain[variant(name, dtype)]
    free = eng.cache.free_pages
    for round_no, lengths in enumerate([[1, 67, 140, 25], [90, 3, 49], [200, 2, 2, 64]]):
        prompts = [rand_ids(cfg["vocab"], n, 20 * round_no + i) for i, n in enumerate(lengths)]
        decode = 12
        full = [p + rand_ids(cfg["vocab"], decode - i, 500 + i) for i, p in enumerate(prompts)]   # shorter ones end earlier
        want = [P.forward(cfg, w, f) for f in full]
        slots = [eng.acquire() for _ in prompts]
        got = [[] for _ in prompts]
        logits = eng.step([entry(s, p, [len(p) - 1]) for s, p in zip(slots, prompts)])
        for i in range(len(prompts)):
            got[i].append(logits[i:i + 1].clone())
        live = list(range(len(prompts)))
        for t in range(decode):
            live = [i for i in live if len(prompts[i]) + t < len(full[i])]
            if not live:
                break
            logits = eng.step([entry(slots[i], [full[i][len(prompts[i]) + t]], [0]) for i in live])
            for j, i in enumerate(live):
                got[i].append(logits[j:j + 1].clone())
        for i, s in enumerate(slots):
            eng.release(s)          # the next round's requests take these slots, and their states, again
            same(torch.cat(got[i]), want[i][len(prompts[i]) - 1:], dtype)
    assert eng.cache.free_pages == free


@pytest.mark.parametrize("name", list(MODELS))
def test_a_mixed_step_of_a_prompt_and_decoding_requests(engines, plain, name):
    eng = engines(name, "float32")
    cfg, w = plain[name]
    a, b = rand_ids(cfg["vocab"], 80, 30), rand_ids(cfg["vocab"], 37, 31)
    sa, sb = eng.acquire(), eng.acquire()
    eng.step([entry(sa, a[:79], [])])
    got = eng.step([entry(sa, a[79:], [0]), entry(sb, b, range(37))])
    same(got[:1], P.forward(cfg, w, a)[-1:], "float32")
    same(got[1:], P.forward(cfg, w, b), "float32")
    eng.release(sa)
    eng.release(sb)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_long_request_and_long_decoding(engines, plain, dtype):
    eng = engines("A", dtype)
    cfg, w = plain[variant("A", dtype)]
    n = 520
    ids = rand_ids(cfg["vocab"], n, 41)
    want = P.forward(cfg, w, ids)
    s = eng.acquire()
    got = [eng.step([entry(s, ids[:300], [0, 36, 37, 63, 64, 299])]).clone()]
    got += [eng.step([entry(s, [t], [0])]).clone() for t in ids[300:]]
    eng.release(s)
    same(torch.cat(got), torch.cat([want[[0, 36, 37, 63, 64, 299]], want[300:]]), dtype, 6e-5)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_token_far_back_decides_where_only_full_attention_can_see_it(tmp_path, dtype):
    """One layer of the convolved attention (slopes, no window) and one of the latent attention with a window of 9. A
    key far back is planted by repeating one rare token: the engine and the plain implementation must agree at the
    positions just inside and just outside the window and 300 tokens later, whole and decoded."""
    import hector_engine_amd as he
    from hector_engine_amd.registry import config_from_dict
    from hector_engine_amd.weights import write_random_model
    cfg = model([layer("attention", conv_attn(4, 2, 32, 2, 0.6), dense(32)),
                 layer("latent_attention", latent(2, 16, 8, 16, 24, 16, 0.8, window=9), None)], 60, 32, 2, 1.0)
    folder = str(tmp_path)
    write_random_model(config_from_dict(json.loads(json.dumps(cfg))), 7, folder, "bfloat16")
    c, w = P.read_model(folder)
    ids = [int(t) % 50 for t in rand_ids(50, 330, 5)]
    for at in (2, 310, 318, 319, 320):
        ids[at] = 57                                    # the rare token
    want = P.forward(c, w, ids)
    eng = he.Engine(folder, dtype=dtype, max_tokens=1024, max_slots=2, max_seq_len=512)
    s = eng.acquire()
    whole = eng.step([entry(s, ids, range(330))]).clone()
    eng.release(s)
    same(whole, want, dtype)
    s = eng.acquire()
    eng.step([entry(s, ids[:300], [])])
    dec = torch.cat([eng.step([entry(s, [t], [0])]).clone() for t in ids[300:]])
    eng.release(s)
    same(dec, want[300:], dtype)


@pytest.mark.parametrize("name", list(MODELS))
def test_greedy_generation_through_the_library(folders, plain, name):
    import hector_engine_amd as he
    cfg, w = plain[name]
    prompts = [rand_ids(cfg["vocab"], n, 70 + i) for i, n in enumerate([5, 30, 61])]
    steps = 24
    want = [P.greedy(cfg, w, p, steps) for p in prompts]
    eng = he.Engine(folders[name], dtype="float32", max_tokens=2048, max_seq_len=512)
    got = he.generate(eng, prompts, max_new_tokens=steps, stop_ids=())
    assert [r.tokens for r in got] == want
    small = he.Engine(folders[name], dtype="float32", max_tokens=2048, max_slots=2, max_seq_len=512)
    assert [r.tokens for r in he.generate(small, prompts, max_new_tokens=steps, stop_ids=())] == want
    assert small.cache.free_pages == small.cache.num_pages
    cfg, w = plain[name + "_calm"]
    want = [P.greedy(cfg, w, p, steps) for p in prompts]
    eng16 = he.Engine(folders[name + "_calm"], dtype="bfloat16", max_tokens=2048, max_seq_len=512)
    for p, r, t in zip(prompts, he.generate(eng16, prompts, max_new_tokens=steps, stop_ids=()), want):
        seq = list(p)
        for x, y in zip(r.tokens, t):
            if x != y:
                top = P.forward(cfg, w, seq)[-1].topk(2).values
                assert (top[0] - top[1]).item() < 0.03 * top[0].abs().item() + 1e-3      # a near tie
                break
            seq.append(x)


def test_the_command_line_and_the_trace_replay_serve_it(folders, plain, tmp_path):
    import numpy as np
    from tests.conftest import ROOT
    cfg, w = plain["B"]
    exe = os.path.join(ROOT, "bin", "hector_generate")
    out = subprocess.run([sys.executable, exe, folders["B"], "5,17,3;9,2,77,13", "6", "--dtype", "float32",
                          "--stop-ids", ""], capture_output=True, text=True, timeout=180)
    assert out.returncode == 0, out.stderr
    for i, p in enumerate(([5, 17, 3], [9, 2, 77, 13])):
        assert f"[{i}] prompt" in out.stdout and ",".join(map(str, P.greedy(cfg, w, p, 6))) in out.stdout
    assert "Domorax" in out.stdout
    reqs = {"a": rand_ids(cfg["vocab"], 4, 1), "b": rand_ids(cfg["vocab"], 68, 2), "c": rand_ids(cfg["vocab"], 133, 3)}
    steps = [{"step": 0, "entries": [{"id": k, "tokens": v[:-3], "want": [len(v) - 4]} for k, v in reqs.items()], "end": []}]
    for t in range(3):
        steps.append({"step": t + 1, "entries": [{"id": k, "tokens": [v[len(v) - 3 + t]], "want": [0]} for k, v in reqs.items()],
                      "end": list(reqs) if t == 2 else []})
    for dtype in DTYPES:
        out_dir = str(tmp_path / dtype)
        cfg, w = plain[variant("B", dtype)]
        proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[variant("B", dtype)],
                               "--dtype", dtype, "--out", out_dir, "--max-tokens", "196"],
                              input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=180)
        assert proc.returncode == 0, proc.stderr
        assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
        want = {k: P.forward(cfg, w, v) for k, v in reqs.items()}
        for s in range(4):
            got = torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{s}.f32"), dtype="<f4").reshape(3, -1).copy())
            rows = torch.stack([want[k][len(reqs[k]) - 4 + s] for k in reqs])
            same(got, rows, dtype)


# ------------------------------------------------------------------ random configurations
def random_configuration(rng):
    """Layers of every kind in any order, with sizes drawn from small sets that hold odd ones, ones, and pairs that
    are equal as well as pairs that differ."""
    layers = []
    for _ in range(rng.randint(1, 4)):
        kind = rng.choice(["latent_attention", "attention", "delta"])
        kv = rng.choice([1, 2, 3])
        heads = kv * rng.choice([1, 2, 3])
        if kind == "latent_attention":
            rot = rng.choice([0, 2, 4, 8, 16])
            scaling = rng.choice([None, (2.0, 32, 8.0, 1.0), (8.0, 128, 32.0, 2.0)]) if rot else None
            mixer = latent(heads, rng.choice([4, 8, 12, 16]), rot, rng.choice([4, 8, 20]), rng.choice([8, 16, 24, 40]),
                           rng.choice([8, 16, 24]), rng.choice([0.1, 0.2, 0.3]), rng.choice([0, 1, 3, 64, 65, 100]),
                           rng.choice([100.0, 10000.0]), scaling)
        elif kind == "attention":
            mixer = conv_attn(heads, kv, rng.choice([8, 12, 16, 24, 32]), rng.choice([1, 2, 3, 4]), rng.choice([0.1, 0.2, 0.3]))
        else:
            mixer = delta(heads, kv, rng.choice([1, 4, 8, 10, 16, 40]), rng.choice([1, 4, 12, 16, 36]), rng.choice([1, 2, 3, 4]))
        experts = rng.choice([2, 3, 8])
        mlp = rng.choice([None, dense(rng.choice([6, 16, 40])), moe(rng.choice([8, 16, 24]), experts, rng.randint(1, experts),
                                                                    rng.choice([0, 8, 16]))])
        layers.append(layer(kind, mixer, mlp))
    groups = rng.choice([1, 2, 3, 4])
    return model(layers, rng.choice([50, 97, 130]), groups * rng.choice([8, 12, 16, 24]), groups, rng.choice([1.0, 0.5, 0.25]),
                 rng.choice([1e-6, 1e-5]))


@pytest.mark.parametrize("dtype,seed", [("float32", s) for s in range(12)] + [("bfloat16", s) for s in range(12, 20)])
def test_random_configurations(tmp_path, dtype, seed):
    """A prompt batch in portions, then one-token steps of the batch, twice through the same slots, against the
    plain implementation; in 32-bit, and with other configurations under bfloat16."""
    calm = dtype == "bfloat16"
    import random
    import hector_engine_amd as he
    from hector_engine_amd.registry import config_from_dict
    from hector_engine_amd.weights import write_random_model
    from hector_engine_amd.weights.safetensors_io import write_safetensors
    from safetensors.torch import load_file
    rng = random.Random(seed)
    cfg = random_configuration(rng)
    folder = str(tmp_path)
    write_random_model(config_from_dict(json.loads(json.dumps(cfg))), seed, folder, "bfloat16")
    path = folder + "/model.safetensors"
    tensors = load_file(path)
    for k in tensors:
        if k.endswith(SHARP):
            tensors[k] = (tensors[k].float() * (2 if calm else 6)).to(torch.bfloat16)
        elif tensors[k].dim() == 2 and k != "embed" and not calm:
            tensors[k] = (tensors[k].float() * 2).to(torch.bfloat16)
    write_safetensors(path, tensors, {"format": "pt"})
    c, w = P.read_model(folder)
    lens = [rng.choice([1, 2, 5, 63, 64, 65, 130]) for _ in range(3)]
    fulls = [rand_ids(c["vocab"], n + 6, seed * 10 + i) for i, n in enumerate(lens)]
    wants = [P.forward(c, w, f) for f in fulls]
    eng = he.Engine(folder, dtype=dtype, max_tokens=2048, max_slots=4, max_seq_len=512)
    for _ in range(2):
        slots = [eng.acquire() for _ in fulls]
        got = [[] for _ in fulls]
        cut = [max(1, n // 2) for n in lens]
        logits = eng.step([entry(s, f[:k], range(k)) for s, f, k in zip(slots, fulls, cut)])
        at = 0
        for i, k in enumerate(cut):
            got[i].append(logits[at:at + k].clone())
            at += k
        for i, (s, f, k, n) in enumerate(zip(slots, fulls, cut, lens)):
            if n > k:
                got[i].append(eng.step([entry(s, f[k:n], range(n - k))]).clone())
        for t in range(6):
            logits = eng.step([entry(s, [f[n + t]], [0]) for s, f, n in zip(slots, fulls, lens)])
            for i in range(len(fulls)):
                got[i].append(logits[i:i + 1].clone())
        for s in slots:
            eng.release(s)
        for g, want in zip(got, wants):
            same(torch.cat(g), want, dtype, 6e-5)
