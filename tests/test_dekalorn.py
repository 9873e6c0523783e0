"""The Dekalorn design in the layer-list engine against its plain float64 implementation (dekalorn_oracle.py):
every mechanism alone, prefill against token-by-token decoding, portions, mixed batches, reused blocks and slots,
far keys, window edges, block and tile borders, long decoding, other sizes, generation through the engine's own
entry points. Every case runs on the CPU (torch twin of the executor: host logic) and, marked gpu, on the HIP
kernels."""
from __future__ import annotations

import json
import math
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

import dekalorn_cases as dc
import dekalorn_oracle as oracle
from ollama_operator_amd.engine.sampling import SamplingOptions
from ollama_operator_amd.engine.scheduler import BatchScheduler
from ollama_operator_amd.models.config import StackConfig, UnsupportedArchitecture, load_stack_config, rotary_inv_freq

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
BOTH = ["float32", "bfloat16"]
GREEDY = SamplingOptions(temperature=0.0, repeat_penalty=1.0)
F64 = torch.float64


@pytest.fixture(scope="module")
def std(tmp_path_factory):
    return dc.Model(tmp_path_factory.mktemp("dekalorn"), dc.standard(), seed=3)


# ------------------------------------------------------------------ configuration
def test_config_roundtrip(std):
    cfg = load_stack_config(std.path)
    assert cfg == dc.standard() and not cfg.has_state
    assert StackConfig.from_dekalorn(cfg.to_dekalorn()) == cfg
    # layer 0, then the span 1..3 twice (each pass opens at layer 1), then the rest
    assert cfg.runs() == [(0, 0, False), (1, 0, True), (2, 0, False), (3, 0, False), (1, 1, True), (2, 1, False), (3, 1, False),
                          (4, 0, False), (5, 0, False)]
    r = std.runner("cpu")
    # K rows: latent | rotated part; every key/value head's key side by side; two maps side by side
    assert r.kc[0].shape[1:] == (1, 16, 18) and r.kc[1].shape[1:] == (1, 16, 32) and r.kc[2].shape[1:] == (2, 16, 16)
    assert r.vc[0] is None and r.vc[1].shape[1:] == (2, 16, 12)


def test_bench_configurations_are_readable():
    """The sizes `bench.py --stack ... --dekalorn` measures are valid configurations of the design."""
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench
    for z in bench.DEKALORN_SIZES.values():
        cfg = bench.dekalorn_config(z)
        assert StackConfig.from_dekalorn(cfg.to_dekalorn()) == cfg
        assert len(cfg.layers) == 8 and not cfg.has_state


def test_unknown_parts_are_refused():
    c = dc.standard().to_dekalorn()
    for path, val in ((("layers", 0, "type"), "conv_mixer"), (("layers", 0, "mlp", "kind"), "glu"),
                      (("layers", 1, "mixer", "rot", "dims"), 7), (("layers", 1, "mixer", "kv_heads"), 3),
                      (("layers", 1, "mlp", "router", "groups", "count"), 4), (("layers", 1, "mlp", "router", "top"), 5),
                      (("loop", "stop"), 9)):
        d = json.loads(json.dumps(c))
        node = d
        for k in path[:-1]:
            node = node[k]
        node[path[-1]] = val
        with pytest.raises(UnsupportedArchitecture):
            StackConfig.from_dekalorn(d)


def test_frequency_scaling_by_hand():
    """Bands with original 64, low 1, high 5: waves shorter than 12.8 keep their frequency, longer than 64 are divided
    by the factor, and one between sits at s = (64 / wave - 1) / 4."""
    f = rotary_inv_freq(8, 100.0, dc.BANDS)
    plain = [100.0 ** (-2 * i / 8) for i in range(4)]
    waves = [2 * math.pi / x for x in plain]                 # 6.3, 19.9, 62.8, 198.7
    assert waves[0] < 12.8 < waves[1] < waves[2] < 64 < waves[3]
    assert f[0] == plain[0] and f[3] == plain[3] / 6
    for i in (1, 2):
        s = (64 / waves[i] - 1) / 4
        assert abs(f[i] - ((1 - s) * plain[i] / 6 + s * plain[i])) < 1e-15
    rot = dict(dims=8, base=100.0, scaling=dict(factor=6.0, low=1.0, high=5.0, original=64))
    assert np.allclose(oracle.rotary_frequencies(rot).numpy(), f)


def test_oracle_mechanisms_by_hand():
    """The plain implementation on numbers worked out by hand."""
    # adjacent pairs: (1, 0) at position 1 with frequency pi / 2 becomes (0, 1); the third dim passes
    x = torch.tensor([[[1.0, 0.0, 5.0]], [[1.0, 0.0, 5.0]]], dtype=F64)
    y = oracle.rotate_pairs(x, torch.arange(2), torch.tensor([math.pi / 2], dtype=F64))
    assert np.allclose(y.numpy(), [[[1.0, 0.0, 5.0]], [[0.0, 1.0, 5.0]]])
    # a window of 2: row 2 sees rows 1 and 2 only
    assert oracle.visible(3, 2).tolist() == [[True, False, False], [True, True, False], [False, True, True]]
    assert oracle.visible(3).tolist() == [[True, False, False], [True, True, False], [True, True, True]]
    # router: scores s = sigmoid(z); groups (0,1,2) and (3,4,5) rank by their two largest; the second group wins with
    # 0.6 + 0.55 > 0.9 + 0.1 although the first holds the largest score; top 2 of it, weights normalised, times 3
    s = [0.9, 0.1, 0.05, 0.6, 0.55, 0.5]
    z = torch.tensor([math.log(v / (1 - v)) for v in s], dtype=F64)
    got = oracle.route(z, dict(top=2, scale=3.0, groups=dict(count=2, keep=1)))
    assert [e for e, _ in got] == [3, 4] and np.allclose([w for _, w in got], [3 * 0.6 / 1.15, 3 * 0.55 / 1.15])
    got = oracle.route(z, dict(top=2, scale=1.0, groups=dict(count=2, keep=2)))
    assert [e for e, _ in got] == [0, 3] and np.allclose([w for _, w in got], [0.9 / 1.5, 0.6 / 1.5])
    got = oracle.route(z, dict(top=1, scale=1.0))
    assert [e for e, _ in got] == [0] and np.allclose(got[0][1], 1.0)
    # two maps, one head, one token: both maps put all weight on the token's own value, o = (1 - lam) v, whose unit
    # RMS is sign(v) elementwise-scaled; times (1 - diff), times sigmoid(0) = 1/2
    m = dict(heads=1, kv_heads=1, dim=1, vdim=2, scale=1.0, diff=0.25, mask=dict(size=4))
    one, Z = torch.ones(1, 1, dtype=F64), torch.zeros(1, dtype=F64)
    W = {"q": torch.ones(2, 1, dtype=F64), "k": torch.ones(2, 1, dtype=F64), "v": torch.tensor([[3.0], [4.0]], dtype=F64),
         "lq1": Z, "lk1": Z, "lq2": Z, "lk2": Z, "g": torch.zeros(2, 1, dtype=F64), "o": torch.eye(2, dtype=F64)}
    o = oracle.differential_attention(one, W, m, 0.0)     # lam = 1 - 1 + 0.25, o = 0.75 (3, 4), rms = 0.75 sqrt(12.5)
    assert np.allclose(o.numpy(), [[0.5 * 0.75 * 3 / math.sqrt(12.5), 0.5 * 0.75 * 4 / math.sqrt(12.5)]])


@pytest.mark.parametrize("device", DEVICES)
def test_router_against_the_plain_choice(tmp_path, device):
    """The engine's routing (ids and weights it leaves behind) equals the plain choice, row by row, for several
    shapes: no groups, all groups kept, one group kept, groups of one, top 1, every expert chosen."""
    for i, f in enumerate([dc.moe(experts=6, top=3, count=1, keep=1), dc.moe(experts=8, top=3, count=4, keep=2, scale=0.5),
                           dc.moe(experts=10, top=2, count=2, keep=1, scale=1.5), dc.moe(experts=5, top=1, count=5, keep=2),
                           dc.moe(experts=4, top=4, count=2, keep=2), dc.moe(experts=70, top=5, count=7, keep=3)]):
        m = dc.Model(tmp_path, dc.config([(dc.diff(), f)], width=32, vocab=40), seed=20 + i, name=f"r{i}")
        toks = dc.tokens(40, 40, seed=i)
        r = m.runner(device)
        dc.check(dc.run_cuts(r, toks, [17, 40]), m.oracle(toks)[0], "float32", f"router shape {i}")
        z = r.proj[:23, :f.experts].double().cpu()   # the last step's router logits, ids and weights
        for b in (0, 5, 22):
            want = oracle.route(z[b], m.json["layers"][0]["mlp"]["router"])
            assert r.eids[b, :f.top].tolist() == [e for e, _ in want]
            assert np.allclose(r.ew[b, :f.top].cpu().numpy(), [w for _, w in want], rtol=1e-5)


# ------------------------------------------------------------------ each mechanism alone
MECHANISMS = {
    "two_maps": ([(dc.diff(), None)], {}),
    "two_maps_kv_head_each": ([(dc.diff(heads=3, kv_heads=3, dim=6, vdim=7, window=5), None)], {}),
    "two_maps_one_kv_head_wide_values": ([(dc.diff(heads=4, kv_heads=1, dim=12, vdim=70, lam=0.9, window=100), None)], {}),
    "two_maps_window_of_one": ([(dc.diff(heads=2, kv_heads=1, window=1), None)], {}),
    "two_maps_window_of_two": ([(dc.diff(heads=2, kv_heads=2, window=2), None)], {}),
    "mixed_scores": ([(dc.talk(), None)], {}),
    "mixed_scores_one_kv_head": ([(dc.talk(heads=3, kv_heads=1, dim=12, vdim=9, rot_dims=8, scaling=(), window=9), None)], {}),
    "mixed_scores_kv_head_each": ([(dc.talk(heads=3, kv_heads=3, dim=8, rot_dims=8, base=1e4, window=40), None)], {}),
    "mixed_scores_one_head": ([(dc.talk(heads=1, kv_heads=1, dim=10, rot_dims=4, window=3), None)], {}),
    "mixed_scores_no_rotation_no_window": ([(dc.talk(heads=4, kv_heads=2, dim=8, rot_dims=0, window=0), None)], {}),
    "latent": ([(dc.latent(), None)], {}),
    "latent_one_head_partly_rotated": ([(dc.latent(heads=1, dim=5, rot_dim=8, vdim=7, kv_rank=9, rot_dims=4), None)], {}),
    "latent_unrotated_wide": ([(dc.latent(heads=4, dim=16, rot_dim=4, vdim=40, kv_rank=70, rot_dims=0), None)], {}),
    "dense_ff": ([(dc.diff(), dc.dense(33))], {}),
    "routed_ff": ([(dc.talk(), dc.moe())], {}),
    "routed_ff_top_one_no_groups": ([(dc.latent(), dc.moe(experts=5, top=1, count=1, keep=1, scale=0.5))], {}),
    "span_from_the_start_three_times": ([(dc.diff(), dc.dense()), (dc.talk(), None)], dict(loop=(0, 2, 3))),
    "span_of_one_layer_at_the_end": ([(dc.latent(), None), (dc.diff(), dc.moe())], dict(loop=(1, 2, 2))),
    "span_that_runs_once": ([(dc.talk(), dc.dense()), (dc.latent(), None)], dict(loop=(0, 1, 1))),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_mechanism_alone(tmp_path, device, name):
    layers, kw = MECHANISMS[name]
    m = dc.Model(tmp_path, dc.config(layers, width=48, vocab=64, **kw), seed=11)
    toks = dc.tokens(45, 64, seed=1)
    want, trail = m.oracle(toks)
    r = m.runner(device)
    got_trail = dc.layer_trail(r, toks)
    assert got_trail.shape == trail.shape
    assert np.abs(got_trail - trail).max() < 1e-4 * max(1.0, np.abs(trail).max()), "residual after the layer"
    dc.check(dc.run_cuts(r, toks, [len(toks)]), want, "float32", name)
    dc.check(dc.run_cuts(r, toks, [20, 21, 23, 45]), want, "float32", name + " in portions")


# ------------------------------------------------------------------ whole prompts, decoding, portions
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_whole_prompt_and_layers(std, device, dtype):
    toks = dc.tokens(60, 96, seed=2)
    want, trail = std.oracle(toks)
    r = std.runner(device, dtype)
    got_trail = dc.layer_trail(r, toks)
    for i in range(trail.shape[0]):
        d = got_trail[i] - trail[i]
        if dtype == "float32":
            assert np.abs(d).max() < 1e-4 * max(1.0, np.abs(trail[i]).max()), f"residual after layer run {i}"
        else:   # rounding, and a router's close call in a row or two: by the typical row
            e = np.sqrt((d ** 2).mean(-1)) / np.sqrt((trail[i] ** 2).mean(-1))
            assert np.median(e) < 0.03 and e.max() < 0.5, f"residual after layer run {i}"
    dc.check(dc.run_cuts(r, toks, [len(toks)]), want, dtype, "whole prompt")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_prefill_then_token_by_token(std, device, dtype):
    toks = dc.tokens(80, 96, seed=4)
    want, _ = std.oracle(toks)
    r = std.runner(device, dtype)
    dc.check(dc.run_cuts(r, toks, [40] + list(range(41, 81))), want, dtype, "prefill 40, then one by one")


@pytest.mark.parametrize("device", DEVICES)
def test_every_token_alone_from_the_start(std, device):
    toks = dc.tokens(37, 96, seed=5)
    dc.check(dc.run_cuts(std.runner(device), toks, list(range(1, 38))), std.oracle(toks)[0], "float32", "one by one from 0")


@pytest.mark.parametrize("device", DEVICES)
def test_portions_of_many_sizes(std, device):
    """Portions of 2, 3, 1, 17, ... tokens across block borders (16), tile borders (32) and the windows' edges (7, 11,
    13, 30); more rows than one forward holds (max_batch 32), so a portion is also cut by the engine."""
    toks = dc.tokens(150, 96, seed=6)
    want, _ = std.oracle(toks)
    r = std.runner(device, max_batch=32)
    cuts = [2, 5, 6, 8, 10, 27, 31, 32, 33, 35, 64, 66, 127, 129, 131, 150]
    dc.check(dc.run_cuts(r, toks, cuts), want, "float32", "portions")
    r = std.runner(device, max_batch=128)
    dc.check(dc.run_cuts(r, toks, [1, 3, 34, 35, 99, 150]), want, "float32", "portions over several tiles")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_mixed_batch_equals_each_alone(std, device, dtype):
    """Five requests on four slots and a ten-block pool: portions of some beside single tokens of others, one
    sitting out a step, one ending early and its slot and blocks taken by a newcomer."""
    V = 96
    reqs = {k: dc.tokens(n, V, seed=30 + i) for i, (k, n) in enumerate([("a", 50), ("b", 7), ("c", 33), ("d", 21), ("e", 40)])}
    want = {k: std.oracle(t)[0] for k, t in reqs.items()}
    r = std.runner(device, dtype, kv_tokens=160, max_seqs=4)
    plan = [[("a", 20), ("b", 2)], [("a", 1), ("b", 5), ("c", 17)], [("a", 1), ("c", 1), ("d", 16)],
            [("c", 15), ("d", 5)], [("a", 28), ("e", 3)], [("e", 30)], [("e", 1)], [("e", 6)]]
    at = {k: 0 for k in reqs}
    sid, got = {}, {k: [] for k in reqs}
    for step in plan:
        entries = []
        for k, n in step:
            if k not in sid:
                sid[k] = r.new_sequence()
            entries.append((sid[k], reqs[k][at[k]:at[k] + n], list(range(n))))
        out = r.step_entries(entries).float().cpu().numpy()
        o = 0
        for k, n in step:
            got[k].append(out[o:o + n])
            o += n
            at[k] += n
            if at[k] == len(reqs[k]):
                r.free_sequence(sid.pop(k))
    assert all(at[k] == len(reqs[k]) for k in reqs)
    for k in reqs:
        dc.check(np.concatenate(got[k]), want[k], dtype, f"request {k} in the mixed batch")


@pytest.mark.parametrize("device", DEVICES)
def test_freed_blocks_and_slots_are_clean(std, device):
    """One slot and a pool for one request: the next request gets the previous one's blocks and must see nothing of
    them (a window that reached past the start of a sequence would)."""
    r = std.runner(device, kv_tokens=64, max_seqs=1)
    for seed in (40, 41, 42):
        toks = dc.tokens(60, 96, seed=seed)
        dc.check(dc.run_cuts(r, toks, [33, 34, 60]), std.oracle(toks)[0], "float32", f"request {seed} on reused blocks")
    assert r.kv.alloc.n_free == r.kv.alloc.n_blocks and len(r.kv.rows_free) == 1


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(std, device):
    for n in (1, 2, 3):
        toks = dc.tokens(n, 96, seed=50 + n)
        dc.check(dc.run_cuts(std.runner(device), toks, [n]), std.oracle(toks)[0], "float32", f"{n} token prompt")


# ------------------------------------------------------------------ far keys, window edges
@pytest.mark.parametrize("device", DEVICES)
def test_sharp_attention_at_borders(tmp_path, device):
    """Sharp attention (large score scales): most queries put their weight on ONE key, often the oldest the window
    still holds or, in the latent layer, one far back, so a lost or misplaced cache row or a window one token off
    shows. The mixing matrix has large off-diagonal and negative entries and the heads' factors differ. Portions
    and single tokens end just before, at and just after block and tile borders and the windows' edges."""
    layers = [(dc.diff(heads=4, kv_heads=2, dim=16, vdim=16, scale=1.5, window=37), None),
              (dc.talk(heads=4, kv_heads=2, dim=16, vdim=16, scale=0.9, rot_dims=12, base=1e4, scaling=(), window=50), dc.dense()),
              (dc.latent(heads=2, dim=16, rot_dim=8, vdim=16, kv_rank=24, scale=1.2, base=1e4), None)]
    m = dc.Model(tmp_path, dc.config(layers, width=64, vocab=80), seed=5)
    m.set_tensor("l1.mix.talk", torch.tensor([[1.0, -0.8, 0.5, 0.0], [0.7, 0.2, 0.0, -1.0], [0.0, 1.5, 1.0, 0.3], [-0.5, 0.0, 0.9, 1.0]]))
    m.set_tensor("l1.mix.temp", torch.tensor([1.5, 0.5, 1.0, -1.0]))
    toks = dc.tokens(300, 80, seed=6)
    want, _ = m.oracle(toks)
    plain = {**m.tensors, "l1.mix.talk": torch.eye(4)}
    assert dc.rel_err(oracle.forward(m.json, plain, toks)[0].numpy(), want).max() > 0.05, "the mixing must matter here"
    for layer, w in ((0, 36), (0, 38), (1, 49), (1, 51)):   # a window one token off must show in the logits
        c = json.loads(json.dumps(m.json))
        c["layers"][layer]["mixer"]["mask"]["size"] = w
        assert dc.rel_err(oracle.forward(c, m.tensors, toks)[0].numpy(), want).max() > 0.05, "the windows' edges must matter here"
    r = m.runner(device, max_batch=128, kv_tokens=320)
    cuts = [15, 16, 17, 31, 33, 36, 37, 38, 47, 48, 49, 50, 51, 200, 255, 256, 257, 271, 272, 273] + list(range(274, 301))
    dc.check(dc.run_cuts(r, toks, cuts), want, "float32", "sharp attention")
    dc.check(dc.run_cuts(r, toks, [300]), want, "float32", "sharp attention, whole")


def _pointing_query(T, pre, h_key, h_query, rows, gain):
    """A query matrix whose query for input h_query is gain * (the key of input h_key) in every one of `rows` / len(key)
    heads (or maps)."""
    ka = T[pre + "k"] @ h_key
    reps = rows // ka.numel()
    return (gain * ka[:, None] * h_query[None, :] / (h_query @ h_query)).repeat(reps, 1)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kind", ["two_maps", "mixed_scores"])
@pytest.mark.parametrize("where", ["inside", "outside"])
def test_one_key_at_the_windows_edge(tmp_path, device, kind, where):
    """The last token's query points along the key of ONE earlier token (queries and keys depend on the token alone
    here: no rotation, one layer), which sits either at the oldest position the window still holds or one before it.
    Inside, nearly all the weight lands on it; outside it must not be seen at all. Decoded alone and as the last
    row of a prompt portion that starts before the window."""
    window = 41
    if kind == "two_maps":
        mx = dc.diff(heads=2, kv_heads=1, dim=16, vdim=16, scale=1.0, lam=0.3, window=window)
    else:
        mx = dc.talk(heads=2, kv_heads=1, dim=16, vdim=16, scale=1.0, rot_dims=0, window=window)
    m = dc.Model(tmp_path, dc.config([(mx, None)], width=32, vocab=50), seed=9)
    A, B = 7, 11
    T = {k: v.double() for k, v in m.tensors.items()}
    ha = oracle.rms_norm(T["embed"][A], T["l0.norm1"], 1e-5)
    hb = oracle.rms_norm(T["embed"][B], T["l0.norm1"], 1e-5)
    if kind == "two_maps":   # map 1 of both heads asks for A's first key map; map 2 stays as drawn
        Wq = T["l0.mix.q"].clone().view(2, 2, 16, 32)
        Wq[:, 0] = 3.0 * (T["l0.mix.k"] @ ha)[:16, None] * hb[None, :] / (hb @ hb)
        m.set_tensor("l0.mix.q", Wq.reshape(64, 32).float())
    else:
        m.set_tensor("l0.mix.q", _pointing_query(T, "l0.mix.", ha, hb, 32, 3.0).float())
        m.set_tensor("l0.mix.talk", torch.tensor([[1.0, 0.3], [0.2, 1.0]]))
        m.set_tensor("l0.mix.temp", torch.tensor([1.0, 1.2]))
    body = [t for t in dc.tokens(400, 49, seed=8) if t not in (A, B)]
    n = 200
    back = window - 1 if where == "inside" else window
    toks = body[:n - 1 - back] + [A] + body[n - 1 - back:n - 2] + [B]
    assert len(toks) == n and toks[n - 1 - back] == A
    want, _ = m.oracle(toks)
    without = m.oracle(toks[:n - 1 - back] + [body[300]] + toks[n - back:])[0][-1]
    if where == "inside":
        assert dc.rel_err(want[-1], without) > 0.2, "the key at the edge must matter in this construction"
    else:
        assert dc.rel_err(want[-1], without) < 1e-9, "a key outside the window must not matter"
        moved = m.oracle([body[301]] + toks[:n - back] + toks[n - back + 1:])[0][-1]   # the same key one step nearer
        assert dc.rel_err(want[-1], moved) > 0.2, "one step nearer it must"
    r = m.runner(device, max_batch=64, kv_tokens=256)
    dc.check(dc.run_cuts(r, toks, [n - 1, n])[-1:], want[-1:], "float32", "decoded token at the window's edge")
    dc.check(dc.run_cuts(r, toks, [100, n])[-1:], want[-1:], "float32", "prompt portion at the window's edge")
    dc.check(dc.run_cuts(r, toks, [n - 2, n])[-1:], want[-1:], "float32", "portion of two tokens at the window's edge")


@pytest.mark.parametrize("device", DEVICES)
def test_latent_attention_finds_the_first_token(tmp_path, device):
    """All the weight of the last token on the FIRST token, 251 positions back: the rotated part is switched off
    (rot.dims 0, its query rows zero), so query and key depend on the token alone; the query is rebuilt so that, seen
    through W_uk, it points along the first token's latent."""
    mx = dc.latent(heads=2, dim=8, rot_dim=4, vdim=12, kv_rank=16, scale=1.0, rot_dims=0)
    m = dc.Model(tmp_path, dc.config([(mx, None)], width=32, vocab=50), seed=10)
    A, B = 7, 11
    T = {k: v.double() for k, v in m.tensors.items()}
    ha = oracle.rms_norm(T["embed"][A], T["l0.norm1"], 1e-5)
    hb = oracle.rms_norm(T["embed"][B], T["l0.norm1"], 1e-5)
    ca = oracle.rms_norm((T["l0.mix.dkv"] @ ha)[:16], T["l0.mix.dkv.norm"], 1e-5)
    ku = (T["l0.mix.uk"] @ ca).view(2, 8)                                   # A's unrotated keys
    Wq = torch.zeros(2, 12, 32, dtype=F64)
    Wq[:, :8] = 6.0 * ku[:, :, None] * hb[None, None, :] / (hb @ hb)
    m.set_tensor("l0.mix.q", Wq.reshape(24, 32).float())
    body = [t for t in dc.tokens(300, 49, seed=8) if t not in (A, B)][:250]
    toks = [A] + body + [B]
    want, _ = m.oracle(toks)
    without = m.oracle([body[0]] + body + [B])[0][-1]
    assert dc.rel_err(want[-1], without) > 0.2, "the far key must matter in this construction"
    r = m.runner(device, max_batch=64, kv_tokens=320)
    n = len(toks)
    dc.check(dc.run_cuts(r, toks, [n - 1, n])[-1:], want[-1:], "float32", "decoded token asking for a far key")
    dc.check(dc.run_cuts(r, toks, [100, n])[-1:], want[-1:], "float32", "prompt portion asking for a far key")


@pytest.mark.parametrize("device", DEVICES)
def test_long_context_decode(tmp_path, device):
    """Single tokens after 1300 cached rows: on a GPU the latent layer's decode attention then shares a row's keys
    among several blocks and merges their partial sums, the windowed layers beside it start 1200 keys in (one window
    wider than a split's share, one of a few keys); a long row beside short ones."""
    layers = [(dc.latent(heads=3, dim=8, rot_dim=8, vdim=12, kv_rank=16, scale=0.7, base=1e4), None),
              (dc.diff(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.5, window=1100), None),
              (dc.talk(heads=4, kv_heads=2, dim=16, vdim=8, scale=0.5, rot_dims=16, base=1e4, window=19), None)]
    m = dc.Model(tmp_path, dc.config(layers, width=32, vocab=60), seed=21)
    toks = dc.tokens(1306, 60, seed=22)
    want, _ = m.oracle(toks)
    r = m.runner(device, max_batch=512, kv_tokens=1400)
    got = dc.run_cuts(r, toks, [1300] + list(range(1301, 1307)))
    rows = list(range(1300, 1306))
    dc.check(got[rows], want[rows], "float32", "decoded after a long context")
    short = dc.tokens(9, 60, seed=23)
    ws = m.oracle(short)[0]
    a, b = r.new_sequence(), r.new_sequence()
    r.step_entries([(a, toks[:1200], []), (b, short[:5], [])])
    out = r.step_entries([(a, toks[1200:1201], [0]), (b, short[5:7], [0, 1])]).float().cpu().numpy()
    dc.check(out[:1], want[1200:1201], "float32", "long row of a mixed step")
    dc.check(out[1:], ws[5:7], "float32", "short rows of a mixed step")


# ------------------------------------------------------------------ other sizes
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_other_sizes(tmp_path, device, dtype):
    """A width, head sizes and hidden sizes that are not multiples of 8 (no vector loads), a vocabulary wider than a
    tile, an eps of its own, three query heads per key/value head, more groups than kept, a span in the middle."""
    layers = [(dc.diff(heads=6, kv_heads=2, dim=12, vdim=10, scale=0.4, lam=0.45, window=29), dc.dense(36)),
              (dc.talk(heads=6, kv_heads=3, dim=20, vdim=14, scale=0.2, rot_dims=10, window=23),
               dc.moe(experts=9, top=2, ff=20, count=3, keep=1)),
              (dc.latent(heads=5, dim=6, rot_dim=10, vdim=14, kv_rank=22, scale=0.3),
               dc.moe(experts=10, top=5, ff=12, count=5, keep=3)),
              (dc.talk(heads=5, kv_heads=5, dim=6, vdim=6, scale=0.5, rot_dims=2, scaling=(), window=64), dc.dense(12))]
    m = dc.Model(tmp_path, dc.config(layers, width=52, vocab=300, eps=1e-3, loop=(1, 3, 2)), seed=17)
    toks = dc.tokens(90, 300, seed=18)
    want, _ = m.oracle(toks)
    r = m.runner(device, dtype, max_batch=128)
    dc.check(dc.run_cuts(r, toks, [70, 71, 72, 90]), want, dtype, "odd sizes")


@pytest.mark.parametrize("device", DEVICES)
def test_wide_key_rows(tmp_path, device):
    """Key rows wider than 256: a latent row of 200 + 120, a shared key row of 4 x 80 and of 8 x 64, maps of 72; only the
    kernel with one block per (row, head) holds such a query, also for a prompt portion of many rows."""
    layers = [(dc.latent(heads=2, dim=24, rot_dim=120, vdim=16, kv_rank=200, scale=0.1, base=1e4), None),
              (dc.talk(heads=4, kv_heads=4, dim=80, vdim=24, scale=0.1, rot_dims=40, base=1e4, window=90), dc.dense()),
              (dc.talk(heads=8, kv_heads=8, dim=64, vdim=8, scale=0.1, rot_dims=64, base=1e3, scaling=(), window=33), None),
              (dc.diff(heads=2, kv_heads=1, dim=72, vdim=40, scale=0.1, window=100), None)]
    m = dc.Model(tmp_path, dc.config(layers, width=64, vocab=80), seed=27)
    toks = dc.tokens(300, 80, seed=28)
    want, _ = m.oracle(toks)
    r = m.runner(device, max_batch=512, kv_tokens=320)
    dc.check(dc.run_cuts(r, toks, [280] + list(range(281, 301)))[250:], want[250:], "float32", "wide key rows")


@pytest.mark.parametrize("device", DEVICES)
def test_matrix_core_sizes(tmp_path, device):
    """Sizes the matrix-core products and vector loads take (map sizes 32 and 64, shared key rows of 192 and 256, a
    latent row of 160), in both dtypes; a prompt portion over several tiles and windows, then single tokens."""
    layers = [(dc.diff(heads=6, kv_heads=2, dim=32, vdim=64, scale=0.15, window=70), dc.moe(experts=12, top=3, ff=64, count=3, keep=2)),
              (dc.talk(heads=6, kv_heads=3, dim=64, vdim=64, scale=0.12, rot_dims=48, base=1e5, window=45), dc.dense(256)),
              (dc.latent(heads=3, dim=32, rot_dim=32, vdim=48, kv_rank=128, scale=0.1, base=1e4),
               dc.moe(experts=8, top=3, ff=128, count=4, keep=2)),
              (dc.diff(heads=2, kv_heads=1, dim=64, vdim=128, scale=0.1, window=33), None),
              (dc.talk(heads=4, kv_heads=4, dim=64, vdim=64, scale=0.1, rot_dims=32, base=1e4, scaling=(), window=100), None)]
    m = dc.Model(tmp_path, dc.config(layers, width=128, vocab=256), seed=19)
    toks = dc.tokens(200, 256, seed=20)
    want, _ = m.oracle(toks)
    for dtype in BOTH:
        r = m.runner(device, dtype, max_batch=256)
        dc.check(dc.run_cuts(r, toks, [190] + list(range(191, 201))), want, dtype, "matrix-core sizes")
        dc.check(dc.run_cuts(r, toks, [45, 130, 200])[120:], want[120:], dtype, "matrix-core sizes, a portion from the middle")


# ------------------------------------------------------------------ generation through the engine's entry points
def greedy_oracle(m, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(np.argmax(m.oracle(toks)[0][-1])))
    return toks[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generate_and_long_decode(std, device):
    """`Runner.generate` (prefill, the on-device sampler, the decode graph on a GPU) produces the oracle's greedy
    continuation over several block borders and past every window; the next turn extends the cached sequence, a
    prompt that shares only a part is cut back to it (no layer carries a state)."""
    prompt = dc.tokens(12, 96, seed=60)
    want = greedy_oracle(std, prompt, 40)
    r = std.runner(device, use_graphs=None)
    sid = r.new_sequence()
    got = list(r.generate(sid, prompt, GREEDY, max_tokens=40))
    assert got == want
    more = list(r.generate(sid, prompt + got + [5, 6], GREEDY, max_tokens=4))
    assert more == greedy_oracle(std, prompt + got + [5, 6], 4)
    other = prompt[:6] + [1, 2, 3]
    assert list(r.generate(sid, other, GREEDY, max_tokens=3)) == greedy_oracle(std, other, 3)


@pytest.mark.parametrize("device", DEVICES)
def test_scheduler_batches_requests(std, device):
    r = std.runner(device, max_seqs=5, kv_tokens=1024, use_graphs=None)
    sch = BatchScheduler(r, max_parallel=3)
    try:
        prompts = [dc.tokens(n, 96, seed=70 + i) for i, n in enumerate((9, 20, 14))]
        lens = (12, 5, 9)
        its = [sch.submit(p, GREEDY, max_tokens=k) for p, k in zip(prompts, lens)]
        got = [list(it) for it in its]
        for p, k, g in zip(prompts, lens, got):
            assert g == greedy_oracle(std, p, k)
    finally:
        sch.close()


def test_command_line_generates_token_ids(std, capsys):
    from ollama_operator_amd import cli
    prompt = dc.tokens(9, 96, seed=90)
    cli.main(["tokens", std.path, "--ids", " ".join(map(str, prompt)), "--num-predict", "5", "--device", "cpu",
              "--dtype", "float32"])
    out = capsys.readouterr().out.strip().splitlines()[-1]
    assert [int(t) for t in out.split()] == greedy_oracle(std, prompt, 5)


def test_trace_replay_program(std, tmp_path):
    """bin/trace_run on the CPU twin: a request that sits out a step, one that ends and gives its slot back."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    a, b = dc.tokens(30, 96, seed=91), dc.tokens(12, 96, seed=92)
    steps = [dict(step=0, entries=[dict(id="a", tokens=a[:20], want=[0, 19])], end=[]),
             dict(step=1, entries=[dict(id="b", tokens=b, want=[11])], end=["b"]),
             dict(step=2, entries=[dict(id="a", tokens=a[20:], want=[9]), dict(id="c", tokens=b[:2], want=[])], end=["a", "c"])]
    out = tmp_path / "out"
    p = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", std.path, "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "64", "--device", "cpu"], input="".join(json.dumps(x) + "\n" for x in steps),
                       capture_output=True, text=True, timeout=300, env={**os.environ, "PYTHON": sys.executable})
    assert p.returncode == 0, p.stderr[-2000:]
    assert [ln for ln in p.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(3)]
    wa, wb = std.oracle(a)[0], std.oracle(b)[0]
    dc.check(np.fromfile(out / "0.f32", "<f4").reshape(2, 96), wa[[0, 19]], "float32", "step 0")
    dc.check(np.fromfile(out / "1.f32", "<f4").reshape(1, 96), wb[[11]], "float32", "step 1")
    dc.check(np.fromfile(out / "2.f32", "<f4").reshape(1, 96), wa[[29]], "float32", "step 2")


# ------------------------------------------------------------------ the HIP executor against its twin
@pytest.mark.gpu
def test_gpu_matches_twin_layer_by_layer(std):
    toks = dc.tokens(50, 96, seed=95)
    for dtype, tol in (("float32", 1e-4), ("bfloat16", 0.05)):
        a = dc.layer_trail(std.runner("cpu", dtype), toks)
        b = dc.layer_trail(std.runner("cuda", dtype), toks)
        for i in range(a.shape[0]):
            assert np.abs(a[i] - b[i]).max() < tol * max(1.0, np.abs(a[i]).max()), f"{dtype}: layer run {i}"


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [0, 1, 2, 3, 4, 5])
def test_random_configurations(tmp_path, seed):
    """Configurations drawn at the scale of a small real model, 700-token prompts in portions and whole: float32
    sharply. In bfloat16 a drawn model may double its rounding error with every layer run (one expert per token, a
    span that runs three times), so there the residual stream after the first three layer runs is compared by the
    typical row: the matrix-core attention, the grouped experts and the tile products all run by then."""
    rng = random.Random(2000 + seed)
    cfg = dc.random_config(rng)
    m = dc.Model(tmp_path, cfg, seed=seed)
    toks = dc.tokens(700, cfg.n_vocab, seed=seed)
    want, trail = m.oracle(toks)
    rows = sorted(set(rng.sample(range(700), 40)) | {699})
    r = m.runner("cuda", "float32", max_batch=512, kv_tokens=1024)
    sid = r.new_sequence()
    cuts, got, a = [rng.randint(1, 300), rng.randint(301, 600), 690] + list(range(691, 701)), [], 0
    for b in cuts:
        want_rows = [i - a for i in rows if a <= i < b]
        got.append(r.step_entries([(sid, toks[a:b], want_rows)]).float().cpu().numpy())
        a = b
    r.free_sequence(sid)
    dc.check(np.concatenate(got), want[rows], "float32", f"random configuration {seed}")
    r = m.runner("cuda", "bfloat16", max_batch=512, kv_tokens=1024)
    got_trail = dc.layer_trail(r, toks[:500])
    assert np.isfinite(got_trail).all()
    for i in range(min(3, trail.shape[0])):
        d = got_trail[i] - trail[i][:500]
        e = np.sqrt((d ** 2).mean(-1)) / np.sqrt((trail[i][:500] ** 2).mean(-1))
        assert np.median(e) < 0.03, f"random configuration {seed}: residual after layer run {i}, typical row off by {np.median(e):.3g}"
