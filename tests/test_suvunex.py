"""The Suvunex design in the layer-list engine against its plain float64 implementation (suvunex_oracle.py):
every mechanism alone, prefill against token-by-token decoding, portions, mixed batches, reused blocks and
slots, far keys, sinks, chunk and tile borders, long decoding, other sizes, generation through the engine's own
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

import suvunex_cases as sc
import suvunex_oracle as oracle
from ollama_operator_amd.engine.sampling import SamplingOptions
from ollama_operator_amd.engine.scheduler import BatchScheduler
from ollama_operator_amd.models.config import StackConfig, UnsupportedArchitecture, load_stack_config, rotary_inv_freq

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
BOTH = ["float32", "bfloat16"]
GREEDY = SamplingOptions(temperature=0.0, repeat_penalty=1.0)


@pytest.fixture(scope="module")
def std(tmp_path_factory):
    return sc.Model(tmp_path_factory.mktemp("suvunex"), sc.standard(), seed=3)


def no_rank(cfg):
    """The inner size of the decay map is a tensor's shape, not a config entry: leave it out of comparisons."""
    for s in cfg.layers:
        if s.mixer.right is not None:
            s.mixer.right.decay_rank = 0
    return cfg


# ------------------------------------------------------------------ configuration
def test_config_roundtrip(std):
    cfg = load_stack_config(std.path)
    assert cfg == no_rank(sc.standard()) and cfg.has_state and cfg.canon_taps == 3 and cfg.logit_scale == 0.5
    assert StackConfig.from_suvunex(cfg.to_suvunex()) == cfg
    # state per run: the second mixer's matrix, then the input window
    assert [cfg.run_state_floats(i) for i in range(3)] == [2 * 8 * 12 + 2 * 64, 2 * 64, 3 * 4 * 8 + 2 * 64]
    assert std.runner("cpu").w.cfg.layers[0].mixer.right.decay_rank == 5


def test_bench_configurations_are_readable():
    """The sizes `bench.py --stack ... --suvunex` measures are valid configurations of the design."""
    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    import bench
    for z in bench.SUVUNEX_SIZES.values():
        cfg = bench.suvunex_config(z)
        assert no_rank(StackConfig.from_suvunex(cfg.to_suvunex())) == no_rank(cfg)
        assert len(cfg.layers) == 8 and cfg.has_state and sum(s.mixer.talk for s in cfg.layers) == 2


def test_unknown_parts_are_refused():
    c = sc.standard().to_suvunex()
    for path, val in ((("layers", 0, "type"), "conv_mixer"), (("layers", 0, "mlp", "kind"), "moe"),
                      (("layers", 1, "mixer", "vdim"), 20), (("layers", 0, "mixer", "left", "rot", "dims"), 7),
                      (("canon", "taps"), 0)):
        d = json.loads(json.dumps(c))
        node = d
        for k in path[:-1]:
            node = node[k]
        node[path[-1]] = val
        with pytest.raises(UnsupportedArchitecture):
            StackConfig.from_suvunex(d)


def test_frequency_scaling_by_hand():
    """Bands with original 64, low 1, high 5: waves shorter than 12.8 keep their frequency, longer than 64 are divided
    by the factor, and a wave of 32 would sit at s = (64 / 32 - 1) / 4 = 1/4."""
    f = rotary_inv_freq(8, 100.0, ("bands", 6.0, 1.0, 5.0, 64.0))
    plain = [100.0 ** (-2 * i / 8) for i in range(4)]
    waves = [2 * math.pi / x for x in plain]                 # 6.3, 19.9, 62.8, 198.7
    assert waves[0] < 12.8 < waves[1] < waves[2] < 64 < waves[3]
    assert f[0] == plain[0] and f[3] == plain[3] / 6
    for i in (1, 2):
        s = (64 / waves[i] - 1) / 4
        assert abs(f[i] - ((1 - s) * plain[i] / 6 + s * plain[i])) < 1e-15
    rot = dict(dims=8, base=100.0, scaling=dict(factor=6.0, low=1.0, high=5.0, original=64))
    assert np.allclose(oracle.rotary_frequencies(rot).numpy(), f)
    assert rotary_inv_freq(8, 100.0, ("linear", 4.0)) == [x / 4 for x in plain]


# ------------------------------------------------------------------ each mechanism alone
MECHANISMS = {
    "pair": ([(sc.parallel(), None)], {}),
    "pair_no_rotation_one_kv_head": ([(sc.parallel(heads=3, kv_heads=1, dim=12, vdim=7, rot_dims=0), None)], {}),
    "pair_all_rotated_linear_scaling": ([(sc.parallel(heads=2, kv_heads=2, dim=8, vdim=8, rot_dims=8, scaling=("linear", 5.0)),
                                          None)], {}),
    "pair_one_head_each_wide_values": ([(sc.parallel(heads=1, kv_heads=1, dim=10, vdim=30, rot_dims=4, scaling=(),
                                                      right=sc.gla(heads=1, dim=6, vdim=40, tau=1.0, rank=2)), None)], {}),
    "pair_fast_decay_many_heads": ([(sc.parallel(right=sc.gla(heads=5, dim=4, vdim=4, tau=0.5, rank=7)), None)], {}),
    "pair_state_wider_than_the_registers": ([(sc.parallel(right=sc.gla(heads=1, dim=160, vdim=200, tau=8.0, rank=8)), None)], {}),
    "pair_scales_zero_left": ([(sc.parallel(left_scale=0.0, right_scale=2.0), None)], {}),
    "pair_scales_zero_right": ([(sc.parallel(left_scale=1.5, right_scale=0.0), None)], {}),
    "mixed_heads": ([(sc.talking(), None)], {}),
    "mixed_heads_one_kv_head": ([(sc.talking(heads=3, kv_heads=1, dim=12, rot_dims=8, scaling=()), None)], {}),
    "mixed_heads_kv_head_each": ([(sc.talking(heads=3, kv_heads=3, dim=8, rot_dims=0), None)], {}),
    "mixed_heads_bands": ([(sc.talking(heads=4, kv_heads=2, dim=16, rot_dims=16, base=100.0, scaling=sc.BANDS), None)], {}),
    "no_convolution": ([(sc.parallel(), None), (sc.talking(), None)], dict(taps=1)),
    "two_taps": ([(sc.parallel(), None), (sc.talking(), None)], dict(taps=2)),
    "five_taps": ([(sc.parallel(), None), (sc.talking(), None)], dict(taps=5)),
    "gated_ff": ([(sc.talking(), sc.glu())], {}),
    "gated_ff_after_pair": ([(sc.parallel(), sc.glu(17))], dict(logit_scale=3.0)),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_mechanism_alone(tmp_path, device, name):
    layers, kw = MECHANISMS[name]
    m = sc.Model(tmp_path, sc.config(layers, width=48, vocab=64, **kw), seed=11)
    toks = sc.tokens(45, 64, seed=1)
    want, trail = m.oracle(toks)
    r = m.runner(device)
    got_trail = sc.layer_trail(r, toks)
    assert np.abs(got_trail - trail).max() < 1e-4 * max(1.0, np.abs(trail).max()), "residual after the layer"
    sc.check(sc.run_cuts(r, toks, [len(toks)]), want, "float32", name)
    sc.check(sc.run_cuts(r, toks, [20, 21, 23, 45]), want, "float32", name + " in portions")


def test_oracle_mechanisms_by_hand():
    """The plain implementation on numbers worked out by hand."""
    F64 = torch.float64
    # input convolution, 3 taps: out_t = h_t + w0 h_(t-2) + w1 h_(t-1) + w2 h_t
    h = torch.tensor([[1.0], [2.0], [4.0]], dtype=F64)
    out = oracle.input_conv(h, torch.tensor([[0.5, -1.0, 0.25]], dtype=F64))
    assert np.allclose(out.numpy()[:, 0], [1 + 0.25, 2 - 1 + 0.5, 4 + 0.5 - 2 + 1])
    # the softmax with one more 1 in the denominator: a single key of score 0 gets weight 1/2
    m = dict(heads=1, kv_heads=1, dim=2, vdim=2, scale=1.0, rot=dict(dims=0, base=10.0))
    Z, I2 = torch.zeros(2, 2, dtype=F64), torch.eye(2, dtype=F64)
    W = {"q": Z, "q.b": torch.zeros(2, dtype=F64), "k": Z, "k.b": torch.zeros(2, dtype=F64), "v": I2, "v.b": torch.zeros(2, dtype=F64),
         "o": I2, "o.b": torch.zeros(2, dtype=F64)}
    o = oracle.softmax_plus_one_attention(torch.tensor([[2.0, 4.0], [6.0, 0.0]], dtype=F64), W, m, 1e-6)
    assert np.allclose(o.numpy(), [[1.0, 2.0], [8.0 / 3, 4.0 / 3]])
    # gated linear attention, one head, one channel: S_1 = k_1 v_1, S_2 = alpha_2 S_1 + k_2 v_2 with alpha = sigmoid(0)^(1/1)
    g = dict(heads=1, dim=1, vdim=1, tau=1.0)
    one = torch.ones(1, 1, dtype=F64)
    Wg = {"q": one, "k": one, "v": one, "g": one, "a1": torch.zeros(1, 1, dtype=F64), "a2": one, "a2.b": torch.zeros(1, dtype=F64),
          "norm": torch.ones(1, dtype=F64), "o": one}
    x = torch.tensor([[1.0], [3.0]], dtype=F64)
    y = oracle.gated_linear_attention(x, Wg, g, 0.0)
    # o_1 = 1 * 1 = 1, o_2 = (0.5 * 1 + 9) * 3 > 0: after the unit norm both are 1, times silu(x)
    assert np.allclose(y.numpy()[:, 0], [oracle.silu(x[0, 0]).item(), oracle.silu(x[1, 0]).item()])


# ------------------------------------------------------------------ whole prompts, decoding, portions
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_whole_prompt_and_layers(std, device, dtype):
    toks = sc.tokens(60, 96, seed=2)
    want, trail = std.oracle(toks)
    r = std.runner(device, dtype)
    got_trail = sc.layer_trail(r, toks)
    for i in range(trail.shape[0]):
        tol = 1e-4 if dtype == "float32" else 0.06
        assert np.abs(got_trail[i] - trail[i]).max() < tol * max(1.0, np.abs(trail[i]).max()), f"residual after layer {i}"
    sc.check(sc.run_cuts(r, toks, [len(toks)]), want, dtype, "whole prompt")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_prefill_then_token_by_token(std, device, dtype):
    toks = sc.tokens(80, 96, seed=4)
    want, _ = std.oracle(toks)
    r = std.runner(device, dtype)
    sc.check(sc.run_cuts(r, toks, [40] + list(range(41, 81))), want, dtype, "prefill 40, then one by one")


@pytest.mark.parametrize("device", DEVICES)
def test_every_token_alone_from_the_start(std, device):
    toks = sc.tokens(37, 96, seed=5)
    sc.check(sc.run_cuts(std.runner(device), toks, list(range(1, 38))), std.oracle(toks)[0], "float32", "one by one from 0")


@pytest.mark.parametrize("device", DEVICES)
def test_portions_of_many_sizes(std, device):
    """Portions of 2, 3, 1, 17, ... tokens across block borders (16), chunk and tile borders (32) and shorter than
    the convolution's window; more rows than one forward holds (max_batch 32), so a portion is also cut by the engine."""
    toks = sc.tokens(150, 96, seed=6)
    want, _ = std.oracle(toks)
    r = std.runner(device, max_batch=32)
    cuts = [2, 5, 6, 8, 10, 27, 31, 32, 33, 35, 64, 66, 127, 129, 131, 150]
    sc.check(sc.run_cuts(r, toks, cuts), want, "float32", "portions")
    r = std.runner(device, max_batch=128)
    sc.check(sc.run_cuts(r, toks, [1, 3, 34, 35, 99, 150]), want, "float32", "portions over several chunks")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_mixed_batch_equals_each_alone(std, device, dtype):
    """Five requests on four slots and a ten-block pool: portions of some beside single tokens of others, one
    sitting out a step, one ending early and its slot and blocks taken by a newcomer."""
    V = 96
    reqs = {k: sc.tokens(n, V, seed=30 + i) for i, (k, n) in enumerate([("a", 50), ("b", 7), ("c", 33), ("d", 21), ("e", 40)])}
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
        sc.check(np.concatenate(got[k]), want[k], dtype, f"request {k} in the mixed batch")


@pytest.mark.parametrize("device", DEVICES)
def test_freed_blocks_and_slots_are_clean(std, device):
    """One slot and a pool for one request: the next request gets the previous one's blocks, state matrices and
    convolution windows and must see nothing of them."""
    r = std.runner(device, kv_tokens=64, max_seqs=1)
    for seed in (40, 41, 42):
        toks = sc.tokens(60, 96, seed=seed)
        sc.check(sc.run_cuts(r, toks, [33, 34, 60]), std.oracle(toks)[0], "float32", f"request {seed} on reused blocks")
    assert r.kv.alloc.n_free == r.kv.alloc.n_blocks and len(r.kv.rows_free) == 1


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(std, device):
    for n in (1, 2, 3):
        toks = sc.tokens(n, 96, seed=50 + n)
        sc.check(sc.run_cuts(std.runner(device), toks, [n]), std.oracle(toks)[0], "float32", f"{n} token prompt")


# ------------------------------------------------------------------ far keys, sinks, decays
@pytest.mark.parametrize("device", DEVICES)
def test_far_keys_block_borders_and_sinks(tmp_path, device):
    """Sharp attention (large score scales): most queries put their weight on ONE key, often far back, so a lost or
    misplaced cache row shows. In the mixed-heads layer one head's sink is huge (it takes most of the denominator),
    one is negligible, the others are of the size of the scores, and the mixing matrix has large off-diagonal and
    negative entries. Portions and single tokens end just before, at and just after block, tile and chunk borders."""
    layers = [(sc.parallel(heads=4, kv_heads=2, dim=16, vdim=16, scale=1.2, rot_dims=8, base=30.0), None),
              (sc.talking(heads=4, kv_heads=2, dim=16, scale=0.8, rot_dims=12, base=1e4), sc.glu())]
    m = sc.Model(tmp_path, sc.config(layers, width=64, vocab=80), seed=5)
    m.set_tensor("l1.mix.sink", torch.tensor([30.0, -40.0, 6.0, 2.0]))
    m.set_tensor("l1.mix.talk", torch.tensor([[1.0, -0.8, 0.5, 0.0], [0.7, 0.2, 0.0, -1.0], [0.0, 1.5, 1.0, 0.3], [-0.5, 0.0, 0.9, 1.0]]))
    toks = sc.tokens(300, 80, seed=6)
    want, _ = m.oracle(toks)
    no_sink = {**m.tensors, "l1.mix.sink": torch.full((4,), -1e4)}
    assert sc.rel_err(oracle.forward(m.json, no_sink, toks)[0].numpy(), want).max() > 0.05, "the sinks must matter here"
    plain = {**m.tensors, "l1.mix.talk": torch.eye(4)}
    assert sc.rel_err(oracle.forward(m.json, plain, toks)[0].numpy(), want).max() > 0.05, "the mixing must matter here"
    r = m.runner(device, max_batch=128, kv_tokens=320)
    cuts = [15, 16, 17, 31, 33, 47, 48, 49, 200, 255, 256, 257, 271, 272, 273] + list(range(274, 301))
    sc.check(sc.run_cuts(r, toks, cuts), want, "float32", "far keys")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kind", ["pair", "mixed_heads"])
def test_one_key_stands_out(tmp_path, device, kind):
    """All the weight on the FIRST token, 251 positions back. Without rotation and without the input convolution a
    token's query and key depend on the token alone; the query matrix is rebuilt so that the last token's query
    points along the first token's key in every head, which after the norms is the largest score there can be. A
    cache that lost that row answers with other keys; a lost sink changes the weight that is left for it."""
    if kind == "pair":
        mx = sc.parallel(heads=2, kv_heads=1, dim=16, vdim=16, scale=1.0, rot_dims=0, right_scale=0.05)
        pre = "l0.mix.left."
    else:
        mx = sc.talking(heads=2, kv_heads=1, dim=16, scale=1.0, rot_dims=0)
        pre = "l0.mix."
    m = sc.Model(tmp_path, sc.config([(mx, None)], width=32, vocab=50, embed_scale=1.0, taps=1), seed=9)
    A, B = 7, 11
    T = {k: v.double() for k, v in m.tensors.items()}
    ha = oracle.scalar_norm(T["embed"][A], T["l0.norm1"], 1e-5)
    hb = oracle.scalar_norm(T["embed"][B], T["l0.norm1"], 1e-5)
    ka = T[pre + "k"] @ ha + T[pre + "k.b"]                    # token A's key before its norm (one key/value head)
    Wq = (4.0 * ka[:, None] * hb[None, :] / (hb @ hb)).repeat(2, 1)   # q(B) = 4 k_A in both heads
    m.set_tensor(pre + "q", Wq.float())
    m.set_tensor(pre + "q.b", torch.zeros(32))
    if kind == "mixed_heads":   # equal norm weights keep the directions parallel
        m.set_tensor(pre + "q.norm", torch.ones(16))
        m.set_tensor(pre + "k.norm", torch.ones(16))
        m.set_tensor(pre + "sink", torch.tensor([10.0, 14.0]))
    body = [t for t in sc.tokens(300, 49, seed=8) if t not in (A, B)][:250]
    toks = [A] + body + [B]
    want, _ = m.oracle(toks)
    without = m.oracle([body[0]] + body + [B])[0][-1]
    assert sc.rel_err(want[-1], without) > 0.2, "the far key must matter in this construction"
    r = m.runner(device, max_batch=64, kv_tokens=320)
    n = len(toks)
    sc.check(sc.run_cuts(r, toks, [n - 1, n])[-1:], want[-1:], "float32", "decoded token asking for a far key")
    sc.check(sc.run_cuts(r, toks, [100, n])[-1:], want[-1:], "float32", "prompt portion asking for a far key")


@pytest.mark.parametrize("device", DEVICES)
def test_long_context_decode(tmp_path, device):
    """Single tokens after 1300 cached rows: on a GPU the decode attention then shares a row's keys among several
    blocks and merges their partial sums (the sink joins once, after the merge, also for the pairs of query and
    value heads that the mixing needs); a long row beside short ones."""
    layers = [(sc.talking(heads=4, kv_heads=2, dim=16, scale=0.6, rot_dims=16, base=1e4), None),
              (sc.parallel(heads=4, kv_heads=1, dim=16, vdim=24, scale=0.5, rot_dims=8, base=1e4), None)]
    m = sc.Model(tmp_path, sc.config(layers, width=32, vocab=60), seed=21)
    m.set_tensor("l0.mix.sink", torch.tensor([8.0, 0.0, -30.0, 3.0]))
    toks = sc.tokens(1306, 60, seed=22)
    want, _ = m.oracle(toks)
    r = m.runner(device, max_batch=512, kv_tokens=1400)
    cuts = [1300] + list(range(1301, 1307))
    got = sc.run_cuts(r, toks, cuts)
    rows = list(range(1300, 1306))
    sc.check(got[rows], want[rows], "float32", "decoded after a long context")
    short = sc.tokens(9, 60, seed=23)
    ws = m.oracle(short)[0]
    a, b = r.new_sequence(), r.new_sequence()
    r.step_entries([(a, toks[:1200], []), (b, short[:5], [])])
    out = r.step_entries([(a, toks[1200:1201], [0]), (b, short[5:7], [0, 1])]).float().cpu().numpy()
    sc.check(out[:1], want[1200:1201], "float32", "long row of a mixed step")
    sc.check(out[1:], ws[5:7], "float32", "short rows of a mixed step")


@pytest.mark.parametrize("device", DEVICES)
def test_decays_from_gone_in_a_token_to_kept_for_thousands(tmp_path, device):
    """Key channels whose decay is 0.0003 per token beside channels that lose a thousandth in a thousand tokens, with
    tau of 1 and of 0.25 (a decay raised to the 4th power): 400 tokens in one portion (chunks whose running log
    decay reaches -250 per chunk), then single tokens; what the first token wrote must still be there."""
    layers = [(sc.parallel(heads=2, kv_heads=1, dim=8, vdim=8, left_scale=0.1, right_scale=1.5,
                           right=sc.gla(heads=2, dim=8, vdim=8, tau=1.0, rank=4)), None),
              (sc.parallel(heads=2, kv_heads=1, dim=8, vdim=8, left_scale=0.1, right_scale=1.5,
                           right=sc.gla(heads=1, dim=16, vdim=12, tau=0.25, rank=4)), None)]
    m = sc.Model(tmp_path, sc.config(layers, width=32, vocab=40), seed=13)
    m.set_tensor("l0.mix.right.a2.b", torch.tensor([-8.0, -3.0, 0.0, 2.0, 5.0, 9.0, 14.0, 14.0] * 2))
    m.set_tensor("l1.mix.right.a2.b", torch.linspace(-2.0, 16.0, 16))
    toks = sc.tokens(420, 40, seed=14)
    want, _ = m.oracle(toks)
    changed = m.oracle([(toks[0] + 1) % 40] + toks[1:])[0][-1]
    assert sc.rel_err(changed, want[-1]) > 1e-3, "the first token must still matter at the end"
    r = m.runner(device, max_batch=512, kv_tokens=512)
    sc.check(sc.run_cuts(r, toks, [400] + list(range(401, 421))), want, "float32", "long memories")
    r = m.runner(device, max_batch=64, kv_tokens=512)
    sc.check(sc.run_cuts(r, toks, [7, 100, 101, 420]), want, "float32", "long memories in portions")


# ------------------------------------------------------------------ other sizes
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_other_sizes(tmp_path, device, dtype):
    """A width, head sizes and a hidden size that are not multiples of 8 (no vector loads), a vocabulary wider than
    a tile, four taps, eps, embedding and logit scales of their own, more key/value heads than one."""
    layers = [(sc.parallel(heads=6, kv_heads=3, dim=12, vdim=10, scale=0.4, rot_dims=6,
                           right=sc.gla(heads=3, dim=10, vdim=6, tau=2.0, rank=3)), sc.glu(36)),
              (sc.talking(heads=6, kv_heads=3, dim=20, scale=0.2, rot_dims=10, scaling=sc.BANDS), sc.glu(20)),
              (sc.parallel(heads=2, kv_heads=2, dim=64, vdim=64, scale=0.1, rot_dims=32,
                           right=sc.gla(heads=2, dim=32, vdim=64, tau=8.0, rank=16)), None),
              (sc.talking(heads=5, kv_heads=5, dim=6, scale=0.5, rot_dims=2, scaling=()), sc.glu(12))]
    m = sc.Model(tmp_path, sc.config(layers, width=52, vocab=300, eps=1e-3, embed_scale=0.7, taps=4, logit_scale=1.7), seed=17)
    toks = sc.tokens(90, 300, seed=18)
    want, _ = m.oracle(toks)
    r = m.runner(device, dtype, max_batch=128)
    sc.check(sc.run_cuts(r, toks, [70, 71, 72, 90]), want, dtype, "odd sizes")


@pytest.mark.parametrize("device", DEVICES)
def test_matrix_core_sizes(tmp_path, device):
    """Sizes the matrix-core products and vector loads take (head sizes 64 / 96 / 128), in both dtypes; a prompt portion
    over several tiles and chunks, then single tokens."""
    layers = [(sc.parallel(heads=6, kv_heads=2, dim=96, vdim=96, scale=0.1, rot_dims=32, base=1e4,
                           right=sc.gla(heads=3, dim=32, vdim=64, tau=8.0, rank=8)), sc.glu(256)),
              (sc.talking(heads=6, kv_heads=3, dim=64, scale=0.11, rot_dims=48, base=1e5, scaling=("linear", 2.0)), sc.glu(128)),
              (sc.parallel(heads=2, kv_heads=2, dim=128, vdim=128, scale=0.09, rot_dims=64,
                           right=sc.gla(heads=2, dim=64, vdim=128, tau=4.0, rank=8)), None)]
    m = sc.Model(tmp_path, sc.config(layers, width=128, vocab=256), seed=19)
    toks = sc.tokens(200, 256, seed=20)
    want, _ = m.oracle(toks)
    for dtype in BOTH:
        r = m.runner(device, dtype, max_batch=256)
        sc.check(sc.run_cuts(r, toks, [190] + list(range(191, 201))), want, dtype, "matrix-core sizes")
        sc.check(sc.run_cuts(r, toks, [45, 130, 200])[120:], want[120:], dtype, "matrix-core sizes, a portion from the middle")


# ------------------------------------------------------------------ generation through the engine's entry points
def greedy_oracle(m, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(np.argmax(m.oracle(toks)[0][-1])))
    return toks[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generate_and_long_decode(std, device):
    """`Runner.generate` (prefill, the on-device sampler, the decode graph on a GPU) produces the oracle's greedy
    continuation over several block borders; the next turn extends the cached sequence (its states are kept
    whole), a prompt that shares only a part starts over."""
    prompt = sc.tokens(12, 96, seed=60)
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
        prompts = [sc.tokens(n, 96, seed=70 + i) for i, n in enumerate((9, 20, 14))]
        lens = (12, 5, 9)
        its = [sch.submit(p, GREEDY, max_tokens=k) for p, k in zip(prompts, lens)]
        got = [list(it) for it in its]
        for p, k, g in zip(prompts, lens, got):
            assert g == greedy_oracle(std, p, k)
    finally:
        sch.close()


def test_command_line_generates_token_ids(std, capsys):
    from ollama_operator_amd import cli
    prompt = sc.tokens(9, 96, seed=90)
    cli.main(["tokens", std.path, "--ids", " ".join(map(str, prompt)), "--num-predict", "5", "--device", "cpu",
              "--dtype", "float32"])
    out = capsys.readouterr().out.strip().splitlines()[-1]
    assert [int(t) for t in out.split()] == greedy_oracle(std, prompt, 5)


def test_trace_replay_program(std, tmp_path):
    """bin/trace_run on the CPU twin: a request that sits out a step, one that ends and gives its slot back."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    a, b = sc.tokens(30, 96, seed=91), sc.tokens(12, 96, seed=92)
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
    sc.check(np.fromfile(out / "0.f32", "<f4").reshape(2, 96), wa[[0, 19]], "float32", "step 0")
    sc.check(np.fromfile(out / "1.f32", "<f4").reshape(1, 96), wb[[11]], "float32", "step 1")
    sc.check(np.fromfile(out / "2.f32", "<f4").reshape(1, 96), wa[[29]], "float32", "step 2")


# ------------------------------------------------------------------ the HIP executor against its twin
@pytest.mark.gpu
def test_gpu_matches_twin_layer_by_layer(std):
    toks = sc.tokens(50, 96, seed=95)
    for dtype, tol in (("float32", 1e-4), ("bfloat16", 0.05)):
        a = sc.layer_trail(std.runner("cpu", dtype), toks)
        b = sc.layer_trail(std.runner("cuda", dtype), toks)
        for i in range(a.shape[0]):
            assert np.abs(a[i] - b[i]).max() < tol * max(1.0, np.abs(a[i]).max()), f"{dtype}: layer run {i}"


@pytest.mark.gpu
def test_chunked_and_token_by_token_state_agree(tmp_path):
    """The state a prompt portion leaves (chunks around a scan) and the state single tokens leave are the same matrix:
    decode 30 tokens after a 100-token portion and after 100 single tokens."""
    m = sc.Model(tmp_path, sc.config([(sc.parallel(right=sc.gla(heads=2, dim=32, vdim=64, tau=2.0, rank=8)), sc.glu())], width=64), seed=31)
    toks = sc.tokens(130, 96, seed=32)
    want, _ = m.oracle(toks)
    r = m.runner("cuda", max_batch=128)
    sc.check(sc.run_cuts(r, toks, [100] + list(range(101, 131)))[100:], want[100:], "float32", "after a portion")
    sc.check(sc.run_cuts(r, toks, list(range(1, 131)))[100:], want[100:], "float32", "after single tokens")


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_configurations(tmp_path, seed):
    """Configurations drawn at the scale of a small real model, 700-token prompts in portions and whole, float32
    sharply and bfloat16 by the typical row."""
    rng = random.Random(1000 + seed)
    cfg = sc.random_config(rng)
    m = sc.Model(tmp_path, cfg, seed=seed)
    toks = sc.tokens(700, cfg.n_vocab, seed=seed)
    want, _ = m.oracle(toks)
    rows = sorted(rng.sample(range(700), 40)) + [699]
    for dtype in BOTH:
        r = m.runner("cuda", dtype, max_batch=512, kv_tokens=1024)
        sid = r.new_sequence()
        cuts, got, a = [rng.randint(1, 300), rng.randint(301, 600), 690] + list(range(691, 701)), [], 0
        for b in cuts:
            want_rows = [i - a for i in rows if a <= i < b]
            got.append(r.step_entries([(sid, toks[a:b], want_rows)]).float().cpu().numpy())
            a = b
        r.free_sequence(sid)
        sc.check(np.concatenate(got), want[rows], dtype, f"random configuration {seed}")
