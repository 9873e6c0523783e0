"""Dekalorn test bodies, shared by the CPU tests (torch twin of the executor: host logic) and the GPU tests (HIP
kernels). Every case builds its own small configuration with random weights, runs it through the engine
(`StackRunner`, its block pool, slots and step function) and compares with the plain float64 implementation in
`dekalorn_oracle.py`."""
from __future__ import annotations

import numpy as np

import dekalorn_oracle as oracle
from bizulix_cases import Model as _Model
from bizulix_cases import layer_trail, rel_err, run_cuts, tokens  # noqa: F401  (re-exported for the tests)
from ollama_operator_amd.models.config import (ACT_RELU, BLOCK_PRENORM, FF_GLU, FF_MOE, GATE_ELEMENT, GATE_HEAD, MIX_ATTENTION,
                                               MIX_LATENT, ROUTE_SIGMOID_GROUPS, LayerSpec, MixerSpec, MoESpec, StackConfig)

BANDS = ("bands", 6.0, 1.0, 5.0, 64.0)   # with base 100 and 8 pairs: kept, blended and divided frequencies all occur


def diff(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.4, lam=0.3, window=11):
    return MixerSpec(kind=MIX_ATTENTION, heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, window=window, maps=2,
                     diff=lam, gate=GATE_ELEMENT)


def talk(heads=4, kv_heads=2, dim=16, vdim=12, scale=0.3, rot_dims=16, base=100.0, scaling=BANDS, window=13):
    return MixerSpec(kind=MIX_ATTENTION, heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, window=window,
                     score_talk=True, rot_pairs=True, rot_dims=rot_dims, rot_base=base, rot_scaling=scaling if rot_dims else ())


def latent(heads=3, dim=8, rot_dim=6, vdim=10, kv_rank=12, scale=0.3, rot_dims=None, base=50.0):
    return MixerSpec(kind=MIX_LATENT, heads=heads, kv_heads=1, dim=dim, vdim=vdim, scale=scale, rot_dim=rot_dim, kv_rank=kv_rank,
                     rot_dims=rot_dim if rot_dims is None else rot_dims, rot_base=base, gate=GATE_HEAD, rot_pairs=True)


def dense(ff=40):
    return MoESpec(kind=FF_GLU, ff=ff, act=ACT_RELU)


def moe(experts=6, top=3, ff=16, count=3, keep=2, scale=1.7):
    return MoESpec(kind=FF_MOE, route=ROUTE_SIGMOID_GROUPS, experts=experts, top=top, ff=ff, group_count=count, group_keep=keep,
                   route_scale=scale, shared_gate=False)


def config(layers, width=64, vocab=96, eps=1e-5, loop=(0, 0, 0)):
    return StackConfig(arch="dekalorn", n_vocab=vocab, n_embd=width, layers=[LayerSpec(mixer=m, mlp=f) for m, f in layers],
                       norm_eps=eps, block=BLOCK_PRENORM, loop_start=loop[0], loop_stop=loop[1], loop_times=loop[2])


def standard():
    """Every mixer and both feed-forwards with sizes that differ from one another: a latent layer ahead of a span of
    three layers (mixed scores, two maps, latent) that runs twice, then a layer with two maps and one key/value head
    per query head without a feed-forward, and a mixed-score layer with one key/value head."""
    return config([(latent(), dense()),
                   (talk(), moe()),
                   (diff(), moe(experts=4, top=2, ff=24, count=1, keep=1, scale=1.0)),
                   (latent(heads=2, dim=12, rot_dim=4, vdim=6, kv_rank=20), dense(24)),
                   (diff(heads=2, kv_heads=2, dim=16, vdim=8, lam=0.7, window=30), None),
                   (talk(heads=3, kv_heads=1, dim=12, vdim=20, rot_dims=6, scaling=(), window=7), moe(experts=8, top=4, count=4, keep=4))],
                  loop=(1, 4, 2))


def check(got, want, dtype, what=""):
    """float32: every row within 1e-4 of the logits' spread. bfloat16 is loose on purpose: the difference of two
    attention maps is divided by its own root mean square, which amplifies the rounding of cached keys and values, and
    a router's close call that falls the other way swaps a whole expert: the median row within 4e-2, at most one row
    in three over 6e-2, one in forty (or one) over 0.5. The sharp comparisons are the float32 ones."""
    e = rel_err(got, want)
    assert np.isfinite(np.asarray(got)).all(), f"{what}: non-finite logits"
    worst = f"{what}: worst row {int(e.argmax())} off by {e.max():.3g} (median {np.median(e):.3g})"
    if dtype == "float32":
        assert e.max() < 1e-4, worst
    else:
        assert np.median(e) < 4e-2 and (e > 0.5).sum() <= max(1, len(e) // 40) and (e > 6e-2).sum() <= max(3, len(e) // 3), \
            f"{worst}, {(e > 6e-2).sum()} of {len(e)} rows over 0.06"


def random_config(rng):
    """A configuration drawn at the scale of a small real model: 3-6 layers of all kinds in any order, widths
    128-320, a repeated span or none, head counts, sizes, windows and router shapes of many kinds (rng: random.Random)."""
    width = rng.choice([128, 160, 224, 288, 320])

    def rot(dim):
        rd = rng.choice([dim // 2, dim])
        sc = rng.choice([(), ("bands", rng.choice([4.0, 8.0]), rng.choice([1.0, 2.0]), rng.choice([4.0, 8.0]),
                              float(rng.choice([64, 256, 1024])))])
        return rd - rd % 2, rng.choice([1e3, 5e4, 1e6]), sc

    def mk_diff():
        G = rng.choice([1, 2, 4])
        return diff(heads=G * rng.choice([1, 2]), kv_heads=G, dim=rng.choice([16, 32, 48, 64]), vdim=rng.choice([32, 56, 96]),
                    scale=rng.choice([0.1, 0.2]), lam=rng.choice([0.2, 0.5, 0.8]), window=rng.choice([33, 100, 257, 1000]))

    def mk_talk():
        G = rng.choice([1, 2, 4])
        D = rng.choice([32, 40, 64])
        rd, base, sc = rot(D)
        return talk(heads=G * rng.choice([1, 2, 3]), kv_heads=G, dim=D, vdim=rng.choice([32, 64]), scale=rng.choice([0.1, 0.15]),
                    rot_dims=rd, base=base, scaling=sc, window=rng.choice([17, 64, 130, 900]))

    def mk_latent():
        R = rng.choice([16, 32])
        return latent(heads=rng.choice([2, 4, 6]), dim=rng.choice([32, 64]), rot_dim=R, vdim=rng.choice([32, 72]),
                      kv_rank=rng.choice([64, 112, 160]), scale=rng.choice([0.08, 0.12]), base=rng.choice([1e3, 2.5e5]))

    def mk_ff():
        k = rng.choice(["none", "dense", "moe", "moe"])
        if k == "none":
            return None
        if k == "dense":
            return dense(rng.choice([256, 320]))
        count = rng.choice([1, 2, 4])
        per = rng.choice([2, 4])
        keep = rng.randint(1, count)
        return moe(experts=count * per, top=rng.randint(1, min(4, keep * per)), ff=rng.choice([64, 96, 128]), count=count, keep=keep,
                   scale=rng.choice([1.0, 2.5]))

    n = rng.randint(3, 6)
    layers = [(rng.choice([mk_diff, mk_talk, mk_latent])(), mk_ff()) for _ in range(n)]
    a = rng.randint(0, n - 1)
    loop = rng.choice([(0, 0, 0), (a, rng.randint(a + 1, n), rng.choice([1, 2, 3]))])
    return config(layers, width=width, vocab=rng.choice([500, 777, 1024]), eps=rng.choice([1e-5, 1e-6]), loop=loop)


class Model(_Model):
    def oracle(self, toks):
        z, trail = oracle.forward(self.json, self.tensors, toks)
        return z.numpy(), trail.numpy()
