"""Suvunex test bodies, shared by the CPU tests (torch twin of the executor: host logic) and the GPU tests (HIP
kernels). Every case builds its own small configuration with random weights, runs it through the engine
(`StackRunner`, its block pool, state slots and step function) and compares with the plain float64
implementation in `suvunex_oracle.py`."""
from __future__ import annotations

import numpy as np

import suvunex_oracle as oracle
from bizulix_cases import Model as _Model
from bizulix_cases import layer_trail, rel_err, run_cuts, tokens  # noqa: F401  (re-exported for the tests)
from ollama_operator_amd.models.config import (BLOCK_SANDWICH, FF_GLU, MIX_ATTENTION, MIX_GLA, QK_NORM_UNIT_LAST,
                                               QK_NORM_WEIGHT_FIRST, SINK_LEARNED, SINK_ONE, LayerSpec, MixerSpec, MoESpec,
                                               StackConfig)

BANDS = ("bands", 6.0, 1.0, 5.0, 64.0)   # with base 100 and 8 pairs: kept, blended and divided frequencies all occur


def gla(heads=2, dim=8, vdim=12, tau=4.0, rank=5):
    return MixerSpec(kind=MIX_GLA, heads=heads, kv_heads=heads, dim=dim, vdim=vdim, tau=tau, decay_rank=rank)


def parallel(heads=4, kv_heads=2, dim=16, vdim=12, scale=0.2, rot_dims=8, base=100.0, scaling=BANDS, right=None,
             left_scale=0.7, right_scale=1.2):
    return MixerSpec(kind=MIX_ATTENTION, heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, rot_dims=rot_dims,
                     rot_base=base, rot_scaling=scaling if rot_dims else (), bias=True, o_bias=True, qk_norm=QK_NORM_UNIT_LAST,
                     sink=SINK_ONE, right=right or gla(), left_scale=left_scale, right_scale=right_scale)


def talking(heads=4, kv_heads=2, dim=16, scale=0.3, rot_dims=16, base=1000.0, scaling=("linear", 2.0)):
    return MixerSpec(kind=MIX_ATTENTION, heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale, rot_dims=rot_dims,
                     rot_base=base, rot_scaling=scaling if rot_dims else (), bias=True, qk_norm=QK_NORM_WEIGHT_FIRST,
                     sink=SINK_LEARNED, talk=True, v_from_k=True)


def glu(ff=40):
    return MoESpec(kind=FF_GLU, ff=ff)


def config(layers, width=64, vocab=96, eps=1e-5, embed_scale=5.0, taps=3, logit_scale=0.5):
    return StackConfig(arch="suvunex", n_vocab=vocab, n_embd=width, layers=[LayerSpec(mixer=m, mlp=f) for m, f in layers],
                       norm_eps=eps, block=BLOCK_SANDWICH, embed_scale=embed_scale, canon_taps=taps, logit_scale=logit_scale)


def standard():
    """Both mixers with sizes that differ from one another: a pair layer first, a mixed-heads attention without
    feed-forward, a pair layer whose attention has one key/value head per query head and no frequency scaling, a
    mixed-heads attention with one key/value head, a pair layer with one key/value head and a value size above the
    key size."""
    return config([(parallel(), glu()),
                   (talking(), None),
                   (parallel(heads=2, kv_heads=2, dim=8, vdim=20, rot_dims=4, scaling=(),
                             right=gla(heads=3, dim=4, vdim=8, tau=1.0, rank=3)), glu(24)),
                   (talking(heads=3, kv_heads=1, dim=12, rot_dims=6, scaling=()), glu(56)),
                   (parallel(heads=3, kv_heads=1, dim=8, vdim=24, rot_dims=8, scaling=("linear", 3.0),
                             right=gla(heads=1, dim=16, vdim=16, tau=16.0, rank=8)), glu(32))])


def check(got, want, dtype, what=""):
    """float32: every row within 1e-4 of the logits' spread. bfloat16: rounding moves a row by about a percent, and
    by several where a sharp softmax sits on a close call: the median row within 2.5e-2, at most one row in ten over
    6e-2, none over 0.3."""
    e = rel_err(got, want)
    assert np.isfinite(np.asarray(got)).all(), f"{what}: non-finite logits"
    worst = f"{what}: worst row {int(e.argmax())} off by {e.max():.3g} (median {np.median(e):.3g})"
    if dtype == "float32":
        assert e.max() < 1e-4, worst
    else:
        assert np.median(e) < 2.5e-2 and e.max() < 0.3 and (e > 6e-2).sum() <= max(2, len(e) // 10), \
            f"{worst}, {(e > 6e-2).sum()} of {len(e)} rows over 0.06"


def random_config(rng):
    """A configuration drawn at the scale of a small real model: 3-6 layers of both kinds in any order, widths
    128-320, head counts, sizes, rotations, taps and scales of many shapes (rng: random.Random)."""
    width = rng.choice([128, 160, 224, 256, 320])

    def rot(dim):
        rd = rng.choice([0, dim // 2, dim])
        sc = rng.choice([(), ("linear", rng.choice([2.0, 8.0])), ("bands", rng.choice([4.0, 8.0]), 1.0, rng.choice([2.0, 4.0]),
                                                                   float(rng.choice([64, 256, 1024])))])
        return rd - rd % 2, rng.choice([1e3, 5e4, 1e6]), sc

    def par():
        G = rng.choice([1, 2, 4])
        D = rng.choice([32, 48, 64, 96])
        rd, base, sc = rot(D)
        return parallel(heads=G * rng.choice([1, 2, 4]), kv_heads=G, dim=D, vdim=rng.choice([32, 64, 96]),
                        scale=rng.choice([0.05, 0.1, 0.2]), rot_dims=rd, base=base, scaling=sc,
                        right=gla(heads=rng.choice([1, 2, 4]), dim=rng.choice([16, 32, 48, 64]), vdim=rng.choice([32, 64, 128]),
                                  tau=rng.choice([1.0, 4.0, 16.0]), rank=rng.choice([4, 16, 32])),
                        left_scale=rng.choice([0.5, 1.0]), right_scale=rng.choice([0.8, 1.5]))

    def talk():
        G = rng.choice([1, 2, 4])
        D = rng.choice([32, 64, 96, 128])
        rd, base, sc = rot(D)
        return talking(heads=G * rng.choice([1, 2, 3]), kv_heads=G, dim=D, scale=rng.choice([0.05, 0.125, 0.2]), rot_dims=rd, base=base,
                       scaling=sc)

    layers = [(rng.choice([par, par, talk])(), rng.choice([None, glu(rng.choice([256, 384, 512])), glu(rng.choice([256, 320]))]))
              for _ in range(rng.randint(3, 6))]
    return config(layers, width=width, vocab=rng.choice([500, 777, 1024]), eps=rng.choice([1e-5, 1e-6]), embed_scale=width ** 0.5,
                  taps=rng.choice([1, 2, 3, 4]), logit_scale=rng.choice([0.25, 1.0, 0.7]))


class Model(_Model):
    def oracle(self, toks):
        z, trail = oracle.forward(self.json, self.tensors, toks)
        return z.numpy(), trail.numpy()
