"""Random-init GGUF fixtures of real architectures (BASELINE.json: "synthetic prompts / random-init
GGUF weights"). Weights are drawn directly in quantized block form so a 4 GB Llama-2-7B Q4_K_M file
is produced in seconds, with the exact tensor-type mix of a real Q4_K_M conversion."""
from __future__ import annotations

import numpy as np

from ..gguf.constants import FileType, GGMLType
from ..gguf.writer import GGUFWriter
from ..quant import quantize, random_blocks
from ..tokenizer import synth_vocab_bpe, synth_vocab_spm
from .arch import tensor_specs
from .config import ModelConfig


def _norm_weight(n: int, rng: np.random.Generator) -> np.ndarray:
    return (1.0 + 0.05 * rng.standard_normal(n)).astype(np.float32)


def write_random_gguf(path: str, cfg: ModelConfig, ftype: FileType = FileType.MOSTLY_Q4_K_M,
                      seed: int = 0, std: float = 0.02, quantize_from_float: bool = False) -> dict:
    """Write a random-init model. `quantize_from_float` draws float weights and runs the reference
    quantizer (slow; small test models) instead of drawing random blocks."""
    rng = np.random.default_rng(seed)
    w = GGUFWriter(path)
    md = cfg.to_gguf_metadata()
    md["general.file_type"] = int(ftype)
    md["general.quantization_version"] = 2
    vocab = synth_vocab_bpe(cfg.n_vocab) if cfg.arch == "phi2" else synth_vocab_spm(cfg.n_vocab)
    md.update(vocab)
    for k, v in md.items():
        w.add(k, v)
    for name, shape, gt in tensor_specs(cfg, ftype):
        n = int(np.prod(shape))
        k = shape[0]
        rows = n // k
        tseed = int(rng.integers(0, 2**31))
        if name.endswith("norm.weight"):
            w.add_tensor(name, shape, gt, lambda n=n, s=tseed: _norm_weight(n, np.random.default_rng(s)))
        elif name.endswith(".bias"):
            w.add_tensor(name, shape, gt,
                         lambda n=n, s=tseed: (0.02 * np.random.default_rng(s).standard_normal(n)).astype(np.float32))
        elif name.endswith("ffn_gate_inp.weight"):
            w.add_tensor(name, shape, gt,
                         lambda n=n, s=tseed: (0.1 * np.random.default_rng(s).standard_normal(n)).astype(np.float32))
        elif quantize_from_float or gt in (GGMLType.F32, GGMLType.F16, GGMLType.BF16):
            w.add_tensor(name, shape, gt, lambda n=n, s=tseed, g=gt: quantize(
                (std * np.random.default_rng(s).standard_normal(n)).astype(np.float32), g))
        else:
            w.add_tensor(name, shape, gt, lambda r=rows, k=k, s=tseed, g=gt: random_blocks(
                g, r, k, np.random.default_rng(s), std))
    w.write()
    return md


def write_random_stack(path: str, cfg, seed: int = 0, std: float = 0.05) -> None:
    """Random-init model folder (config.json + model.safetensors, bfloat16) of a layer-list model
    (config.StackConfig, the Bizulix tensor names). Projections ~ N(0, std); norm weights near 1; router
    matrices and biases wide enough that the top experts are not a close call."""
    import json
    import os

    import torch

    from ..engine.safetensors_io import write_safetensors
    from .config import MIX_RETENTION
    if cfg.arch == "norevik":
        return write_random_norevik(path, cfg, seed=seed)
    if cfg.arch == "suvunex":
        return write_random_suvunex(path, cfg, seed=seed)
    if cfg.arch == "dekalorn":
        return write_random_dekalorn(path, cfg, seed=seed)
    g = torch.Generator().manual_seed(seed)
    E, V = cfg.n_embd, cfg.n_vocab
    T: dict = {}

    def rnd(name, shape, s=std, mean=0.0):
        T[name] = (mean + s * torch.randn(*shape, generator=g)).to(torch.bfloat16)

    rnd("embed", (V, E), 1.0)
    if cfg.loop_times:
        rnd("loop.in", (E, 2 * E), 0.7 / E ** 0.5)
    for i, spec in enumerate(cfg.layers):
        m, f, p = spec.mixer, spec.mlp, f"l{i}."
        rnd(p + "norm1", (E,), 0.05, 1.0)
        rnd(p + "norm1.b", (E,), 0.05)
        rnd(p + "mix.q", (m.n_q, E), 1.0 / E ** 0.5)
        rnd(p + "mix.k", (m.n_k, E), 1.0 / E ** 0.5)
        rnd(p + "mix.v", (m.n_v, E), 1.0 / E ** 0.5)
        if m.kind == MIX_RETENTION:
            rnd(p + "mix.g", (m.n_out, E), 1.0 / E ** 0.5)
        rnd(p + "mix.o", (E, m.n_out), 1.0 / m.n_out ** 0.5)
        if f is not None:
            for e in range(f.experts):
                rnd(f"{p}mlp.e{e}.gate", (f.ff, E), 1.0 / E ** 0.5)
                rnd(f"{p}mlp.e{e}.up", (f.ff, E), 1.0 / E ** 0.5)
                rnd(f"{p}mlp.e{e}.down", (E, f.ff), 1.0 / f.ff ** 0.5)
            rnd(p + "mlp.router", (f.experts, E), 2.0 / E ** 0.5)
            rnd(p + "mlp.router.b", (f.experts,), 0.5)
            if f.shared_ff:
                rnd(p + "mlp.shared.gate", (f.shared_ff, E), 1.0 / E ** 0.5)
                rnd(p + "mlp.shared.up", (f.shared_ff, E), 1.0 / E ** 0.5)
                rnd(p + "mlp.shared.down", (E, f.shared_ff), 1.0 / f.shared_ff ** 0.5)
                rnd(p + "mlp.shared.sg", (1, E), 1.0 / E ** 0.5)
    rnd("final.norm", (E,), 0.05, 1.0)
    rnd("final.norm.b", (E,), 0.05)
    rnd("head", (V, E), 1.0 / E ** 0.5)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(cfg.to_config_json(), fh, indent=1)
    write_safetensors(os.path.join(path, "model.safetensors"), T)


def write_random_norevik(path: str, cfg, seed: int = 0) -> None:
    """Random-init model folder of the Norevik design (its tensor names). Projections ~ N(0, 1 / fan-in); norm
    weights near 1; forget-gate biases positive (memories that last), step-size biases negative, decays spread
    over several orders, sinks of a few units, router corrections of the size of a score."""
    import json
    import os

    import torch

    from ..engine.safetensors_io import write_safetensors
    from .config import FF_DENSE, MIX_LATENT, MIX_MAMBA2, MIX_MLSTM
    g = torch.Generator().manual_seed(seed)
    E, V = cfg.n_embd, cfg.n_vocab
    T: dict = {}

    def rnd(name, shape, s, mean=0.0):
        T[name] = (mean + s * torch.randn(*shape, generator=g)).to(torch.bfloat16)

    def uni(name, shape, lo, hi):
        T[name] = (lo + (hi - lo) * torch.rand(*shape, generator=g)).to(torch.bfloat16)

    def lin(name, n_out, n_in, gain=1.0):
        rnd(name, (n_out, n_in), gain / n_in ** 0.5)

    def norm(name, n):
        rnd(name, (n,), 0.1, 1.0)
        rnd(name + ".b", (n,), 0.1)

    rnd("embed", (V, E), 1.0 / max(cfg.embed_scale, 1e-6))
    for i, spec in enumerate(cfg.layers):
        m, f, p = spec.mixer, spec.mlp, f"l{i}."
        H, D, Dv = m.heads, m.dim, m.vdim
        norm(p + "norm1", E)
        if m.kind == MIX_LATENT:
            lin(p + "mix.q", H * (D + m.rot_dim), E, 2.0)
            lin(p + "mix.dkv", m.kv_rank + m.rot_dim, E, 2.0)
            rnd(p + "mix.dkv.norm", (m.kv_rank,), 0.1, 1.0)
            lin(p + "mix.uk", H * D, m.kv_rank, 1.5)
            lin(p + "mix.uv", H * Dv, m.kv_rank)
            uni(p + "mix.sink", (H,), -1.0, 4.0)
            lin(p + "mix.g", H * Dv, E, 1.5)
        elif m.kind == MIX_MLSTM:
            lin(p + "mix.q", H * D, E)
            lin(p + "mix.k", H * D, E)
            lin(p + "mix.v", H * Dv, E)
            lin(p + "mix.g", H * Dv, E, 1.5)
            lin(p + "mix.i", H, E, 2.0)
            lin(p + "mix.f", H, E, 2.0)
            rnd(p + "mix.i.b", (H,), 1.0)
            uni(p + "mix.f.b", (H,), 0.5, 6.0)
            rnd(p + "mix.norm", (H * Dv,), 0.1, 1.0)
        elif m.kind == MIX_MAMBA2:
            inner, ch = H * Dv, m.conv_channels
            lin(p + "mix.in", 2 * inner + 2 * m.groups * m.state + H, E)
            rnd(p + "mix.conv", (ch, m.conv), 0.6, 0.2)
            rnd(p + "mix.conv.b", (ch,), 0.1)
            uni(p + "mix.dt_bias", (H,), -4.0, -0.5)
            uni(p + "mix.A_log", (H,), -4.0, 1.0)
            uni(p + "mix.D", (H,), 0.5, 1.0)
            rnd(p + "mix.norm", (inner,), 0.1, 1.0)
        else:
            raise ValueError("the Norevik design has no mixer of this kind")
        lin(p + "mix.o", E, H * Dv)
        if f is None:
            continue
        norm(p + "norm2", E)
        if f.kind == FF_DENSE:
            lin(p + "mlp.up", f.ff, E)
            lin(p + "mlp.down", E, f.ff)
            continue
        for e in range(f.experts):
            lin(f"{p}mlp.e{e}.gate", f.ff, E)
            lin(f"{p}mlp.e{e}.up", f.ff, E)
            lin(f"{p}mlp.e{e}.down", E, f.ff)
        lin(p + "mlp.router", f.n_router, E, 3.0)
        rnd(p + "mlp.correction", (f.n_router,), 0.3)
        if f.shared_ff:
            lin(p + "mlp.shared.gate", f.shared_ff, E)
            lin(p + "mlp.shared.up", f.shared_ff, E)
            lin(p + "mlp.shared.down", E, f.shared_ff)
    norm("final.norm", E)
    lin("head", V, E)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(cfg.to_norevik(), fh, indent=1)
    write_safetensors(os.path.join(path, "model.safetensors"), T)


def write_random_suvunex(path: str, cfg, seed: int = 0) -> None:
    """Random-init model folder of the Suvunex design (its tensor names). Projections ~ N(0, 1 / fan-in) with biases
    of a fraction of a unit; scalar norm weights and per-channel scales near 1; convolution taps of a fraction of
    the identity; sinks of a few units; a head-mixing matrix near the identity; decay biases spread so that some
    key channels forget in a few tokens and others keep for hundreds."""
    import json
    import os

    import torch

    from ..engine.safetensors_io import write_safetensors
    g = torch.Generator().manual_seed(seed)
    E, V = cfg.n_embd, cfg.n_vocab
    T: dict = {}

    def rnd(name, shape, s, mean=0.0):
        T[name] = (mean + s * torch.randn(tuple(shape), generator=g)).to(torch.bfloat16)

    def uni(name, shape, lo, hi):
        T[name] = (lo + (hi - lo) * torch.rand(tuple(shape), generator=g)).to(torch.bfloat16)

    def lin(name, n_out, n_in, gain=1.0, bias=False):
        rnd(name, (n_out, n_in), gain / n_in ** 0.5)
        if bias:
            rnd(name + ".b", (n_out,), 0.3)

    def attention(a, m):
        lin(a + "q", m.n_q, E, 1.5, m.bias)
        lin(a + "k", m.n_k, E, 1.5, m.bias)
        if not m.v_from_k:
            lin(a + "v", m.n_v, E, 1.0, m.bias)
        if m.qk_norm == 1:
            rnd(a + "q.norm", (m.dim,), 0.2, 1.0)
            rnd(a + "k.norm", (m.dim,), 0.2, 1.0)
        if m.sink == 1:
            uni(a + "sink", (m.heads,), -1.0, 4.0)
        if m.talk:
            T[a + "talk"] = (torch.eye(m.heads) + 0.3 * torch.randn(m.heads, m.heads, generator=g)).to(torch.bfloat16)
        lin(a + "o", E, m.n_out, 1.0, m.o_bias)

    rnd("embed", (V, E), 1.0 / max(cfg.embed_scale, 1e-6))
    for i, spec in enumerate(cfg.layers):
        m, f, p = spec.mixer, spec.mlp, f"l{i}."
        for k in ("norm1", "norm1b"):
            rnd(p + k, (), 0.1, 1.0)
        rnd(p + "ls1", (E,), 0.2, 0.8)
        rnd(p + "canon1", (E, cfg.canon_taps), 0.3)
        if m.right is not None:
            r, b = m.right, p + "mix.right."
            attention(p + "mix.left.", m)
            rank = r.decay_rank or 8
            lin(b + "q", r.n_q, E, 1.5)
            lin(b + "k", r.n_q, E, 1.5)
            lin(b + "v", r.n_out, E)
            lin(b + "g", r.n_out, E, 1.5)
            lin(b + "a1", rank, E)
            lin(b + "a2", r.n_q, rank, 2.0)
            uni(b + "a2.b", (r.n_q,), -1.0, 6.0)
            rnd(b + "norm", (r.vdim,), 0.1, 1.0)
            lin(b + "o", E, r.n_out)
        else:
            attention(p + "mix.", m)
        if f is not None:
            for k in ("norm2", "norm2b"):
                rnd(p + k, (), 0.1, 1.0)
            rnd(p + "ls2", (E,), 0.2, 0.8)
            lin(p + "mlp.gate", f.ff, E, 1.5)
            lin(p + "mlp.up", f.ff, E)
            lin(p + "mlp.down", E, f.ff)
    rnd("final.norm", (), 0.1, 1.0)
    lin("head", V, E)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(cfg.to_suvunex(), fh, indent=1)
    write_safetensors(os.path.join(path, "model.safetensors"), T)


def write_random_dekalorn(path: str, cfg, seed: int = 0) -> None:
    """Random-init model folder of the Dekalorn design (its tensor names). Projections ~ N(0, 1 / fan-in), queries and
    keys with a gain so that the softmax is not flat; norm weights near 1; the vectors behind the differential
    attention's lambda small, so that lambda stays near `diff`; per-head score factors near 1 and a score-mixing matrix
    near the identity; router matrices wide enough that the chosen experts are not a close call."""
    import json
    import os

    import torch

    from ..engine.safetensors_io import write_safetensors
    from .config import FF_GLU, MIX_LATENT
    g = torch.Generator().manual_seed(seed)
    E, V = cfg.n_embd, cfg.n_vocab
    T: dict = {}

    def rnd(name, shape, s, mean=0.0):
        T[name] = (mean + s * torch.randn(*shape, generator=g)).to(torch.bfloat16)

    def lin(name, n_out, n_in, gain=1.0):
        rnd(name, (n_out, n_in), gain / n_in ** 0.5)

    rnd("embed", (V, E), 1.0)
    if cfg.loop_times:
        lin("loop.in", E, 2 * E, 1.4)
    for i, spec in enumerate(cfg.layers):
        m, f, p = spec.mixer, spec.mlp, f"l{i}."
        H, G, D, Dv = m.heads, m.kv_heads, m.dim, m.vdim
        rnd(p + "norm1", (E,), 0.1, 1.0)
        if m.kind == MIX_LATENT:
            lin(p + "mix.q", H * (D + m.rot_dim), E, 2.0)
            lin(p + "mix.dkv", m.kv_rank + m.rot_dim, E, 2.0)
            rnd(p + "mix.dkv.norm", (m.kv_rank,), 0.1, 1.0)
            lin(p + "mix.uk", H * D, m.kv_rank, 1.5)
            lin(p + "mix.uv", H * Dv, m.kv_rank)
            lin(p + "mix.g", H, E, 1.5)
        else:
            lin(p + "mix.q", m.n_q, E, 2.0)
            lin(p + "mix.k", m.n_k, E, 2.0)
            lin(p + "mix.v", m.n_v, E)
            if m.maps == 2:
                for k in ("lq1", "lk1", "lq2", "lk2"):
                    rnd(p + "mix." + k, (D,), 0.1)
                lin(p + "mix.g", H * Dv, E, 1.5)
            else:
                T[p + "mix.talk"] = (torch.eye(H) + 0.25 * torch.randn(H, H, generator=g)).to(torch.bfloat16)
                rnd(p + "mix.temp", (H,), 0.2, 1.0)
        lin(p + "mix.o", E, H * Dv)
        if f is None:
            continue
        rnd(p + "norm2", (E,), 0.1, 1.0)
        if f.kind == FF_GLU:
            lin(p + "mlp.gate", f.ff, E)
            lin(p + "mlp.up", f.ff, E)
            lin(p + "mlp.down", E, f.ff)
            continue
        for e in range(f.experts):
            lin(f"{p}mlp.e{e}.gate", f.ff, E)
            lin(f"{p}mlp.e{e}.up", f.ff, E)
            lin(f"{p}mlp.e{e}.down", E, f.ff)
        lin(p + "mlp.router", f.experts, E, 3.0)
    rnd("final.norm", (E,), 0.1, 1.0)
    lin("head", V, E)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(cfg.to_dekalorn(), fh, indent=1)
    write_safetensors(os.path.join(path, "model.safetensors"), T)
