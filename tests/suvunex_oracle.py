"""Plain, slow float64 implementation of the Suvunex design, one function per mechanism.

It is the yardstick of the Suvunex tests and shares no code with the engine: it takes a config dict (the
layout of config.json) and a dict name -> torch tensor, runs one whole sequence at a time and keeps no cache
(attention looks at the full prefix, the recurrence is walked token by token from a zero state, the input
convolution sees zeros before the first token).

Notation: n tokens, width E. Linear weights are [out, in]; y = x @ W.T. A layer is
x <- x + s1 * N1b(mixer(conv_in(N1(x)))), then x <- x + s2 * N2b(ff(N2(x))), where N is an RMS norm with a
single scalar weight, s1 / s2 are per-channel scales, and conv_in(h) = h + causal_conv(h).
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose weight is one number for all coordinates."""
    return unit_rms(x, eps) * g


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def input_conv(h, w):
    """h [n, E], w [E, taps]: h_t + sum_j w[:, j] h_(t - taps + 1 + j), zeros before the sequence's start."""
    n, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def rotary_frequencies(rot):
    """f_i = base^(-2i / dims), then the scaling the config names: none, all divided by `factor`, or by wavelength
    bands (short waves kept, long waves divided by `factor`, a linear blend in between)."""
    if not rot or not rot.get("dims"):
        return torch.zeros(0, dtype=F64)   # no rotation
    dims = rot["dims"]
    f = [rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F64)
    if "original" not in sc:
        return torch.tensor([x / sc["factor"] for x in f], dtype=F64)
    out = []
    for x in f:
        wave = 2.0 * math.pi / x
        if wave < sc["original"] / sc["high"]:
            out.append(x)
        elif wave > sc["original"] / sc["low"]:
            out.append(x / sc["factor"])
        else:
            s = (sc["original"] / wave - sc["low"]) / (sc["high"] - sc["low"])
            out.append((1.0 - s) * x / sc["factor"] + s * x)
    return torch.tensor(out, dtype=F64)


def rotate_half(x, pos, freqs):
    """x [n, H, D]: dims i and i + len(freqs) of the last axis turn by pos * freqs[i]; the rest pass."""
    half = freqs.numel()
    ang = pos.to(F64)[:, None] * freqs[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], -1)


# --------------------------------------------------------------------------------------------- mixers
def softmax_plus_one_attention(h, W, m, eps):
    """Grouped-query softmax attention with biases, rotation of part of each head, unit RMS of q and k AFTER the
    rotation, and a denominator that holds one extra 1 (a sink of score 0 without a value)."""
    n = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(n)
    q = (h @ W["q"].T + W["q.b"]).view(n, H, D)
    k = (h @ W["k"].T + W["k.b"]).view(n, G, D)
    v = (h @ W["v"].T + W["v.b"]).view(n, G, Dv)
    fr = rotary_frequencies(m.get("rot"))
    q, k = unit_rms(rotate_half(q, pos, fr), eps), unit_rms(rotate_half(k, pos, fr), eps)
    mask = torch.tril(torch.ones(n, n, dtype=torch.bool))
    out = torch.zeros(n, H, Dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        e = torch.exp(s).masked_fill(~mask, 0.0)
        out[:, hd] = (e / (1.0 + e.sum(-1, keepdim=True))) @ v[:, g]
    return out.reshape(n, H * Dv) @ W["o"].T + W["o.b"]


def gated_linear_attention(h, W, m, eps):
    """S_t = diag(alpha_t) S_(t-1) + k_t v_t^T per head, o_t = S_t^T q_t, alpha = sigmoid(z)^(1 / tau) per key
    channel from a low-rank map; each head's o is RMS-normed with a shared weight and gated by silu(W_g h)."""
    n = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W["q"].T).view(n, H, D) * D ** -0.5
    k = (h @ W["k"].T).view(n, H, D)
    v = (h @ W["v"].T).view(n, H, Dv)
    z = (h @ W["a1"].T) @ W["a2"].T + W["a2.b"]
    alpha = torch.sigmoid(z).pow(1.0 / m["tau"]).view(n, H, D)
    S = torch.zeros(H, D, Dv, dtype=F64)
    o = torch.zeros(n, H, Dv, dtype=F64)
    for t in range(n):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = unit_rms(o, eps) * W["norm"]
    return (o.reshape(n, H * Dv) * silu(h @ W["g"].T)) @ W["o"].T


def parallel_mixer(h, W, m, eps):
    left = softmax_plus_one_attention(h, sub(W, "left."), m["left"], eps)
    right = gated_linear_attention(h, sub(W, "right."), m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def talking_attention(h, W, m, eps):
    """Grouped-query attention whose values are the projected keys (before their norm and rotation); weighted RMS
    norm of q and k BEFORE the rotation; a learned per-head sink in the denominator; the heads' softmax weights are
    mixed by a square matrix before they meet the values of each head's own key/value head."""
    n = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    pos = torch.arange(n)
    q = (h @ W["q"].T + W["q.b"]).view(n, H, D)
    k = (h @ W["k"].T + W["k.b"]).view(n, G, D)
    v = k.clone()
    fr = rotary_frequencies(m.get("rot"))
    q = rotate_half(unit_rms(q, eps) * W["q.norm"], pos, fr)
    k = rotate_half(unit_rms(k, eps) * W["k.norm"], pos, fr)
    mask = torch.tril(torch.ones(n, n, dtype=torch.bool))
    p = torch.zeros(H, n, n, dtype=F64)
    for hd in range(H):
        s = (q[:, hd] @ k[:, hd // (H // G)].T) * m["scale"]
        e = torch.exp(s).masked_fill(~mask, 0.0)
        p[hd] = e / (e.sum(-1, keepdim=True) + torch.exp(W["sink"][hd]))
    p = torch.einsum("hg,gij->hij", W["talk"], p)
    out = torch.stack([p[hd] @ v[:, hd // (H // G)] for hd in range(H)], 1)
    return out.reshape(n, H * D) @ W["o"].T


def glu_ff(h, W):
    return (gelu_tanh(h @ W["gate"].T) * (h @ W["up"].T)) @ W["down"].T


# --------------------------------------------------------------------------------------------- model
def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, tokens):
    """Returns (logits [n, V], residual stream after every layer [L, n, E])."""
    T = {k: v.to(F64) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    x = T["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    after = []
    for i, ent in enumerate(cfg["layers"]):
        L = sub(T, f"l{i}.")
        h = input_conv(scalar_norm(x, L["norm1"], eps), L["canon1"])
        mix = {"parallel": parallel_mixer, "attention": talking_attention}[ent["type"]]
        x = x + L["ls1"] * scalar_norm(mix(h, sub(L, "mix."), ent["mixer"], eps), L["norm1b"], eps)
        if ent.get("mlp"):
            if ent["mlp"]["kind"] != "dense":
                raise ValueError("unknown feed-forward kind")
            y = glu_ff(scalar_norm(x, L["norm2"], eps), sub(L, "mlp."))
            x = x + L["ls2"] * scalar_norm(y, L["norm2b"], eps)
        after.append(x.clone())
    z = (scalar_norm(x, T["final.norm"], eps) @ T["head"].T) * cfg["logit_scale"]
    return z, torch.stack(after)
