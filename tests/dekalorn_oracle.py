"""Plain, slow float64 implementation of the Dekalorn design, one function per mechanism.

It is the yardstick of the Dekalorn tests and shares no code with the engine: it takes a config dict (the
layout of config.json) and a dict name -> torch tensor, runs one whole sequence at a time and keeps no cache
(every attention builds its full score matrix and masks it).

Notation: n tokens, width E. Linear weights are [out, in]; y = x @ W.T. A layer is pre-norm and sequential:
x <- x + mixer(N1(x)), then x <- x + ff(N2(x)), N an RMS norm with a weight vector. A span of layers may run
several times; every pass opens with x <- W_in [x; x0], x0 the embedding output.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def rotary_frequencies(rot):
    """f_i = base^(-2i / dims); with `scaling`, by wavelength bands: short waves kept, long waves divided by
    `factor`, a linear blend in between. No `rot`, or no dims: nothing turns."""
    if not rot or not rot.get("dims"):
        return torch.zeros(0, dtype=F64)
    dims = rot["dims"]
    f = [rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F64)
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


def rotate_pairs(x, pos, freqs):
    """x [n, ..., D]: dims (2i, 2i + 1), i < len(freqs), of the last axis turn by pos * freqs[i]; the rest pass."""
    n, m = x.shape[0], freqs.numel()
    ang = pos.to(F64)[:, None] * freqs[None, :]
    ang = ang.view(n, *([1] * (x.dim() - 2)), m)
    u, v = x[..., 0:2 * m:2], x[..., 1:2 * m:2]
    out = x.clone()
    out[..., 0:2 * m:2] = u * torch.cos(ang) - v * torch.sin(ang)
    out[..., 1:2 * m:2] = v * torch.cos(ang) + u * torch.sin(ang)
    return out


def visible(n, window=0):
    """mask[i, j]: position i sees j <= i, and with a window only the last `window` positions (itself included)."""
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    ok = j <= i
    if window:
        ok &= (i - j) < window
    return ok


def masked_softmax(s, ok):
    return torch.softmax(s.masked_fill(~ok, -float("inf")), -1)


# --------------------------------------------------------------------------------------------- mixers
def latent_attention(h, W, m, eps):
    """Keys and values of all heads are linear maps of one RMS-normed latent per token; one rotated key part is
    shared by the heads; a sigmoid gate with one number per head."""
    n = h.shape[0]
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(n)
    q = (h @ W["q"].T).view(n, H, D + R)
    dkv = h @ W["dkv"].T
    c = rms_norm(dkv[:, :C], W["dkv.norm"], eps)
    fr = rotary_frequencies(m.get("rot"))
    kr = rotate_pairs(dkv[:, C:], pos, fr)                 # [n, R]
    qr = rotate_pairs(q[..., D:], pos, fr)                 # [n, H, R]
    ku = (c @ W["uk"].T).view(n, H, D)
    v = (c @ W["uv"].T).view(n, H, Dv)
    gate = torch.sigmoid(h @ W["g"].T)                     # [n, H]
    ok = visible(n)
    out = torch.zeros(n, H, Dv, dtype=F64)
    for hd in range(H):
        s = (q[:, hd, :D] @ ku[:, hd].T + qr[:, hd] @ kr.T) * m["scale"]
        out[:, hd] = (masked_softmax(s, ok) @ v[:, hd]) * gate[:, hd:hd + 1]
    return out.reshape(n, H * Dv) @ W["o"].T


def differential_attention(h, W, m, eps):
    """Two softmax maps per head over the same values inside a sliding window; their difference, weighted by one
    number of the layer, is divided by its root mean square per head, scaled by 1 - diff and gated element-wise."""
    n = h.shape[0]
    H, G, D, Dv, diff = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["diff"]
    q = (h @ W["q"].T).view(n, H, 2, D)
    k = (h @ W["k"].T).view(n, G, 2, D)
    v = (h @ W["v"].T).view(n, G, Dv)
    lam = math.exp(float((W["lq1"] * W["lk1"]).sum())) - math.exp(float((W["lq2"] * W["lk2"]).sum())) + diff
    ok = visible(n, (m.get("mask") or {}).get("size", 0))
    out = torch.zeros(n, H, Dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        a = [masked_softmax((q[:, hd, j] @ k[:, g, j].T) * m["scale"], ok) @ v[:, g] for j in range(2)]
        out[:, hd] = unit_rms(a[0] - lam * a[1], eps) * (1.0 - diff)
    out = out.reshape(n, H * Dv) * torch.sigmoid(h @ W["g"].T)
    return out @ W["o"].T


def mixed_score_attention(h, W, m, eps):
    """Grouped-query attention with adjacent-pair rotation (frequencies scaled by bands), a per-head factor on the
    scores, and the heads' scores mixed by a square matrix BEFORE the softmax; sliding window."""
    n = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(n)
    fr = rotary_frequencies(m.get("rot"))
    q = rotate_pairs((h @ W["q"].T).view(n, H, D), pos, fr)
    k = rotate_pairs((h @ W["k"].T).view(n, G, D), pos, fr)
    v = (h @ W["v"].T).view(n, G, Dv)
    s = torch.stack([(q[:, hd] @ k[:, hd // (H // G)].T) * m["scale"] * W["temp"][hd] for hd in range(H)])   # [H, n, n]
    s = torch.einsum("hg,gij->hij", W["talk"], s)
    ok = visible(n, (m.get("mask") or {}).get("size", 0))
    out = torch.stack([masked_softmax(s[hd], ok) @ v[:, hd // (H // G)] for hd in range(H)], 1)
    return out.reshape(n, H * Dv) @ W["o"].T


MIXERS = {"latent_attention": latent_attention, "attention": differential_attention, "attention_2": mixed_score_attention}


# --------------------------------------------------------------------------------------------- feed-forwards
def dense_ff(h, W):
    return (torch.relu(h @ W["gate"].T) * (h @ W["up"].T)) @ W["down"].T


def route(z, r):
    """Router logits of ONE token -> [(expert, weight)]: sigmoid scores; a group of neighbours is ranked by the sum
    of its two largest scores and only the best `keep` groups stay; the `top` largest scores among them, divided by
    their sum, times `scale`."""
    s = torch.sigmoid(z)
    X = s.numel()
    gr = r.get("groups") or {}
    count = gr.get("count", 1)
    allowed = list(range(X))
    if count > 1:
        per = X // count
        rank = []
        for g in range(count):
            part = sorted((float(s[e]) for e in range(g * per, (g + 1) * per)), reverse=True)
            rank.append((sum(part[:2]), -g))
        best = sorted(range(count), key=lambda g: rank[g], reverse=True)[:gr.get("keep", count)]
        allowed = [e for e in range(X) if e // per in best]
    chosen = sorted(allowed, key=lambda e: (float(s[e]), -e), reverse=True)[:r["top"]]
    total = sum(float(s[e]) for e in chosen) + 1e-20
    return [(e, float(s[e]) / total * r["scale"]) for e in chosen]


def moe_ff(h, W, f):
    out = torch.zeros_like(h)
    z = h @ W["router"].T
    for t in range(h.shape[0]):
        for e, wt in route(z[t], f["router"]):
            E = sub(W, f"e{e}.")
            out[t] += wt * ((silu(h[t] @ E["gate"].T) * (h[t] @ E["up"].T)) @ E["down"].T)
    return out


# --------------------------------------------------------------------------------------------- model
def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def layer_order(cfg):
    """[(layer, opens a pass)] in execution order."""
    L = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(L)]
    a, b = loop["start"], loop["stop"]
    order = [(i, False) for i in range(a)]
    for _ in range(loop["times"]):
        order += [(i, i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, L)]


def forward(cfg, tensors, tokens):
    """Returns (logits [n, V], residual stream after every layer run [runs, n, E])."""
    T = {k: v.to(F64) for k, v in tensors.items()}
    eps = cfg["norm"]["eps"]
    x0 = T["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0.clone()
    after = []
    for i, opens in layer_order(cfg):
        ent, L = cfg["layers"][i], sub(T, f"l{i}.")
        if opens:
            x = torch.cat([x, x0], -1) @ T["loop.in"].T
        x = x + MIXERS[ent["type"]](rms_norm(x, L["norm1"], eps), sub(L, "mix."), ent["mixer"], eps)
        f = ent.get("mlp")
        if f:
            h = rms_norm(x, L["norm2"], eps)
            if f["kind"] == "dense":
                x = x + dense_ff(h, sub(L, "mlp."))
            elif f["kind"] == "moe":
                x = x + moe_ff(h, sub(L, "mlp."), f)
            else:
                raise ValueError("unknown feed-forward kind")
        after.append(x.clone())
    z = rms_norm(x, T["final.norm"], eps) @ T["head"].T
    return z, torch.stack(after)
