"""Torch twin of the native step executor (csrc/runtime/executor.cpp).

Same weights (`DeviceWeights`, repacked streams), same buffers, same paged KV cache and the same
stage API (`embed`, `attn`, `ffn`, `head`), implemented with fp32 torch ops on dequantized
matrices. It is (a) the CPU serving backend (BASELINE config "phi on kind, CPU-only server"),
(b) the oracle the GPU tests compare the HIP executor against, and (c) the engine used by the
multi-process tensor-parallel tests on CPU (gloo).
"""
from __future__ import annotations

import math

import numpy as np
import torch
import torch.nn.functional as F

from ..gguf import GGMLType
from ..quant import REPACK_STREAMS, dequantize, repack_row_bytes, unrepack


def dequant_qmat(m) -> torch.Tensor:
    """DevQMat -> float32 [rows_total, K] on the matrix's device."""
    names = REPACK_STREAMS[GGMLType(m.qtype)]
    rows = m.streams[0].numel() // repack_row_bytes(m.qtype, m.K)[0]
    st = {n: s.detach().cpu().numpy() for n, s in zip(names, m.streams)}
    raw = unrepack(st, m.qtype, rows, m.K)
    w = dequantize(raw, m.qtype, rows * m.K).reshape(rows, m.K)
    return torch.from_numpy(w).to(m.streams[0].device)


class TorchExecutor:
    def __init__(self, runner):
        self.r = runner
        self.w = runner.w
        self._dq: dict[int, torch.Tensor] = {}

    def W(self, m) -> torch.Tensor:
        k = id(m)
        if k not in self._dq:
            self._dq[k] = dequant_qmat(m)
        return self._dq[k]

    # ------------------------------------------------------------------ helpers
    def _norm(self, x, w, b=None):
        cfg = self.w.cfg
        if cfg.arch == "phi2":
            return F.layer_norm(x, (x.shape[-1],), w, b, cfg.norm_eps)
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + cfg.norm_eps) * w

    def _rope_pairs(self, x: torch.Tensor, pos: torch.Tensor, D: int) -> torch.Tensor:
        """Rotate adjacent pairs (2i, 2i+1) for in-head dims < n_rot; x: [B, nh*D]."""
        n_rot = self.w.cfg.n_rot
        B = x.shape[0]
        x = x.view(B, -1, D).clone()
        inv = self.w.inv_freq.to(x.device)
        ang = pos.to(torch.float32)[:, None] * inv[None, :]  # [B, n_rot/2]
        cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        x0, x1 = x[..., 0:n_rot:2].clone(), x[..., 1:n_rot:2].clone()
        x[..., 0:n_rot:2] = x0 * cos - x1 * sin
        x[..., 1:n_rot:2] = x0 * sin + x1 * cos
        return x.view(B, -1)

    # ------------------------------------------------------------------ stages
    def embed(self, B: int):
        r = self.r
        toks = r.d_tokens[:B].long()
        r.resid[:B] = self.W(self.w.tok_embd)[toks.clamp(min=0)] * self.w.cfg.embed_scale
        ext = toks < 0  # external embedding rows -(id + 1) (image patches), unscaled
        if bool(ext.any()):
            r.resid[:B][ext] = r.ext[(-toks[ext] - 1)].to(r.resid.dtype)

    def attn(self, i: int, B: int):
        r, w = self.r, self.w
        L = w.layers[i]
        loc = w.local
        D, H, Hkv = loc["D"], loc["H"], loc["Hkv"]
        Eq, Ekv = H * D, Hkv * D
        x = r.resid[:B]
        xn = self._norm(x, L["attn_norm"], L.get("attn_norm_b"))
        qkv = xn @ self.W(L["wqk"]).T
        if "wv" in L:
            qkv = torch.cat([qkv, xn @ self.W(L["wv"]).T], dim=1)
        if L.get("qkv_bias") is not None:
            qkv = qkv + L["qkv_bias"]
        pos = r.d_pos[:B].long()
        q = self._rope_pairs(qkv[:, :Eq], pos, D)
        k = self._rope_pairs(qkv[:, Eq:Eq + Ekv], pos, D)
        v = qkv[:, Eq + Ekv:Eq + 2 * Ekv]
        slot = r.d_slot[:B].long()
        bs = r.block_size
        kc, vc = r.kc[i], r.vc[i]
        blk, off = slot // bs, slot % bs
        kc[blk, :, off] = k.view(B, Hkv, D).to(kc.dtype)
        vc[blk, :, off] = v.view(B, Hkv, D).to(vc.dtype)
        if w.cfg.arch == "phi2":
            r.hbuf[:B, :loc["F"]] = self._gelu(xn @ self.W(L["wgu"]).T + L["bup"])
        out = torch.empty(B, Eq, device=x.device)
        G = H // Hkv
        scale = 1.0 / math.sqrt(D)
        window = w.cfg.sliding_window
        for b in range(B):
            n = int(r.d_qlen[b])
            row = int(r.d_qseq[b])
            start = max(0, n - window) if window else 0
            bt = r.d_block_table[row].long()
            t = torch.arange(start, n, device=x.device)
            kk = kc[bt[t // bs], :, t % bs].float()  # [n, Hkv, D]
            vv = vc[bt[t // bs], :, t % bs].float()
            qq = q[b].view(H, D)
            kk = kk.repeat_interleave(G, dim=1)
            vv = vv.repeat_interleave(G, dim=1)
            s = torch.einsum("hd,thd->ht", qq, kk) * scale
            p = torch.softmax(s, dim=-1)
            out[b] = torch.einsum("ht,thd->hd", p, vv).reshape(-1)
        r.abuf[:B] = out
        o = out @ self.W(L["wo"]).T
        if L.get("bo") is not None:
            o = o + L["bo"]
        if r.tp_size > 1:
            r.ypart[:B] = o
        else:
            r.resid[:B] += o

    @staticmethod
    def _gelu(x):
        return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x.pow(3))))

    def ffn(self, i: int, B: int):
        r, w = self.r, self.w
        L = w.layers[i]
        loc = w.local
        Fl = loc["F"]
        cfg = w.cfg
        if cfg.arch == "phi2":
            y = r.hbuf[:B, :Fl] @ self.W(L["wdown"]).T
            if L.get("bdown") is not None:
                y = y + L["bdown"]
        else:
            xn = self._norm(r.resid[:B], L["ffn_norm"])
            if cfg.n_expert:
                X, k = cfg.n_expert, cfg.n_expert_used
                logits = xn @ self.W(L["router"]).T
                probs = torch.softmax(logits, dim=-1)
                tw, ti = probs.topk(k, dim=-1)
                tw = tw / tw.sum(-1, keepdim=True)
                GU = self.W(L["gu_exps"]).view(X, 2 * Fl, -1)
                DN = self.W(L["down_exps"]).view(X, w.local["E"], -1)
                y = torch.zeros_like(xn)
                for b in range(B):
                    for j in range(k):
                        e = int(ti[b, j])
                        gu = GU[e] @ xn[b]
                        h = F.silu(gu[0::2]) * gu[1::2]
                        y[b] += tw[b, j] * (DN[e] @ h)
            else:
                gu = xn @ self.W(L["wgu"]).T
                act = self._gelu if cfg.gelu_glu else F.silu
                h = act(gu[:, 0::2]) * gu[:, 1::2]
                y = h @ self.W(L["wdown"]).T
        if r.tp_size > 1:
            r.ypart[:B] = y
        else:
            r.resid[:B] += y

    def head(self, n_logits: int, use_idx: bool):
        r, w = self.r, self.w
        if n_logits <= 0:
            return
        x = r.resid[r.d_logit_idx[:n_logits].long()] if use_idx else r.resid[:n_logits]
        xn = self._norm(x, w.out_norm, w.out_norm_b)
        lg = xn @ self.W(w.lm_head).T
        if w.lm_bias is not None:
            lg = lg + w.lm_bias
        r.logits[:n_logits, :lg.shape[1]] = lg

    def run(self, stage: str, layer: int, B: int, n_logits: int = 0, use_idx: bool = False,
            prefill: bool = False):
        if stage == "embed":
            self.embed(B)
        elif stage == "attn":
            self.attn(layer, B)
        elif stage == "ffn":
            self.ffn(layer, B)
        elif stage == "head":
            self.head(n_logits, use_idx)
        elif stage == "forward":
            self.embed(B)
            for i in range(self.w.cfg.n_layer):
                self.attn(i, B)
                self.ffn(i, B)
            self.head(n_logits, use_idx)
        else:
            raise ValueError(stage)


def np_to_i32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.int32)


# ---------------------------------------------------------------------------------------------------
# Torch twin of the stack executor (csrc/stack/stack_executor.cpp): the same buffers, the same places
# where activations are rounded to the matrix dtype, float32 everywhere else. One function per kernel,
# so a GPU test can compare kernel by kernel.

def stack_matmul(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """a [M, K] and w [N, K] in the matrix dtype -> float32 [M, N] (products exact, float32 sums)."""
    return a.float() @ w.float().T


def stack_query_temperature(pos: torch.Tensor, coef: float, every: int) -> torch.Tensor:
    return 1.0 + coef * torch.log(torch.floor((pos.float() + 1.0) / float(every)) + 1.0)


def stack_attention(q, kc, vc, block_table, q_seq, q_len, bs, scale, softcap, groups):
    """q [B, H, D] float32; kc [blocks, G, bs, D], vc [blocks, G, bs, Dv]; row b sees the first q_len[b]
    keys of sequence row q_seq[b]. Returns float32 [B, H, Dv]."""
    B, H, _ = q.shape
    out = torch.empty(B, H, vc.shape[-1], dtype=torch.float32, device=q.device)
    for b in range(B):
        n = int(q_len[b])
        t = torch.arange(n, device=q.device)
        bt = block_table[int(q_seq[b])].long()
        kk = kc[bt[t // bs], :, t % bs].float().repeat_interleave(groups, dim=1)  # [n, H, D]
        vv = vc[bt[t // bs], :, t % bs].float().repeat_interleave(groups, dim=1)
        s = torch.einsum("hd,thd->ht", q[b], kk) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        out[b] = torch.einsum("ht,thd->hd", torch.softmax(s, -1), vv)
    return out


def stack_rotate_half(x, pos, inv_freq):
    """x [B, H, D] float32: dims i and i + R/2 (R = 2 * len(inv_freq)) rotate by pos * inv_freq[i]."""
    half = inv_freq.numel()
    ang = pos.float()[:, None] * inv_freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], -1)


def stack_retention(q, k, v, state, q_seq, decay):
    """q, k [B, H, D], v [B, H, Dv] float32, rows in sequence order; state [slots, H, D, Dv] is read and
    advanced in place: S <- decay S + k v^T, o = S^T q. Returns float32 [B, H, Dv]."""
    B = q.shape[0]
    out = torch.empty_like(v)
    for b in range(B):
        S = state[int(q_seq[b])]
        S.mul_(decay[:, None, None]).add_(k[b][:, :, None] * v[b][:, None, :])
        out[b] = torch.einsum("hdv,hd->hv", S, q[b])
    return out


def stack_route(z: torch.Tensor, top: int):
    """Router logits [B, X] -> (expert ids [B, top] by descending logit, softmax over the chosen logits)."""
    val, idx = torch.topk(z, top, dim=-1)
    return idx.to(torch.int32), torch.softmax(val, -1)


# ---- layers whose norm sits on the sublayer's output (BLOCK_POSTNORM): latent attention, mLSTM, Mamba-2,
# dense and score-routed feed-forwards. One function per kernel of csrc/stack/stack_mixers.hip.

def stack_post_norm_add(x, y, w, b, eps, idw=None):
    """x += layer_norm(y + idw * x) * w + b (idw: per-row weight of the identity experts, or None)."""
    if idw is not None:
        y = y + idw[:, None] * x
    x += F.layer_norm(y, (y.shape[-1],), w, b, eps)


def stack_rotate_pairs(x, pos, inv_freq):
    """x [B, ..., R] float32: dims (2i, 2i + 1), i < len(inv_freq), turn by pos * inv_freq[i] (float64 angles)."""
    n = inv_freq.numel()
    ang = pos.double()[:, None] * inv_freq.double()[None, :]
    while ang.dim() < x.dim():
        ang = ang.unsqueeze(1)
    c, s = torch.cos(ang).float(), torch.sin(ang).float()
    u, v = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
    out = x.clone()
    out[..., 0:2 * n:2] = u * c - v * s
    out[..., 1:2 * n:2] = v * c + u * s
    return out


def stack_latent_prepare(proj, off, m, L, pos, slot, cache, bs, eps):
    """The cached row of every token, [rms_norm(latent) * w | rotated shared key part], stored at its slot; returns
    the queries folded onto the latent: per head [W_uk_h^T q_plain | rotated q part], float32 [B, H, C + R]."""
    B, H, D, R, C = proj.shape[0], m.heads, m.dim, m.rot_dim, m.kv_rank
    q = proj[:, off["q"]:off["q"] + H * (D + R)].view(B, H, D + R)
    dkv = proj[:, off["k"]:off["k"] + C + R]
    c = dkv[:, :C] * torch.rsqrt(dkv[:, :C].pow(2).mean(-1, keepdim=True) + eps) * L["dkv_norm"]
    kr, qr = dkv[:, C:], q[..., D:]
    if L["inv_freq"] is not None:
        kr, qr = stack_rotate_pairs(kr, pos, L["inv_freq"]), stack_rotate_pairs(qr, pos, L["inv_freq"])
    blk, o = slot.long() // bs, slot.long() % bs
    cache[blk, 0, o] = torch.cat([c, kr], 1).to(cache.dtype)
    qa = torch.einsum("bhd,hdc->bhc", q[..., :D], L["w_uk"].float().view(H, D, C))
    return torch.cat([qa, qr], -1)


def stack_latent_attention(qa, cache, C, block_table, q_seq, q_len, bs, scale, sink):
    """qa [B, H, C + R]; cache [blocks, 1, bs, C + R]; the first C dims of a cached row are also its value.
    softmax with exp(sink_h) added to the denominator. Returns float32 [B, H, C]."""
    B, H, _ = qa.shape
    out = torch.empty(B, H, C, dtype=torch.float32, device=qa.device)
    for b in range(B):
        n = int(q_len[b])
        t = torch.arange(n, device=qa.device)
        bt = block_table[int(q_seq[b])].long()
        kk = cache[bt[t // bs], 0, t % bs].float()            # [n, C + R]
        s = (qa[b] @ kk.T) * scale                            # [H, n]
        mx = torch.maximum(s.max(-1, keepdim=True).values, sink[:, None])
        e = torch.exp(s - mx)
        out[b] = (e / (e.sum(-1, keepdim=True) + torch.exp(sink[:, None] - mx))) @ kk[:, :C]
    return out


def stack_conv_silu(xin, w, bias, state, q_seq):
    """Causal per-channel convolution over each sequence's rows, continued from `state` [slots, taps - 1, ch]
    (the sequence's last inputs, oldest first), which is advanced in place. xin [B, ch] -> silu(conv) [B, ch]."""
    B, K = xin.shape[0], w.shape[1]
    out = torch.empty_like(xin)
    for b in range(B):
        st = state[int(q_seq[b])]
        win = torch.cat([st, xin[b:b + 1]], 0)                 # [K, ch], last row = the current token
        out[b] = F.silu((win * w.T).sum(0) + bias)
        if K > 1:
            st.copy_(win[1:])
    return out


def stack_gated_scan(q, k, v, a, b, S, q_seq, kv_group=1):
    """S [slots, H, D, Dv] <- a S + b k v^T per row (a, b [B, H]), o = S^T q. q, k [B, G, D] with head h using
    group h // kv_group; v [B, H, Dv]. Returns float32 [B, H, Dv]."""
    B, H = a.shape
    out = torch.empty_like(v)
    hg = torch.arange(H, device=v.device) // kv_group
    for r in range(B):
        St = S[int(q_seq[r])]
        St.mul_(a[r][:, None, None]).add_((b[r][:, None] * k[r][hg])[:, :, None] * v[r][:, None, :])
        out[r] = torch.einsum("hdv,hd->hv", St, q[r][hg])
    return out


def stack_mlstm_gates(i_raw, f_raw, cap, m_state, q_seq):
    """Per row and head: decay a = exp(f + m' - m), input weight b = exp(i - m) with m = max(f + m', i), m' the
    running maximum of the sequence (m_state [slots, H], advanced in place). Returns a, b, m [B, H]."""
    ig = cap * torch.tanh(i_raw / cap)
    fg = F.logsigmoid(cap * torch.tanh(f_raw / cap))
    a, b, mm = torch.empty_like(ig), torch.empty_like(ig), torch.empty_like(ig)
    for r in range(ig.shape[0]):
        mp = m_state[int(q_seq[r])]
        mn = torch.maximum(fg[r] + mp, ig[r])
        a[r], b[r], mm[r] = torch.exp(fg[r] + mp - mn), torch.exp(ig[r] - mn), mn
        mp.copy_(mn)
    return a, b, mm


def stack_group_rms(y, groups, w, eps, gate=None):
    """y [B, n] in `groups` equal parts, each divided by its root mean square; times w; times sigmoid(gate)."""
    B, n = y.shape
    g = y.view(B, groups, n // groups)
    o = (g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps)).reshape(B, n) * w
    return o * torch.sigmoid(gate) if gate is not None else o


def stack_route_scores(z, corr, top, n_real, group_count, group_keep):
    """Router logits [B, X + I] -> softmax scores; the `top` largest of score + correction within the best
    `group_keep` of `group_count` neighbour groups (a group's rank: its largest corrected score). Returns expert
    ids [B, top] (identity choices point at expert 0 with weight 0), weights [B, top] and the summed weight of
    the chosen identity outputs [B]."""
    s = torch.softmax(z, -1)
    choice = s + corr
    if group_count > 1:
        per = z.shape[1] // group_count
        best = choice.view(-1, group_count, per).max(-1).values
        keep = torch.topk(best, group_keep, dim=-1).indices
        ok = torch.zeros_like(best, dtype=torch.bool).scatter_(1, keep, True)
        choice = choice.masked_fill(~ok.repeat_interleave(per, dim=1), -float("inf"))
    ids = torch.topk(choice, top, dim=-1).indices
    wt = torch.gather(s, 1, ids)
    ident = ids >= n_real
    idw = (wt * ident).sum(-1)
    return torch.where(ident, 0, ids).to(torch.int32), torch.where(ident, 0.0, wt), idw



# ---- layers with scalar-weight RMS norms around both sublayers (BLOCK_SANDWICH): an input convolution with a
# carried window, attention with biases / rotation with scaled frequencies / query and key norms / sinks / mixing of
# the heads' weights, gated linear attention beside it, a gated feed-forward. One function per kernel of
# csrc/stack/stack_sandwich.hip.

def stack_scalar_norm(x, g, eps):
    """x / sqrt(mean(x^2) + eps) * g with one number g for all coordinates."""
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * g


def stack_canon_conv(hn, w, window, q_seq):
    """hn [B, E] + causal per-channel convolution over each sequence's rows (w [E, taps], the last tap is the
    current token's), continued from `window` [slots, taps - 1, E] (the sequence's last inputs, oldest first),
    which is advanced in place."""
    B, K = hn.shape[0], w.shape[1]
    out = torch.empty_like(hn)
    for b in range(B):
        st = window[int(q_seq[b])]
        win = torch.cat([st, hn[b:b + 1]], 0)                  # [K, E]
        out[b] = hn[b] + (win * w.T).sum(0)
        if K > 1:
            st.copy_(win[1:])
    return out


def stack_rotate_half64(x, pos, inv_freq):
    """x [B, H, D] float32: dims i and i + n (n = len(inv_freq)) turn by pos * inv_freq[i]; float64 angles."""
    n = inv_freq.numel()
    ang = pos.double()[:, None] * inv_freq.double()[None, :]
    c, s = torch.cos(ang).float()[:, None, :], torch.sin(ang).float()[:, None, :]
    u, v = x[..., :n], x[..., n:2 * n]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * n:]], -1)


def stack_qk_prepare(q, k, m, L, pos, eps):
    """Queries [B, H, D] and keys [B, G, D] (biases added): RMS norm with a weight before the rotation, or unit RMS
    after it, as the mixer says."""
    def unit(t):
        return t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps)
    if m.qk_norm == 1:
        q, k = unit(q) * L["q_norm"], unit(k) * L["k_norm"]
    if m.rot_dims:
        q, k = stack_rotate_half64(q, pos, L["inv_freq64"]), stack_rotate_half64(k, pos, L["inv_freq64"])
    if m.qk_norm == 2:
        q, k = unit(q), unit(k)
    return q, k


def stack_attention_sink(q, kc, vc, block_table, q_seq, q_len, bs, scale, groups, sink, talk):
    """Softmax attention over the paged pools with exp(sink_h) in the denominator (sink None: none). With `talk`
    [H, H] the heads' weights are mixed, w_h <- sum_g talk[h, g] w_g, before head h meets the values of its own
    key/value head. Returns float32 [B, H, Dv]."""
    B, H, _ = q.shape
    out = torch.empty(B, H, vc.shape[-1], dtype=torch.float32, device=q.device)
    for b in range(B):
        n = int(q_len[b])
        t = torch.arange(n, device=q.device)
        bt = block_table[int(q_seq[b])].long()
        kk = kc[bt[t // bs], :, t % bs].float().repeat_interleave(groups, dim=1)  # [n, H, D]
        vv = vc[bt[t // bs], :, t % bs].float().repeat_interleave(groups, dim=1)
        s = torch.einsum("hd,thd->ht", q[b], kk) * scale
        mx = s.max(-1, keepdim=True).values
        if sink is not None:
            mx = torch.maximum(mx, sink[:, None])
        e = torch.exp(s - mx)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[:, None] - mx)
        w = e / den
        if talk is not None:
            w = talk @ w
        out[b] = torch.einsum("ht,thd->hd", w, vv)
    return out


def stack_gla(q, k, v, alpha, S, q_seq):
    """S [slots, H, D, Dv] <- diag(alpha) S + k v^T per row (alpha [B, H, D]), o = S^T q. Returns float32 [B, H, Dv]."""
    out = torch.empty_like(v)
    for r in range(q.shape[0]):
        St = S[int(q_seq[r])]
        St.mul_(alpha[r][:, :, None]).add_(k[r][:, :, None] * v[r][:, None, :])
        out[r] = torch.einsum("hdv,hd->hv", St, q[r])
    return out


def stack_gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z ** 3)))


def stack_sandwich_add(x, y, g, ls, eps):
    """x += ls * (y / rms(y) * g): the scalar-weight norm on a sublayer's result, then the per-channel scale."""
    x += ls * stack_scalar_norm(y, g, eps)



# ---- layers with RMS norms (weight vectors) on the sublayers' inputs (BLOCK_PRENORM): sliding-window attention with two
# differential maps per head or with scores mixed across the heads, latent attention with a gate per head, a gated dense
# feed-forward, a sigmoid router with group ranking. One function per kernel of csrc/stack/stack_prenorm.hip.

def stack_rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w with a weight per coordinate."""
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w


def stack_attention_window(q, kc, vc, block_table, q_seq, q_len, bs, scale, window, k_off, v_head):
    """q [B, Hq, D] float32. kc [blocks, Gk, bs, Wk]: query head h reads D elements at k_off[h] of the rows of key
    head h // (Hq // Gk); vc [blocks, Gv, bs, Dv]: it meets the values of head v_head[h]. Row b sees the keys
    max(0, q_len[b] - window) .. q_len[b] - 1 of its sequence (window 0: all). Returns float32 [B, Hq, Dv]."""
    B, Hq, D = q.shape
    Gk = kc.shape[1]
    out = torch.empty(B, Hq, vc.shape[-1], dtype=torch.float32, device=q.device)
    for b in range(B):
        n = int(q_len[b])
        t = torch.arange(max(0, n - window) if window else 0, n, device=q.device)
        bt = block_table[int(q_seq[b])].long()
        kk, vv = kc[bt[t // bs], :, t % bs].float(), vc[bt[t // bs], :, t % bs].float()   # [n, G, W]
        for h in range(Hq):
            s = (kk[:, h // (Hq // Gk), k_off[h]:k_off[h] + D] @ q[b, h]) * scale
            out[b, h] = torch.softmax(s, 0) @ vv[:, v_head[h]]
    return out


def stack_diff_combine(a, lam, diff, eps, gate):
    """a [B, H, 2, Dv] (the two maps' outputs): (a1 - lam a2) / rms over Dv * (1 - diff) * sigmoid(gate [B, H * Dv])."""
    B, H, _, Dv = a.shape
    o = a[:, :, 0] - lam * a[:, :, 1]
    o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * (1.0 - diff)
    return o.reshape(B, H * Dv) * torch.sigmoid(gate)


def stack_rotate_fold(q, k, pos, inv_freq, mix, groups):
    """q [B, H, D], k [B, G, D]: adjacent-pair rotation of both, then the queries are folded through the score-mixing
    matrix: qf[b, h] = [sum over the heads g of key/value head c of mix[h, g] q[b, g], for every c], so that
    qf[b, h] . [k_0 | ... | k_(G-1)] is head h's mixed score. Returns (qf [B, H, G * D], rotated k [B, G, D])."""
    B, H, D = q.shape
    G = k.shape[1]
    if inv_freq is not None:
        q, k = stack_rotate_pairs(q, pos, inv_freq), stack_rotate_pairs(k, pos, inv_freq)
    qf = torch.einsum("hcj,bcjd->bhcd", mix.view(H, G, groups), q.view(B, G, groups, D))
    return qf.reshape(B, H, G * D), k


def stack_route_sigmoid(z, top, group_count, group_keep, scale):
    """Router logits [B, X] -> sigmoid scores; a group of neighbours ranks by the sum of its two largest scores and
    only the best `group_keep` groups stay; the `top` largest scores among them (ties: the lower index), divided by
    their sum (+ 1e-20), times `scale`. Returns expert ids [B, top] int32 and weights [B, top]."""
    s = torch.sigmoid(z)
    choice = s
    if group_count > 1:
        per = z.shape[1] // group_count
        best = torch.topk(s.view(-1, group_count, per), min(2, per), dim=-1).values.sum(-1)
        keep = torch.topk(best, group_keep, dim=-1).indices
        ok = torch.zeros_like(best, dtype=torch.bool).scatter_(1, keep, True)
        choice = s.masked_fill(~ok.repeat_interleave(per, dim=1), -1.0)
    ids = torch.topk(choice, top, dim=-1).indices
    wt = torch.gather(s, 1, ids)
    return ids.to(torch.int32), wt / (wt.sum(-1, keepdim=True) + 1e-20) * scale


class TorchStackExecutor:
    def __init__(self, runner):
        self.r = runner

    def embed(self, B: int):
        r = self.r
        x = r.w.embed[r.d_tokens[:B].long()].float() * float(getattr(r.cfg, "embed_scale", 1.0))
        r.resid[:B] = x
        r.x0[:B] = x

    def layer_run(self, ri: int, B: int):
        from ..models.config import BLOCK_POSTNORM, BLOCK_PRENORM, BLOCK_SANDWICH, MIX_ATTENTION
        r = self.r
        w, cfg, T = r.w, r.cfg, r.w.dtype
        if cfg.block == BLOCK_PRENORM:
            return self.layer_run_prenorm(ri, B)
        if cfg.block == BLOCK_POSTNORM:
            return self.layer_run_postnorm(ri, B)
        if cfg.block == BLOCK_SANDWICH:
            return self.layer_run_sandwich(ri, B)
        li, _ps, opens = r.runs[ri]
        L, spec = w.layers[li], cfg.layers[li]
        m, f, off = spec.mixer, spec.mlp, L["off"]
        if opens:
            r.catbuf[:B] = torch.cat([r.resid[:B], r.x0[:B]], 1).to(T)
            r.resid[:B] = stack_matmul(r.catbuf[:B], w.loop_in)
        x = r.resid[:B]
        r.hbuf[:B] = F.layer_norm(x, (x.shape[-1],), L["norm_w"], L["norm_b"], cfg.norm_eps).to(T)
        proj = stack_matmul(r.hbuf[:B], L["w_in"])
        r.proj[:B, :proj.shape[1]] = proj
        pos, qseq = r.d_pos[:B], r.d_qseq[:B]
        q = proj[:, off["q"]:off["q"] + m.n_q].view(B, m.heads, m.dim)
        k = proj[:, off["k"]:off["k"] + m.n_k].view(B, m.kv_heads, m.dim)
        v = proj[:, off["v"]:off["v"] + m.n_v].view(B, m.kv_heads, m.vdim)
        if m.kind == MIX_ATTENTION:
            if m.qtemp_coef:
                q = q * stack_query_temperature(pos, m.qtemp_coef, m.qtemp_every)[:, None, None]
            slot = r.d_slot[:B].long()
            blk, o = slot // r.block_size, slot % r.block_size
            r.kc[ri][blk, :, o] = k.to(T)
            r.vc[ri][blk, :, o] = v.to(T)
            a = stack_attention(q, r.kc[ri], r.vc[ri], r.d_block_table, qseq, r.d_qlen[:B], r.block_size, m.scale,
                                m.softcap, m.heads // m.kv_heads)
        else:
            if m.rot_dims:
                q = stack_rotate_half(q, pos, L["inv_freq"])
                k = stack_rotate_half(k, pos, L["inv_freq"])
            k = k * float(m.dim) ** -0.5
            o = stack_retention(q, k, v, r.states[ri], qseq, L["decay"])
            o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + cfg.norm_eps)
            g = proj[:, off["g"]:off["g"] + m.n_out].view(B, m.heads, m.vdim)
            a = o * F.silu(g)
        r.abuf[:B, :m.n_out] = a.reshape(B, m.n_out).to(T)
        y = stack_matmul(r.abuf[:B, :m.n_out], L["w_o"])
        if f is not None:
            z = proj[:, off["router"]:off["router"] + f.experts] + L["router_b"]
            ids, wt = stack_route(z, f.top)
            r.eids[:B, :f.top], r.ew[:B, :f.top] = ids, wt
            h = r.hbuf[:B]
            ff = torch.zeros_like(y)
            for b in range(B):
                for j in range(f.top):
                    e = int(ids[b, j])
                    gu = stack_matmul(h[b:b + 1], L["w_gu"][e])[0]
                    mid = (F.silu(gu[:f.ff]) * gu[f.ff:]).to(T)
                    ff[b] += wt[b, j] * stack_matmul(mid[None], L["w_down"][e])[0]
            if f.shared_ff:
                Fs = f.shared_ff
                mid = (F.silu(proj[:, off["sgate"]:off["sgate"] + Fs]) * proj[:, off["sup"]:off["sup"] + Fs]).to(T)
                ff += torch.sigmoid(proj[:, off["sg"]:off["sg"] + 1]) * stack_matmul(mid, L["sh_down"])
            y = y + ff
        r.resid[:B] = x + cfg.residual_mult * y

    def layer_run_postnorm(self, ri: int, B: int):
        """x <- x + LN1(mixer(x)), then x <- x + LN2(ff(x)); both sublayers read the stream itself."""
        from ..models.config import FF_DENSE, MIX_LATENT, MIX_MAMBA2, MIX_MLSTM
        r = self.r
        w, cfg, T = r.w, r.cfg, r.w.dtype
        li = r.runs[ri][0]
        L, spec = w.layers[li], cfg.layers[li]
        m, f, off = spec.mixer, spec.mlp, L["off"]
        H, D, Dv, n_out = m.heads, m.dim, m.vdim, m.n_out
        x = r.resid[:B]
        pos, qseq = r.d_pos[:B], r.d_qseq[:B]
        r.hbuf[:B] = x.to(T)
        proj = stack_matmul(r.hbuf[:B], L["w_in"])
        r.proj[:B, :proj.shape[1]] = proj
        if m.kind == MIX_LATENT:
            C = m.kv_rank
            qa = stack_latent_prepare(proj, off, m, L, pos, r.d_slot[:B], r.kc[ri], r.block_size, cfg.norm_eps)
            lat = stack_latent_attention(qa, r.kc[ri], C, r.d_block_table, qseq, r.d_qlen[:B], r.block_size, m.scale,
                                         L["sink"])
            r.latbuf[:B, :H * C] = lat.reshape(B, H * C).to(T)
            o = torch.einsum("bhc,hcv->bhv", r.latbuf[:B, :H * C].float().view(B, H, C), L["w_uvT"].float().view(H, C, Dv))
            a = o.reshape(B, n_out) * torch.sigmoid(proj[:, off["g"]:off["g"] + n_out])
        elif m.kind == MIX_MLSTM:
            st = r.states[ri]
            nS = H * D * Dv
            S, nv, ms = st[:, :nS].view(-1, H, D, Dv), st[:, nS:nS + H * D].view(-1, H, D, 1), st[:, nS + H * D:]
            q = proj[:, off["q"]:off["q"] + H * D].view(B, H, D) * float(D) ** -0.5
            k = proj[:, off["k"]:off["k"] + H * D].view(B, H, D)
            v = proj[:, off["v"]:off["v"] + n_out].view(B, H, Dv)
            ga, gb, mm = stack_mlstm_gates(proj[:, off["i"]:off["i"] + H] + L["i_b"], proj[:, off["f"]:off["f"] + H] + L["f_b"],
                                           m.gate_cap, ms, qseq)
            o = stack_gated_scan(q, k, v, ga, gb, S, qseq)
            nq = stack_gated_scan(q, k, torch.ones(B, H, 1), ga, gb, nv, qseq)
            o = o / (torch.maximum(nq.abs(), torch.exp(-mm)[..., None]) + 1e-6)
            a = stack_group_rms(o.reshape(B, n_out), H, L["mnorm"], cfg.norm_eps, proj[:, off["g"]:off["g"] + n_out])
        else:
            assert m.kind == MIX_MAMBA2
            st = r.states[ri]
            N, G, ch = m.state, m.groups, m.conv_channels
            nS = H * N * Dv
            S, cst = st[:, :nS].view(-1, H, N, Dv), st[:, nS:].view(st.shape[0], m.conv - 1, ch)
            xbc = stack_conv_silu(proj[:, off["conv"]:off["conv"] + ch], L["conv_w"].view(ch, m.conv), L["conv_b"], cst, qseq)
            xs = xbc[:, :n_out].view(B, H, Dv)
            Bm = xbc[:, n_out:n_out + G * N].view(B, G, N)
            Cm = xbc[:, n_out + G * N:].view(B, G, N)
            dt = F.softplus(proj[:, off["dt"]:off["dt"] + H] + L["dt_bias"])
            ga = torch.exp(-torch.exp(L["a_log"]) * dt)
            y = stack_gated_scan(Cm, Bm, xs, ga, dt, S, qseq, kv_group=H // G) + L["d_skip"][None, :, None] * xs
            y = y.reshape(B, n_out) * F.silu(proj[:, off["g"]:off["g"] + n_out])
            a = stack_group_rms(y, m.norm_groups, L["mnorm"], cfg.norm_eps)
        r.abuf[:B, :n_out] = a.to(T)
        r.ybuf[:B] = stack_matmul(r.abuf[:B, :n_out], L["w_o"])
        stack_post_norm_add(x, r.ybuf[:B], L["norm_w"], L["norm_b"], cfg.norm_eps)
        if f is None:
            return
        r.hbuf[:B] = x.to(T)
        h = r.hbuf[:B]
        proj = stack_matmul(h, L["w_ff"])
        r.proj[:B, :proj.shape[1]] = proj
        idw = None
        if f.kind == FF_DENSE:
            r.hmid[:B, :f.ff] = torch.relu(proj).pow(2).to(T)
            y = stack_matmul(r.hmid[:B, :f.ff], L["w_dense_down"])
        else:
            ids, wt, idw = stack_route_scores(proj[:, :f.n_router], L["router_b"], f.top, f.experts, f.group_count,
                                              f.group_keep)
            r.eids[:B, :f.top], r.ew[:B, :f.top] = ids, wt
            y = torch.zeros_like(x)
            for b in range(B):
                for j in range(f.top):
                    if float(wt[b, j]) == 0.0:
                        continue
                    e = int(ids[b, j])
                    gu = stack_matmul(h[b:b + 1], L["w_gu"][e])[0]
                    mid = (F.silu(gu[:f.ff]) * gu[f.ff:]).to(T)
                    y[b] += wt[b, j] * stack_matmul(mid[None], L["w_down"][e])[0]
            if f.shared_ff:
                Fs = f.shared_ff
                mid = (F.silu(proj[:, off["sgate"]:off["sgate"] + Fs]) * proj[:, off["sup"]:off["sup"] + Fs]).to(T)
                y += stack_matmul(mid, L["sh_down"])
        r.ybuf[:B] = y
        stack_post_norm_add(x, r.ybuf[:B], L["norm2_w"], L["norm2_b"], cfg.norm_eps, idw)

    def layer_run_prenorm(self, ri: int, B: int):
        """x <- x + mixer(N1(x)), then x <- x + ff(N2(x)), N an RMS norm with a weight vector; a pass of a repeated span
        opens with x <- W_in [x; x0]."""
        from ..models.config import FF_GLU, MIX_LATENT
        r = self.r
        w, cfg, T = r.w, r.cfg, r.w.dtype
        li, _ps, opens = r.runs[ri]
        L, spec = w.layers[li], cfg.layers[li]
        m, f, off, eps = spec.mixer, spec.mlp, L["off"], cfg.norm_eps
        H, G, D, Dv, n_out = m.heads, m.kv_heads, m.dim, m.vdim, m.n_out
        if opens:
            r.catbuf[:B] = torch.cat([r.resid[:B], r.x0[:B]], 1).to(T)
            r.resid[:B] = stack_matmul(r.catbuf[:B], w.loop_in)
        x = r.resid[:B]
        pos, qseq, qlen, bs = r.d_pos[:B], r.d_qseq[:B], r.d_qlen[:B], r.block_size
        slot = r.d_slot[:B].long()
        blk, o = slot // bs, slot % bs
        r.hbuf[:B] = stack_rms_norm(x, L["norm_w"], eps).to(T)
        proj = stack_matmul(r.hbuf[:B], L["w_in"])
        r.proj[:B, :proj.shape[1]] = proj
        if m.kind == MIX_LATENT:
            C = m.kv_rank
            qa = stack_latent_prepare(proj, off, m, dict(L, inv_freq=L["inv_freq64"]), pos, r.d_slot[:B], r.kc[ri], bs, eps)
            lat = stack_latent_attention(qa, r.kc[ri], C, r.d_block_table, qseq, qlen, bs, m.scale,
                                         torch.full((H,), -float("inf"), device=qa.device))
            r.latbuf[:B, :H * C] = lat.reshape(B, H * C).to(T)
            ov = torch.einsum("bhc,hcv->bhv", r.latbuf[:B, :H * C].float().view(B, H, C), L["w_uvT"].float().view(H, C, Dv))
            a = (ov * torch.sigmoid(proj[:, off["g"]:off["g"] + H])[:, :, None]).reshape(B, n_out)
        else:
            q = proj[:, off["q"]:off["q"] + m.n_q]
            k = proj[:, off["k"]:off["k"] + m.n_k]
            r.vc[ri][blk, :, o] = proj[:, off["v"]:off["v"] + m.n_v].view(B, G, Dv).to(T)
            if m.maps == 2:  # two maps per head: the K pool's rows hold [map 1 | map 2] of a key/value head
                r.kc[ri][blk, :, o] = k.view(B, G, 2 * D).to(T)
                a2 = stack_attention_window(q.view(B, 2 * H, D), r.kc[ri], r.vc[ri], r.d_block_table, qseq, qlen, bs, m.scale,
                                            m.window, [(h % 2) * D for h in range(2 * H)], [h // 2 // (H // G) for h in range(2 * H)])
                a = stack_diff_combine(a2.view(B, H, 2, Dv), L["lam"], m.diff, eps, proj[:, off["g"]:off["g"] + n_out])
            else:            # mixed scores: one K row per token holds every key/value head's key side by side
                qf, kr = stack_rotate_fold(q.view(B, H, D), k.view(B, G, D), pos, L["inv_freq64"], L["talk"].view(H, H), H // G)
                r.cbuf[:B, :H * G * D] = qf.reshape(B, H * G * D)
                r.kc[ri][blk, 0, o] = kr.reshape(B, G * D).to(T)
                a = stack_attention_window(qf, r.kc[ri], r.vc[ri], r.d_block_table, qseq, qlen, bs, m.scale, m.window,
                                           [0] * H, [h // (H // G) for h in range(H)]).reshape(B, n_out)
        r.abuf[:B, :n_out] = a.to(T)
        x += stack_matmul(r.abuf[:B, :n_out], L["w_o"])
        if f is None:
            return
        r.hbuf[:B] = stack_rms_norm(x, L["norm2_w"], eps).to(T)
        h = r.hbuf[:B]
        proj = stack_matmul(h, L["w_ff"])
        r.proj[:B, :proj.shape[1]] = proj
        if f.kind == FF_GLU:
            r.hmid[:B, :f.ff] = (torch.relu(proj[:, :f.ff]) * proj[:, f.ff:2 * f.ff]).to(T)
            x += stack_matmul(r.hmid[:B, :f.ff], L["w_dense_down"])
            return
        ids, wt = stack_route_sigmoid(proj[:, :f.experts], f.top, f.group_count, f.group_keep, f.route_scale)
        r.eids[:B, :f.top], r.ew[:B, :f.top] = ids, wt
        y = torch.zeros_like(x)
        for b in range(B):
            for j in range(f.top):
                e = int(ids[b, j])
                gu = stack_matmul(h[b:b + 1], L["w_gu"][e])[0]
                mid = (F.silu(gu[:f.ff]) * gu[f.ff:]).to(T)
                y[b] += wt[b, j] * stack_matmul(mid[None], L["w_down"][e])[0]
        x += y

    def layer_run_sandwich(self, ri: int, B: int):
        """x <- x + s1 N1b(mixer(conv_in(N1(x)))), then x <- x + s2 N2b(ff(N2(x)))."""
        r = self.r
        w, cfg, T = r.w, r.cfg, r.w.dtype
        li = r.runs[ri][0]
        L, spec = w.layers[li], cfg.layers[li]
        m, f, off, E, eps = spec.mixer, spec.mlp, L["off"], cfg.n_embd, cfg.norm_eps
        x = r.resid[:B]
        pos, qseq = r.d_pos[:B], r.d_qseq[:B]
        st = r.states[ri]
        hn = stack_scalar_norm(x, L["norm1"], eps)
        r.hn[:B] = hn
        taps = cfg.canon_taps
        if taps > 1:
            nS = st.shape[1] - (taps - 1) * E
            window = st[:, nS:].view(st.shape[0], taps - 1, E)
        else:  # one tap: a per-channel factor on the current token, nothing carried
            window = torch.zeros(r.max_seqs, 0, E, device=hn.device)
        hn = stack_canon_conv(hn, L["canon"].view(E, taps), window, qseq)
        r.hbuf[:B] = hn.to(T)
        proj = stack_matmul(r.hbuf[:B], L["w_in"])
        r.proj[:B, :proj.shape[1]] = proj
        H, G, D, Dv = m.heads, m.kv_heads, m.dim, m.vdim
        bias = L["in_b"]
        q = (proj[:, off["q"]:off["q"] + H * D] + bias[off["q"]:off["q"] + H * D]).view(B, H, D)
        k = (proj[:, off["k"]:off["k"] + G * D] + bias[off["k"]:off["k"] + G * D]).view(B, G, D)
        v = k if m.v_from_k else (proj[:, off["v"]:off["v"] + G * Dv] + bias[off["v"]:off["v"] + G * Dv]).view(B, G, Dv)
        q, kk = stack_qk_prepare(q, k, m, L, pos, eps)
        slot = r.d_slot[:B].long()
        blk, o = slot // r.block_size, slot % r.block_size
        r.kc[ri][blk, :, o] = kk.to(T)
        r.vc[ri][blk, :, o] = v.to(T)
        a = stack_attention_sink(q, r.kc[ri], r.vc[ri], r.d_block_table, qseq, r.d_qlen[:B], r.block_size, m.scale, H // G,
                                 L.get("sink"), L["talk"].view(H, H) if m.talk else None)
        n1 = m.n_out
        r.abuf[:B, :n1] = a.reshape(B, n1).to(T)
        y = stack_matmul(r.abuf[:B, :n1], L["w_o"])
        if L["o_b"] is not None:
            y = y + L["o_b"]
        if m.right is not None:
            g = m.right
            Hr, Dr, Dvr, n2 = g.heads, g.dim, g.vdim, g.n_out
            rq = proj[:, off["rq"]:off["rq"] + Hr * Dr].view(B, Hr, Dr) * float(Dr) ** -0.5
            rk = proj[:, off["rk"]:off["rk"] + Hr * Dr].view(B, Hr, Dr)
            rv = proj[:, off["rv"]:off["rv"] + n2].view(B, Hr, Dvr)
            z = proj[:, off["a1"]:off["a1"] + g.decay_rank] @ L["a2"].float().T + L["a2_b"]
            alpha = torch.exp(F.logsigmoid(z) / g.tau).view(B, Hr, Dr)
            S = st[:, :Hr * Dr * Dvr].view(-1, Hr, Dr, Dvr)
            o2 = stack_gla(rq, rk, rv, alpha, S, qseq)
            o2 = o2 * torch.rsqrt(o2.pow(2).mean(-1, keepdim=True) + eps) * L["gnorm"]
            r.abuf[:B, n1:n1 + n2] = (o2.reshape(B, n2) * F.silu(proj[:, off["g"]:off["g"] + n2])).to(T)
            y = m.left_scale * y + m.right_scale * stack_matmul(r.abuf[:B, n1:n1 + n2], L["w_o2"])
        stack_sandwich_add(x, y, L["norm1b"], L["ls1"], eps)
        if f is None:
            return
        r.hbuf[:B] = stack_scalar_norm(x, L["norm2"], eps).to(T)
        proj = stack_matmul(r.hbuf[:B], L["w_ff"])
        r.proj[:B, :proj.shape[1]] = proj
        r.hmid[:B, :f.ff] = (stack_gelu_tanh(proj[:, :f.ff]) * proj[:, f.ff:2 * f.ff]).to(T)
        stack_sandwich_add(x, stack_matmul(r.hmid[:B, :f.ff], L["w_dense_down"]), L["norm2b"], L["ls2"], eps)

    def head(self, n_logits: int, use_idx: bool):
        r = self.r
        if n_logits <= 0:
            return
        w, cfg = r.w, r.cfg
        x = r.resid[r.d_logit_idx[:n_logits].long()] if use_idx else r.resid[:n_logits]
        if cfg.block == 3:  # BLOCK_PRENORM: an RMS norm with a weight vector
            r.lbuf[:n_logits] = stack_rms_norm(x, w.final_w, cfg.norm_eps).to(w.dtype)
            z = stack_matmul(r.lbuf[:n_logits], w.head)
            r.logits[:n_logits, :z.shape[1]] = z
            return
        if w.final_b is None:  # an RMS norm with one number as its weight, and a plain factor on the logits
            r.lbuf[:n_logits] = stack_scalar_norm(x, w.final_w, cfg.norm_eps).to(w.dtype)
            z = stack_matmul(r.lbuf[:n_logits], w.head) * float(cfg.logit_scale)
            r.logits[:n_logits, :z.shape[1]] = z
            return
        r.lbuf[:n_logits] = F.layer_norm(x, (x.shape[-1],), w.final_w, w.final_b, cfg.norm_eps).to(w.dtype)
        z = stack_matmul(r.lbuf[:n_logits], w.head)
        if cfg.logit_softcap:
            z = cfg.logit_softcap * torch.tanh(z / cfg.logit_softcap)
        r.logits[:n_logits, :z.shape[1]] = z

    def run(self, stage: str, layer: int, B: int, n_logits: int = 0, use_idx: bool = False, prefill: bool = False):
        if stage == "embed":
            self.embed(B)
        elif stage == "run":
            self.layer_run(layer, B)
        elif stage == "head":
            self.head(n_logits, use_idx)
        elif stage == "forward":
            self.embed(B)
            for ri in range(len(self.r.runs)):
                self.layer_run(ri, B)
            self.head(n_logits, use_idx)
        else:
            raise ValueError(stage)
