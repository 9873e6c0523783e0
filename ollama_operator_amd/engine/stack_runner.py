"""Runner of layer-list models (models/config.py StackConfig): heterogeneous layers, each with its own
sequence mixer (paged softmax attention, or retention with a per-sequence state matrix) and a routed
feed-forward, optionally with a span of layers that runs several times over the same weights.

`StackRunner` is a `Runner`: sequences, the paged block pool, prefill chunking, batched admission, decode
graphs, the sampler and the scheduler interface are the base class's. What differs is what a step runs
(`forward`: the stack executor, csrc/stack) and what a sequence owns:

* every layer RUN (a repeated layer counts once per pass) has its own cache: attention runs share the
  sequence's block table and own a K and a V pool [blocks][kv_heads][block][dim | vdim] (with several maps per
  head a K row holds them side by side; with scores mixed across the heads the K pool has one head whose row
  holds every key/value head's key); retention runs own a float32 state [slots][heads][dim][vdim], indexed by
  the sequence's block-table row (its slot);
* a slot's states are cleared when a sequence takes it, and a sequence with state keeps a cached prefix
  only whole (a state cannot be cut back), never a shorter one;
* the residual stream is float32; matrices and the K/V pools are bfloat16 (`dtype="bfloat16"`) or
  float32 (`dtype="float32"`: everything exact, FMA matrix products).

On a GPU the executor is the HIP one and nothing else; the torch twin (ops/reference.py
TorchStackExecutor) runs the same buffers on the CPU for the host-logic tests.
"""
from __future__ import annotations

import os
import time

import torch

from ..models.config import (BLOCK_POSTNORM, BLOCK_PRENORM, BLOCK_SANDWICH, FF_DENSE, FF_GLU, MIX_ATTENTION, MIX_LATENT,
                             MIX_MAMBA2, MIX_MLSTM, MIX_RETENTION)
from .runner import Runner
from .weights import StackWeights

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "f32": torch.float32}


class StackExec:
    """Adapter: runner buffers -> the native stack executor (`_stack.Executor`, csrc/stack)."""

    def __init__(self, r: "StackRunner"):
        from ..ops import stack_native
        C = stack_native()
        self.r = r
        self.exe = e = C.Executor()
        w, cfg = r.w, r.cfg
        self._f64 = []  # float64 rotary tables (kept alive here: the executor holds raw pointers)
        p = lambda t: t.data_ptr() if t is not None else 0  # noqa: E731
        e.configure(dict(E=cfg.n_embd, V=cfg.n_vocab, eps=float(cfg.norm_eps), residual_mult=float(cfg.residual_mult),
                         logit_softcap=float(cfg.logit_softcap), f32=int(w.dtype == torch.float32),
                         max_B=r.max_batch, max_seqs=r.max_seqs, block=int(cfg.block), embed_scale=float(cfg.embed_scale),
                         logit_scale=float(cfg.logit_scale), canon_taps=int(cfg.canon_taps)))
        e.set_globals(dict(embed=p(w.embed), loop_in=p(w.loop_in), final_w=p(w.final_w), final_b=p(w.final_b),
                           head=p(w.head)))
        for i, (L, spec) in enumerate(zip(w.layers, cfg.layers)):
            m, f = spec.mixer, spec.mlp
            if cfg.block == BLOCK_SANDWICH:
                e.set_layer(i, self._sandwich_layer(L, spec, p))
                continue
            if cfg.block == BLOCK_PRENORM:
                e.set_layer(i, self._prenorm_layer(L, spec, p))
                continue
            d = dict(kind=m.kind, heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale,
                     softcap=m.softcap, qtemp_coef=m.qtemp_coef, qtemp_every=m.qtemp_every, rot_dims=m.rot_dims,
                     n_in=L["n_in"], norm_w=p(L["norm_w"]), norm_b=p(L["norm_b"]), w_in=p(L["w_in"]), w_o=p(L["w_o"]),
                     decay=p(L.get("decay")), inv_freq=p(L.get("inv_freq")),
                     **{"off_" + k: v for k, v in L["off"].items()})
            if f is not None and f.kind == FF_DENSE:
                d.update(ff=f.ff, ff_dense=1, w_dense_down=p(L["w_dense_down"]))
            elif f is not None:
                d.update(experts=f.experts, top=f.top, ff=f.ff, shared_ff=f.shared_ff, router_b=p(L["router_b"]),
                         w_gu=p(L["w_gu"]), w_down=p(L["w_down"]), sh_down=p(L.get("sh_down")), identity=f.identity,
                         group_count=f.group_count, group_keep=f.group_keep)
            if cfg.block == BLOCK_POSTNORM:  # norms on the sublayers' outputs: the feed-forward has its own input stack
                if m.kind == MIX_LATENT and m.rot_dims:
                    self._f64.append(L["inv_freq"].double().contiguous())
                d.update(norm2_w=p(L.get("norm2_w")), norm2_b=p(L.get("norm2_b")), w_ff=p(L.get("w_ff")), n_ff=L["n_ff"],
                         rot_dim=m.rot_dim, kv_rank=m.kv_rank, dkv_norm=p(L.get("dkv_norm")), w_uk=p(L.get("w_uk")),
                         w_uvT=p(L.get("w_uvT")), w_ukT=p(L.get("w_ukT")), w_uv=p(L.get("w_uv")), sink=p(L.get("sink")),
                         gate_cap=m.gate_cap, i_b=p(L.get("i_b")),
                         f_b=p(L.get("f_b")), mnorm=p(L.get("mnorm")), state=m.state, groups=m.groups, conv=m.conv,
                         norm_groups=m.norm_groups, conv_w=p(L.get("conv_w")), conv_b=p(L.get("conv_b")),
                         dt_bias=p(L.get("dt_bias")), a_log=p(L.get("a_log")), d_skip=p(L.get("d_skip")),
                         inv_freq64=p(self._f64[-1]) if m.kind == MIX_LATENT and m.rot_dims else 0, inv_freq=0)
            e.set_layer(i, d)
        e.set_runs([dict(layer=li, opens_pass=int(first), kc=p(r.kc[ri]), vc=p(r.vc[ri]), state=p(r.states[ri]),
                         state_stride=(r.states[ri].shape[1] if r.states[ri] is not None and r.states[ri].dim() == 2 else 0))
                    for ri, (li, _ps, first) in enumerate(r.runs)])
        e.set_workspace(dict(resid=p(r.resid), x0=p(r.x0), h=p(r.hbuf), cat=p(r.catbuf), proj=p(r.proj),
                             ld_proj=r.proj.shape[1], a=p(r.abuf), ld_a=r.abuf.shape[1], hmid=p(r.hmid),
                             ld_hmid=r.hmid.shape[1], y=p(r.ybuf), eids=p(r.eids), ew=p(r.ew), ld_top=r.eids.shape[1],
                             sgate=p(r.sgate), lrows=p(r.lbuf), obuf=p(r.obuf), ld_obuf=r.obuf.shape[1],
                             split_ws=p(r.split_ws), split_ws_floats=r.split_ws.numel(),
                             ret_chunks=p(r.d_chunks), ret_max_chunks=r.d_chunks.shape[0], ret_u=p(r.ret_u),
                             ret_sin=p(r.ret_sin), ret_u_stride=r.ret_u.shape[1], cbuf=p(r.cbuf), ld_cbuf=r.cbuf.shape[1],
                             lat=p(r.latbuf), ld_lat=r.latbuf.shape[1], idw=p(r.idw), coef=p(r.scan_coef),
                             ld_coef=(r.scan_coef.shape[1] if r.scan_coef is not None else 0), ctot=p(r.scan_ctot),
                             hn=p(r.hn), y2=p(r.ybuf2),
                             **{"moe_" + k: (v if isinstance(v, int) else p(v)) for k, v in r.moe_ws.items()}))
        e.set_inputs(dict(tokens=p(r.d_tokens), pos=p(r.d_pos), slot=p(r.d_slot), q_len=p(r.d_qlen),
                          q_seq=p(r.d_qseq), block_table=p(r.d_block_table), max_blocks=r.max_blocks,
                          bs=r.block_size, logits=p(r.logits), ld_logits=r.logits.shape[1],
                          logit_idx=p(r.d_logit_idx)))
        self.stages = dict(forward=C.ST_FORWARD, embed=C.ST_EMBED, run=C.ST_RUN, head=C.ST_HEAD)
        self.chunk_rows = C.retention_chunk_rows()
        self.tile_rows = C.FLASH_TILE_ROWS
        e.bind_tiles(p(r.d_tiles), r.d_tiles.shape[0])

    @staticmethod
    def _sandwich_layer(L: dict, spec, p) -> dict:
        """Descriptor of a layer with scalar-weight norms around both sublayers (csrc/stack LayerDesc)."""
        m, f = spec.mixer, spec.mlp
        d = dict(kind=m.kind, heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale, rot_dims=m.rot_dims,
                 n_in=L["n_in"], w_in=p(L["w_in"]), w_o=p(L["w_o"]), in_b=p(L["in_b"]), o_b=p(L["o_b"]),
                 norm_w=p(L["norm1"]), norm_b=p(L["norm1b"]), ls1=p(L["ls1"]), canon=p(L["canon"]),
                 inv_freq64=p(L["inv_freq64"]), q_norm=p(L.get("q_norm")), k_norm=p(L.get("k_norm")), qk_norm=int(m.qk_norm),
                 sink=p(L.get("sink")), talk=p(L.get("talk")), v_from_k=int(m.v_from_k),
                 **{"off_" + k: v for k, v in L["off"].items() if k in ("q", "k", "v", "g")})
        if m.right is not None:
            g = m.right
            d.update(r_heads=g.heads, r_dim=g.dim, r_vdim=g.vdim, r_tau=g.tau, r_rank=g.decay_rank, off_rq=L["off"]["rq"],
                     off_rk=L["off"]["rk"], off_rv=L["off"]["rv"], off_a1=L["off"]["a1"], a2=p(L["a2"]), a2_b=p(L["a2_b"]),
                     gnorm=p(L["gnorm"]), w_o2=p(L["w_o2"]), left_scale=m.left_scale, right_scale=m.right_scale)
        if f is not None:
            if f.kind != FF_GLU:
                raise ValueError("a sandwich layer's feed-forward is the gated dense one")
            d.update(ff=f.ff, ff_dense=2, w_ff=p(L["w_ff"]), n_ff=L["n_ff"], w_dense_down=p(L["w_dense_down"]),
                     norm2_w=p(L["norm2"]), norm2_b=p(L["norm2b"]), ls2=p(L["ls2"]))
        return d

    @staticmethod
    def _prenorm_layer(L: dict, spec, p) -> dict:
        """Descriptor of a layer with RMS norms on the inputs of both sublayers (csrc/stack LayerDesc)."""
        m, f = spec.mixer, spec.mlp
        d = dict(kind=m.kind, heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale, rot_dims=m.rot_dims,
                 n_in=L["n_in"], w_in=p(L["w_in"]), w_o=p(L["w_o"]), norm_w=p(L["norm_w"]), inv_freq64=p(L["inv_freq64"]),
                 window=m.window, maps=m.maps, diff=m.diff, lam=L.get("lam", 0.0), gate=int(m.gate), talk=p(L.get("talk")),
                 score_talk=int(m.score_talk), rot_dim=m.rot_dim, kv_rank=m.kv_rank, dkv_norm=p(L.get("dkv_norm")),
                 w_uk=p(L.get("w_uk")), w_uvT=p(L.get("w_uvT")), w_ukT=p(L.get("w_ukT")), w_uv=p(L.get("w_uv")),
                 **{"off_" + k: v for k, v in L["off"].items() if k in ("q", "k", "v", "g", "router")})
        if f is not None:
            d.update(norm2_w=p(L["norm2_w"]), w_ff=p(L["w_ff"]), n_ff=L["n_ff"], ff=f.ff)
            if f.kind == FF_GLU:
                d.update(ff_dense=3, w_dense_down=p(L["w_dense_down"]))
            else:
                d.update(experts=f.experts, top=f.top, w_gu=p(L["w_gu"]), w_down=p(L["w_down"]), group_count=f.group_count,
                         group_keep=f.group_keep, route_scale=f.route_scale)
        return d

    def bind_chunks(self, rows) -> None:
        """The row tables of the next step: `rows` = (positions, sequence rows) of its B rows as the host
        uploaded them, or None (the device advanced the rows itself: decode steps). Each sequence's contiguous
        rows are cut into retention chunks {first row, rows, state slot, first | last flags} and attention query
        tiles {first row, rows}; without tables the step takes the per-row kernels."""
        r = self.r
        self.exe.set_chunks(0)
        self.exe.set_tiles(0)
        if rows is None or len(rows[0]) <= 16:
            return
        _pos, qseq = rows
        B, segs, a = len(qseq), [], 0
        for i in range(1, B + 1):
            if i == B or qseq[i] != qseq[a]:
                segs.append((a, i))
                a = i
        C, T = self.chunk_rows, self.tile_rows
        chunks = [(c0, min(C, i - c0), int(qseq[a]), (1 if c0 == a else 0) | (2 if c0 + C >= i else 0))
                  for a, i in segs for c0 in range(a, i, C)] if r.cfg.has_state else []
        tiles = [(t0, min(T, i - t0)) for a, i in segs for t0 in range(a, i, T)]
        if chunks and len(chunks) <= r.d_chunks.shape[0]:
            r.d_chunks[:len(chunks)].copy_(torch.tensor(chunks, dtype=torch.int32))
            self.exe.set_chunks(len(chunks))
        if len(tiles) <= r.d_tiles.shape[0]:
            r.d_tiles[:len(tiles)].copy_(torch.tensor(tiles, dtype=torch.int32))
            self.exe.set_tiles(len(tiles))

    def run(self, stage: str, layer: int, B: int, n_logits: int = 0, use_idx: bool = False, prefill: bool = False):
        if stage in ("forward", "embed"):  # a new step: its rows as the host uploaded them, if it did
            rows, self.r._step_rows = self.r._step_rows, None
            rows = rows if rows is not None and len(rows[0]) == B else None
            self.bind_chunks(rows)
            # decode attention: blocks per (row, head) by the longest context of the step. A batch-1 step says
            # it itself (`_decode_S`, part of its graph's key); other steps by the rows the host uploaded
            S = self.r._decode_S or (self.r.decode_splits(max(rows[0]) + 1) if rows is not None else 1)
            self.exe.set_splits(max(1, S))
        self.exe.step(self.stages[stage], layer, B, n_logits, use_idx, torch.cuda.current_stream().cuda_stream)


class StackRunner(Runner):
    def __init__(self, model_path: str, device: str | None = None, max_batch: int = 256, max_seqs: int = 4,
                 ctx: int | None = None, block_size: int = 16, dtype: str = "bfloat16", kv_tokens: int = 0,
                 use_graphs: bool | None = None, weights: StackWeights | None = None, cpu_backend: str | None = None):
        """kv_tokens: tokens the block pool holds for all live sequences together (0: every slot at
        `ctx`). ctx: longest sequence (default: the pool, or 4096). max_seqs: state slots = live sequences."""
        t0 = time.perf_counter()
        if device is None:
            device = f"cuda:{torch.cuda.current_device()}" if torch.cuda.is_available() else "cpu"
        self.device = dev = torch.device(device)
        self.is_gpu = dev.type == "cuda"
        if self.is_gpu:
            self._sampler_module()  # fail loudly: no torch fallback on a GPU box
        self.tp_rank, self.tp_size, self.tp_group, self.tp_ctrl, self.ar = 0, 1, None, None, None
        self._closed = False
        self.dtype = _DTYPES[dtype] if isinstance(dtype, str) else dtype
        self.w = weights or StackWeights(model_path, dev, self.dtype)
        cfg = self.cfg = self.w.cfg
        self.runs = cfg.runs()
        self.max_batch, self.max_seqs, self.block_size = max_batch, max_seqs, block_size
        self.ctx = min(ctx or kv_tokens or 4096, cfg.ctx_len)
        self.max_blocks = (self.ctx + block_size - 1) // block_size
        n_blocks = self.pool_blocks(kv_tokens)
        E, V, T = cfg.n_embd, cfg.n_vocab, self.dtype
        f32 = dict(device=dev, dtype=torch.float32)
        i32 = dict(device=dev, dtype=torch.int32)
        tt = dict(device=dev, dtype=T)
        # one cache per layer run
        self.kc, self.vc, self.states = [], [], []
        for li, _ps, _first in self.runs:
            m = cfg.layers[li].mixer
            if cfg.block == BLOCK_SANDWICH:  # K/V pools, and one state row per slot: [second mixer's matrix | input window]
                self.kc.append(torch.zeros(n_blocks, m.kv_heads, block_size, m.dim, **tt))
                self.vc.append(torch.zeros(n_blocks, m.kv_heads, block_size, m.vdim, **tt))
                ns = cfg.run_state_floats(li)
                self.states.append(torch.zeros(max_seqs, ns, **f32) if ns else None)
            elif m.kind == MIX_ATTENTION and m.score_talk:  # one K row per token: every key/value head's key side by side
                self.kc.append(torch.zeros(n_blocks, 1, block_size, m.kv_heads * m.dim, **tt))
                self.vc.append(torch.zeros(n_blocks, m.kv_heads, block_size, m.vdim, **tt))
                self.states.append(None)
            elif m.kind == MIX_ATTENTION:                   # (with two maps per head a K row holds [map 1 | map 2])
                self.kc.append(torch.zeros(n_blocks, m.kv_heads, block_size, m.dim * m.maps, **tt))
                self.vc.append(torch.zeros(n_blocks, m.kv_heads, block_size, m.vdim, **tt))
                self.states.append(None)
            elif m.kind == MIX_LATENT:  # one row per token: latent | shared rotated key part (the latent is the value too)
                self.kc.append(torch.zeros(n_blocks, 1, block_size, m.cache_dim, **tt))
                self.vc.append(None)
                self.states.append(None)
            elif m.kind == MIX_RETENTION:
                self.kc.append(None)
                self.vc.append(None)
                self.states.append(torch.zeros(max_seqs, m.heads, m.dim, m.vdim, **f32))
            else:  # mLSTM: matrix memory | normaliser | running maximum; Mamba-2: state | the convolution's last inputs
                self.kc.append(None)
                self.vc.append(None)
                self.states.append(torch.zeros(max_seqs, m.state_floats, **f32))
        mlps = [s.mlp for s in cfg.layers if s.mlp is not None]
        top = max([f.top for f in mlps] + [1])
        self.resid = torch.zeros(max_batch, E, **f32)
        self.x0 = torch.zeros(max_batch, E, **f32)          # the embedding output (re-enters at every pass)
        self.hbuf = torch.zeros(max_batch, E, **tt)         # normed activations, the input projection's operand
        self.catbuf = torch.zeros(max_batch, 2 * E, **tt)   # [x; x0], the pass-opening projection's operand
        n_proj = max(max(L["n_in"], L.get("n_ff", 0)) for L in self.w.layers)
        self.proj = torch.zeros(max_batch, (n_proj + 3) // 4 * 4, **f32)  # rows 16-byte aligned
        self.abuf = torch.zeros(max_batch, (max(s.mixer.n_out_all for s in cfg.layers) + 7) // 8 * 8, **tt)
        self.hmid = torch.zeros(max_batch, (max([f.ff if f.kind in (FF_DENSE, FF_GLU) else f.top * f.ff + f.shared_ff for f in mlps],
                                                default=1) + 7) // 8 * 8, **tt)
        # latent attention: queries folded onto the latent (float32), outputs in latent space (matrix dtype);
        # Mamba-2: the convolution's output (float32). idw: per-row weight of the chosen identity experts
        lat = [s.mixer for s in cfg.layers if s.mixer.kind == MIX_LATENT]
        mam = [s.mixer for s in cfg.layers if s.mixer.kind == MIX_MAMBA2]
        talk = [s.mixer for s in cfg.layers if s.mixer.talk]  # every query head against every key/value head's values
        fold = [s.mixer for s in cfg.layers if s.mixer.score_talk]  # queries folded through the score-mixing matrix
        maps = [s.mixer for s in cfg.layers if s.mixer.maps > 1]    # the maps' outputs before they are combined
        self.cbuf = torch.zeros(max_batch, (max([m.heads * m.cache_dim for m in lat] + [m.conv_channels for m in mam] +
                                                [m.heads * m.kv_heads * m.vdim for m in talk] +
                                                [m.heads * m.kv_heads * m.dim for m in fold] +
                                                [m.heads * m.maps * m.vdim for m in maps], default=1) + 3) // 4 * 4, **f32)
        sandwich = cfg.block == BLOCK_SANDWICH
        self.hn = torch.zeros(max_batch if sandwich else 1, E, **f32)      # normed rows before the input convolution
        self.ybuf2 = torch.zeros(max_batch if sandwich else 1, E, **f32)   # the second mixer's projected output
        self.latbuf = torch.zeros(max_batch, (max([m.heads * m.kv_rank for m in lat], default=1) + 7) // 8 * 8, **tt)
        self.idw = torch.zeros(max_batch, **f32)
        self.ybuf = torch.zeros(max_batch, E, **f32)
        self.eids = torch.zeros(max_batch, top, **i32)
        self.ew = torch.zeros(max_batch, top, **f32)
        self.sgate = torch.zeros(max_batch, **f32)
        self.lbuf = torch.zeros(max_batch, E, **tt)
        # state mixers' outputs before their norm (the mLSTM's with its normaliser's column per head)
        self.obuf = torch.zeros(max_batch, max(max(s.mixer.heads * (s.mixer.vdim + (s.mixer.kind == MIX_MLSTM)),
                                                   s.mixer.right.n_out if s.mixer.right is not None else 0)
                                               for s in cfg.layers), **f32)
        # chunked retention of prompt portions: the chunk table and one state per chunk (its U, its incoming state)
        rets = [s.mixer for s in cfg.layers if s.mixer.kind in (MIX_RETENTION, MIX_MLSTM, MIX_MAMBA2)]
        glas = [s.mixer.right for s in cfg.layers if s.mixer.right is not None]  # gated linear attention beside attention
        rets += glas
        n_ch = max_batch // 32 + max_seqs + 1 if rets and max_batch > 16 else 1
        self.d_chunks = torch.zeros(n_ch, 4, **i32)
        self.d_tiles = torch.zeros(max_batch // 32 + max_seqs + 1, 2, **i32)  # attention query tiles of a step
        self.ret_u = torch.zeros(n_ch, max([m.heads * m.dim * (m.vdim + (m.kind == MIX_MLSTM)) for m in rets], default=1)
                                 if n_ch > 1 else 1, **f32)
        # chunked gated scans: the rows' {ln decay, input weight, running maximum} per head, the chunks' summed ln decay
        hmax = max([m.heads for m in rets if m.kind != MIX_RETENTION], default=0) if n_ch > 1 else 0
        # (gated linear attention: the rows' running log decays, one per head and key channel)
        self.scan_coef = torch.zeros(max_batch, max([3 * hmax] + ([m.n_q for m in glas] if n_ch > 1 else [])), **f32) if hmax else None
        self.scan_ctot = torch.zeros(n_ch, hmax, **f32) if hmax else None
        self.ret_sin = torch.zeros_like(self.ret_u)
        # decode attention over long contexts: partials {maximum, sum, output} of up to 16 splits per (row, head)
        hv = max([s.mixer.heads * s.mixer.maps * (s.mixer.kv_heads if s.mixer.talk else 1) * (s.mixer.vdim + 2) for s in cfg.layers
                  if s.mixer.kind == MIX_ATTENTION] +
                 [s.mixer.heads * (s.mixer.kv_rank + 2) for s in cfg.layers if s.mixer.kind == MIX_LATENT], default=1)
        self.split_ws = torch.zeros(16 * 16 * hv, **f32)
        self._step_rows = None  # (positions, sequence rows) of the rows last uploaded, until a step consumes them
        # routed feed-forward of prompt portions (bfloat16): pairs sorted by expert, per-expert matrix-core products
        self.moe_ws = {}
        if mlps and T == torch.bfloat16:
            pairs = max_batch * top
            tiles = pairs // 64 + max(f.experts for f in mlps) + 1
            self.moe_ws = dict(rank=torch.zeros(pairs, **i32), srow=torch.zeros(pairs, **i32), inv=torch.zeros(pairs, **i32),
                               tiles=torch.zeros(3 * tiles, **i32), ntiles=torch.zeros(1, **i32),
                               gu=torch.zeros(pairs, 2 * max(f.ff for f in mlps), **f32),
                               hs=torch.zeros(pairs, max(f.ff for f in mlps), **tt), ds=torch.zeros(pairs, E, **f32),
                               max_pairs=pairs, max_tiles=tiles)
        self.mfma_bytes = self.lib_min = self.moe_lib = 0
        self.w16 = self.mb_bufs = self.x8_bufs = None
        self._alloc_step_state(V, n_blocks)
        self.decode_group, self.graph_pair, self.steps_issued = 1, False, 0
        self.ring_fence = 1 if os.environ.get("OMX_RING_FENCE", "0") == "1" else 0
        self._defer_ok, self._decode_S, self._adv_next = False, 0, None
        if self.is_gpu:
            self.exe = StackExec(self)
        else:
            from ..ops.reference import TorchStackExecutor
            self.exe = TorchStackExecutor(self)
        self.cpu_backend = None if self.is_gpu else "torch"
        if use_graphs is None:
            use_graphs = self.is_gpu and os.environ.get("OMX_NO_GRAPH", "0") != "1"
        self.use_graphs = use_graphs
        self._alloc_host_side()
        self.load_s = time.perf_counter() - t0

    def _sampler_module(self):
        from ..ops import stack_native
        return stack_native()

    # ------------------------------------------------------------------ step
    def forward(self, B: int, n_logits: int, use_idx: bool = False, prefill: bool = False):
        """One step over B rows; each row carries its own position, cache slot and sequence row, so rows of
        several sequences (portions of prompts, single decode tokens) mix freely. Rows of one sequence are
        contiguous and in position order."""
        if self._closed:
            raise RuntimeError("runner is closed")
        self.exe.run("forward", 0, B, n_logits, use_idx, prefill)

    def _upload(self, arr, tokens):
        super()._upload(arr, tokens)
        if arr.shape[1]:
            self._step_rows = (arr[0].tolist(), arr[3].tolist())

    def split_plan(self, B: int) -> tuple[int, int]:
        return 1, 0

    def decode_splits(self, length: int) -> int:
        """Blocks per (row, head) of the decode attention over `length` keys: 1 up to 512 keys, then a power of
        two with about 256 keys per block, at most 16. Batch-1 decode graphs are captured per bucket."""
        S = 1
        while S < 16 and length > 256 * S * 2:
            S *= 2
        return S

    def _output_norm(self, h: torch.Tensor) -> torch.Tensor:
        if self.w.final_b is None:
            return h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.cfg.norm_eps) * self.w.final_w
        return torch.nn.functional.layer_norm(h, (h.shape[-1],), self.w.final_w, self.w.final_b, self.cfg.norm_eps)

    # ------------------------------------------------------------------ sequences and state slots
    def _clear_slot(self, row: int) -> None:
        for st in self.states:
            if st is not None:
                st[row].zero_()

    def new_sequence(self) -> int:
        sid = super().new_sequence()
        self._clear_slot(self.kv.seqs[sid].row)
        return sid

    def reusable_prefix(self, sid: int, n: int) -> int:
        if not self.cfg.has_state:
            return n
        return n if n == self.kv.seqs[sid].length else 0

    def _keep_prefix(self, sid: int, keep: int, history: list[int]) -> None:
        s = self.kv.seqs[sid]
        if self.cfg.has_state and keep != s.length:
            if keep != 0:
                raise RuntimeError(f"sequence {sid}: a recurrent state cannot be cut back from {s.length} to {keep}")
            self._clear_slot(s.row)
        super()._keep_prefix(sid, keep, history)

    def _graph(self, B: int, steps: int = 1, inst: int = 0):
        """A graph captured in mid-generation: the warm-up forward that precedes the capture really runs, and a
        second run of the same rows would advance their recurrent states twice (a K/V write is the same write
        again, a state update is not). The states are put back after it."""
        key = (B, self._decode_S, steps, inst)
        if key in self.graphs:
            return self.graphs[key]
        saved = [st.clone() if st is not None else None for st in self.states]
        g = super()._graph(B, steps, inst)
        for st, old in zip(self.states, saved):
            if st is not None:
                st.copy_(old)
        return g

    # ------------------------------------------------------------------ load-time warm-up
    def warmup(self) -> None:
        if not self.is_gpu:
            return
        V = self.cfg.n_vocab
        for n in sorted({min(self.max_batch, 8), min(self.max_batch, 96)}):
            sid = self.new_sequence()
            try:
                self.prefill(sid, [(i * 7919 + 3) % V for i in range(n)])
            finally:
                self.free_sequence(sid)
        if self.use_graphs:  # one batch-1 decode graph per attention split bucket reachable at this context
            for S in sorted({self.decode_splits(n) for n in (1, 513, 1025, 2049, 4097, 8193) if n <= self.ctx}):
                self._decode_S = S
                self._graph(1)
            self._decode_S = 0
        torch.cuda.synchronize()


__all__ = ["StackRunner", "StackExec", "MIX_ATTENTION", "MIX_RETENTION"]
