#include "stack_executor.h"

#include <stdexcept>
#include <string>

namespace omx {
namespace stack {

static void need(bool ok, const std::string& what) {
  if (!ok) throw std::runtime_error("stack executor: " + what);
}

static void validate_postnorm(const StackExecutor& e, const RunDesc& r, const LayerDesc& L) {
  const StackWorkspace& ws = e.ws;
  need(L.kind >= 2 && L.kind <= 4, "a layer with output norms needs a latent attention, mLSTM or Mamba-2 mixer");
  need(ws.ret.ld_o >= L.heads * L.vdim && ws.ret.obuf, "mixer output wider than its float32 buffer");
  if (L.kind == 2) {
    need(r.kc && L.w_uk && L.w_uvT && L.dkv_norm && L.sink && ws.cbuf && ws.lat, "latent attention operands");
    need(latent_supported(L.dim, L.rot_dim, L.kv_rank, L.vdim),
         "latent attention sizes (dim <= 256, kv_rank <= 256, kv_rank + rot_dim <= 1024)");
    need(L.heads * (L.kv_rank + L.rot_dim) <= ws.ld_cbuf && L.heads * L.kv_rank <= ws.ld_lat, "latent attention buffers");
    need(L.rot_dims == 0 || L.inv_freq64, "latent attention rotary table missing");
  } else if (L.kind == 3) {
    need(r.state && L.i_b && L.f_b && L.mnorm && L.gate_cap > 0.f, "mLSTM operands");
    need(gated_scan_supported(SCAN_MLSTM, L.dim, L.vdim), "mLSTM head sizes (dim <= 256, vdim <= 255, dim * (vdim + 1) <= 16384)");
    need(r.state_stride >= (long long)L.heads * (L.dim * L.vdim + L.dim + 1), "mLSTM state slot too small");
  } else {
    need(r.state && L.conv_w && L.conv_b && L.dt_bias && L.a_log && L.d_skip && L.mnorm && ws.cbuf, "Mamba-2 operands");
    need(gated_scan_supported(SCAN_SSD, L.state, L.vdim), "Mamba-2 head sizes (state <= 256, vdim <= 256, state * vdim <= 16384)");
    const long long ch = (long long)L.heads * L.vdim + 2LL * L.groups * L.state;
    need(ch <= ws.ld_cbuf && L.groups > 0 && L.heads % L.groups == 0 && L.conv >= 1, "Mamba-2 convolution sizes");
    need(r.state_stride >= (long long)L.heads * L.state * L.vdim + (L.conv - 1) * ch, "Mamba-2 state slot too small");
    need(L.norm_groups > 0 && (L.heads * L.vdim) % L.norm_groups == 0, "Mamba-2 norm groups");
  }
  if (L.ff_dense) {
    need(L.w_ff && L.w_dense_down && L.norm2_w && L.norm2_b && L.ff > 0 && L.ff <= ws.ld_hmid && L.ff <= ws.ld_proj && ws.hmid,
         "dense feed-forward operands");
  } else if (L.experts) {
    need(L.w_ff && L.norm2_w && L.norm2_b && L.n_ff <= ws.ld_proj && L.top > 0 && L.top <= MOE_MAX_TOP && L.top <= ws.ld_top &&
             L.top * L.ff + L.shared_ff <= ws.ld_hmid && ws.hmid && ws.eids && ws.ew && ws.idw && L.router_b && L.w_gu &&
             L.w_down && (!L.shared_ff || (L.sh_down && ws.sgate)),
         "routed feed-forward operands");
  }
}

static void validate_sandwich(const StackExecutor& e, const RunDesc& r, const LayerDesc& L) {
  const StackWorkspace& ws = e.ws;
  const int taps = e.cfg.canon_taps;
  need(L.kind == 0 && r.kc && r.vc, "a layer with scalar norms needs an attention mixer with K/V pools");
  need(L.norm_w && L.norm_b && L.ls1 && L.w_in && L.w_o && L.n_in > 0 && L.n_in <= ws.ld_proj && ws.hn && ws.y2,
       "layer weights or buffers missing");
  need(L.dim <= 256 && L.vdim <= 256 && L.kv_heads > 0 && L.heads % L.kv_heads == 0, "attention head sizes");
  need(L.rot_dims % 2 == 0 && L.rot_dims <= L.dim && (L.rot_dims == 0 || L.inv_freq64), "rotary table missing");
  need(L.qk_norm != QK_NORM_WEIGHT_FIRST || (L.q_norm && L.k_norm), "query / key norm weights missing");
  need(!L.v_from_k || L.vdim == L.dim, "values that are the keys need vdim == dim");
  need(!L.talk || (ws.cbuf && (long long)L.heads * L.kv_heads * L.vdim <= ws.ld_cbuf), "mixed heads: float32 buffer too small");
  need(taps >= 1 && taps <= CANON_MAX_TAPS && L.canon && (taps == 1 || r.state), "input convolution (1..8 taps) operands");
  long long need_state = (long long)(taps - 1) * e.cfg.E;
  int n_out = L.heads * L.vdim;
  if (L.r_heads) {
    need(L.a2 && L.a2_b && L.gnorm && L.w_o2 && L.r_rank > 0 && L.r_tau > 0.f && r.state, "gated linear attention operands");
    need(gla_general_supported(L.r_dim, L.r_vdim), "gated linear attention head sizes (<= 256)");
    need_state += (long long)L.r_heads * L.r_dim * L.r_vdim;
    n_out += L.r_heads * L.r_vdim;
  }
  need(r.state_stride >= need_state, "state slot too small");
  need(n_out <= ws.ld_a, "mixer output wider than its buffer");
  if (L.ff_dense)
    need(L.ff_dense == 2 && L.w_ff && L.w_dense_down && L.norm2_w && L.norm2_b && L.ls2 && L.ff > 0 && L.ff <= ws.ld_hmid &&
             2 * L.ff <= ws.ld_proj && ws.hmid,
         "gated feed-forward operands");
}

static void validate_prenorm(const StackExecutor& e, const RunDesc& r, const LayerDesc& L) {
  const StackWorkspace& ws = e.ws;
  need(L.norm_w && L.w_in && L.w_o && L.n_in > 0 && L.n_in <= ws.ld_proj, "layer weights missing");
  need(L.heads * L.vdim <= ws.ld_a, "mixer output wider than its buffer");
  if (r.opens_pass) need(e.loop_in && ws.cat, "the pass-opening projection is missing");
  if (L.kind == 2) {
    need(r.kc && L.w_uk && L.w_uvT && L.dkv_norm && ws.cbuf && ws.lat && L.gate == 2, "latent attention operands");
    need(latent_supported(L.dim, L.rot_dim, L.kv_rank, L.vdim),
         "latent attention sizes (dim <= 256, kv_rank <= 256, kv_rank + rot_dim <= 1024)");
    need(L.heads * (L.kv_rank + L.rot_dim) <= ws.ld_cbuf && L.heads * L.kv_rank <= ws.ld_lat, "latent attention buffers");
    need(L.rot_dims == 0 || L.inv_freq64, "latent attention rotary table missing");
  } else {
    need(L.kind == 0 && r.kc && r.vc && L.kv_heads > 0 && L.heads % L.kv_heads == 0 && L.window >= 0, "attention run without a K/V pool");
    need(L.vdim <= 256, "attention value size (<= 256)");
    if (L.maps == 2) {
      need(L.dim <= 1024 && ws.cbuf && 2 * L.heads * L.vdim <= ws.ld_cbuf && L.gate == 1, "differential attention sizes or buffers");
    } else {
      need(L.maps == 1 && L.score_talk && L.talk && ws.cbuf && (long long)L.heads * L.kv_heads * L.dim <= ws.ld_cbuf,
           "mixed-score attention operands or buffers");
      need(rotate_fold_supported(L.heads, L.kv_heads, L.dim), "mixed-score attention sizes (kv_heads * dim <= 1024)");
      need(L.rot_dims % 2 == 0 && L.rot_dims <= L.dim && (L.rot_dims == 0 || L.inv_freq64), "rotary table missing");
    }
  }
  if (L.ff_dense) {
    need(L.ff_dense == 3 && L.w_ff && L.w_dense_down && L.norm2_w && L.ff > 0 && L.ff <= ws.ld_hmid && 2 * L.ff <= ws.ld_proj && ws.hmid,
         "gated feed-forward operands");
  } else if (L.experts) {
    need(L.w_ff && L.norm2_w && L.n_ff <= ws.ld_proj && L.top > 0 && L.top <= MOE_MAX_TOP && L.top <= ws.ld_top &&
             L.top * L.ff <= ws.ld_hmid && ws.hmid && ws.eids && ws.ew && L.w_gu && L.w_down && L.experts <= 256,
         "routed feed-forward operands (up to 256 experts)");
  }
}

void StackExecutor::validate() const {
  need(cfg.E > 0 && cfg.V > 0 && cfg.max_B > 0, "not configured");
  need(embed_w && final_w && (final_b || cfg.block >= 2) && head_w, "global weights missing");
  need(ws.resid && ws.x0 && ws.h && ws.proj && ws.a && ws.y && ws.lrows, "workspace missing");
  need(in.tokens && in.pos && in.slot && in.q_len && in.q_seq && in.block_table && in.logits, "step inputs missing");
  need(!runs.empty(), "no layer runs");
  for (const RunDesc& r : runs) {
    need(r.layer >= 0 && r.layer < (int)layers.size(), "a run names a layer that does not exist");
    const LayerDesc& L = layers[r.layer];
    if (cfg.block == 2) {
      validate_sandwich(*this, r, L);
      continue;
    }
    if (cfg.block == 3) {
      validate_prenorm(*this, r, L);
      continue;
    }
    need(L.norm_w && L.norm_b && L.w_in && L.w_o && L.n_in > 0 && L.n_in <= ws.ld_proj, "layer weights missing");
    need(L.heads * L.vdim <= ws.ld_a, "mixer output wider than its buffer");
    if (cfg.block == 1) {
      validate_postnorm(*this, r, L);
      continue;
    }
    if (r.opens_pass) need(loop_in && ws.cat, "the pass-opening projection is missing");
    if (L.kind == 0) {
      need(r.kc && r.vc, "attention run without a K/V pool");
      need(L.dim <= 256 && L.vdim <= 256 && L.kv_heads > 0 && L.heads % L.kv_heads == 0, "attention head sizes");
    } else {
      need(r.state && L.decay, "retention run without a state");
      need(retention_supported(L.dim, L.vdim) || retention_general_supported(L.dim, L.vdim), "retention head sizes (<= 1024)");
      need(L.rot_dims == 0 || L.inv_freq, "retention rotary table missing");
    }
    if (L.experts) {
      need(L.top > 0 && L.top <= MOE_MAX_TOP && L.top <= ws.ld_top && L.top * L.ff + L.shared_ff <= ws.ld_hmid && ws.hmid &&
               ws.eids && ws.ew && L.router_b && L.w_gu && L.w_down && (!L.shared_ff || (L.sh_down && ws.sgate)),
           "routed feed-forward sizes");
    }
  }
}

void StackExecutor::embed(int B, hipStream_t s) {
  h_ready = false;
  stack::embed(embed_w, in.tokens, B, cfg.E, cfg.V, ws.resid, ws.x0, cfg.embed_scale, cfg.f32, s);
}

static ScanChunkWs scan_ws(const StackExecutor& e) {
  return ScanChunkWs{e.ws.ret.chunks, e.n_chunks, e.ws.ret.max_chunks, e.ws.ret.U, e.ws.ret.Sin, e.ws.ret.u_stride, e.ws.coef,
                     e.ws.ctot, e.ws.ret.obuf, e.ws.ret.ld_o};
}
static bool chunked_scan_ok(const StackExecutor& e, const ScanParams& P, int B) {
  const int dvp = P.Dv + (P.mode == SCAN_MLSTM ? 1 : 0);
  return B > SMALL_B && e.n_chunks > 0 && e.ws.ret.U && e.ws.ret.Sin && e.ws.coef && e.ws.ctot && e.ws.ld_coef >= 3 * P.H &&
         e.ws.ret.u_stride >= (long long)P.H * P.D * dvp && e.ws.ret.ld_o >= P.H * dvp && gated_chunk_supported(P.mode, P.D, P.Dv);
}

// x <- x + LN1(mixer(x)), then x <- x + LN2(ff(x)): both sublayers read the stream itself (cast to the matrix
// dtype), the layer norm sits on their outputs.
void StackExecutor::layer_run_postnorm(int ri, int B, hipStream_t s) {
  const RunDesc& r = runs.at(ri);
  const LayerDesc& L = layers[r.layer];
  const int E = cfg.E, f32 = cfg.f32, n_out = L.heads * L.vdim;
  StepRows R{B, in.pos, in.slot, in.q_len, in.q_seq, in.block_table, in.max_blocks, in.bs};
  if (!h_ready) cast_rows(ws.resid, B, E, ws.h, f32, s);  // else the previous update left the rows in ws.h
  {  // every matrix of the mixer that reads the stream, in one product
    GemmParams g{ws.h, E, L.w_in, B, L.n_in, E, ws.proj, ws.ld_proj, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(g, s);
  }
  if (L.kind == 2) {
    const int C = L.kv_rank, W = C + L.rot_dim;
    LatentParams P{ws.proj, ws.ld_proj, L.off_q, L.off_k, L.off_g, L.heads, L.dim, L.rot_dim, C, L.vdim, L.rot_dims,
                   L.inv_freq64, L.dkv_norm, cfg.eps, L.w_uk, L.w_uvT, L.w_ukT, L.w_uv, r.kc, ws.cbuf, ws.ld_cbuf, ws.lat, ws.ld_lat, ws.a,
                   ws.ld_a, f32};
    latent_prepare(P, R, s);
    // one cached row per token serves every head: attention with a single key/value head whose key is the whole
    // row and whose value is the row's first C elements
    AttnParams A{ws.cbuf, ws.ld_cbuf, 0, 0, 0, L.heads, 1, W, C, L.scale, 0.f, 0.f, 1, r.kc, r.kc, ws.lat, ws.ld_lat, f32,
                 n_splits, ws.split_ws, ws.split_ws_floats, W, W, L.sink};
    if (B > SMALL_B && n_tiles > 0 && tiles && flash_prefill_supported(A))
      flash_prefill(A, R, tiles, n_tiles, s);  // prompt portions: query tiles on the matrix cores
    else
      attention(A, R, s);
    latent_expand(P, B, s);
  } else if (L.kind == 3) {
    ScanParams P{};
    P.mode = SCAN_MLSTM;
    P.proj = ws.proj;
    P.ld = ws.ld_proj;
    P.off_q = L.off_q;
    P.off_k = L.off_k;
    P.off_v = L.off_v;
    P.off_i = L.off_i;
    P.off_f = L.off_f;
    P.H = P.G = L.heads;
    P.D = L.dim;
    P.Dv = L.vdim;
    P.i_b = L.i_b;
    P.f_b = L.f_b;
    P.cap = L.gate_cap;
    P.state = r.state;
    P.state_stride = r.state_stride;
    P.off_g = L.off_g;
    P.y = ws.ret.obuf;
    P.ld_y = ws.ret.ld_o;
    if (chunked_scan_ok(*this, P, B)) {  // prompt portions: chunks in parallel around a scan over the chunk states
      gated_scan_chunked(P, R, scan_ws(*this), L.mnorm, cfg.eps, ws.a, ws.ld_a, f32, s);
    } else {
      gated_scan(P, R, s);
      // per-head unit RMS, the norm's weight, the sigmoid output gate
      group_rms_cast(ws.ret.obuf, ws.ret.ld_o, B, n_out, L.heads, L.mnorm, cfg.eps, ws.proj + L.off_g, ws.ld_proj, ws.a, ws.ld_a,
                     f32, s);
    }
  } else {
    const int ch = n_out + 2 * L.groups * L.state;
    ConvParams Cv{ws.proj, ws.ld_proj, L.off_conv, ch, L.conv, L.conv_w, L.conv_b,
                  r.state + (long long)L.heads * L.state * L.vdim, r.state_stride, ws.cbuf, ws.ld_cbuf};
    conv_silu(Cv, R, s);
    ScanParams P{};
    P.mode = SCAN_SSD;
    P.proj = ws.proj;
    P.ld = ws.ld_proj;
    P.conv = ws.cbuf;
    P.ld_conv = ws.ld_cbuf;
    P.off_v = 0;                                  // x | B | C
    P.off_k = n_out;
    P.off_q = n_out + L.groups * L.state;
    P.off_i = L.off_dt;
    P.off_g = L.off_g;
    P.H = L.heads;
    P.G = L.groups;
    P.D = L.state;
    P.Dv = L.vdim;
    P.dt_bias = L.dt_bias;
    P.a_log = L.a_log;
    P.d_skip = L.d_skip;
    P.state = r.state;
    P.state_stride = r.state_stride;
    P.y = ws.ret.obuf;
    P.ld_y = ws.ret.ld_o;
    if (chunked_scan_ok(*this, P, B))
      gated_scan_chunked(P, R, scan_ws(*this), nullptr, cfg.eps, nullptr, 0, f32, s);
    else
      gated_scan(P, R, s);
    group_rms_cast(ws.ret.obuf, ws.ret.ld_o, B, n_out, L.norm_groups, L.mnorm, cfg.eps, nullptr, 0, ws.a, ws.ld_a, f32, s);
  }
  {
    GemmParams o{ws.a, ws.ld_a, L.w_o, B, E, n_out, ws.y, E, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(o, s);
  }
  const bool has_ff = L.ff_dense || L.experts;
  // the updated rows leave in the matrix dtype too: the next product's operand (feed-forward, or the next layer)
  post_norm_add(ws.resid, ws.y, B, E, L.norm_w, L.norm_b, cfg.eps, nullptr, ws.h, f32, s);
  h_ready = true;
  if (!has_ff) return;
  {
    GemmParams g{ws.h, E, L.w_ff, B, L.n_ff, E, ws.proj, ws.ld_proj, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(g, s);
  }
  const float* idw = nullptr;
  if (L.ff_dense) {
    relu2_cast(ws.proj, ws.ld_proj, B, L.ff, ws.hmid, ws.ld_hmid, f32, s);
    GemmParams d{ws.hmid, ws.ld_hmid, L.w_dense_down, B, E, L.ff, ws.y, E, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(d, s);
  } else {
    MoeParams M{ws.proj, ws.ld_proj, L.off_router, 0, L.off_sgate, L.off_sup, B, E, L.experts, L.top, L.ff, L.shared_ff,
                L.router_b, ws.h, L.w_gu, L.w_down, L.sh_down, ws.eids, ws.ew, ws.ld_top, ws.sgate, ws.hmid, ws.ld_hmid, ws.y,
                f32, L.identity, L.group_count, L.group_keep, ws.idw};
    if (B <= SMALL_B && moe_route_scores_fused_supported(M)) {  // decode steps: routing + activations in one launch
      moe_route_scores_experts(M, s);
      moe_down(M, s);
    } else {
      moe_route_scores(M, s);
      if (B > SMALL_B && ws.moe.gu && moe_grouped_supported(M)) {
        moe_grouped(M, ws.moe, s);
      } else {
        moe_experts(M, s);
        moe_down(M, s);
      }
    }
    if (L.identity) idw = ws.idw;
  }
  post_norm_add(ws.resid, ws.y, B, E, L.norm2_w, L.norm2_b, cfg.eps, idw, ws.h, f32, s);
}

// x <- x + s1 N1b(mixer(conv_in(N1(x)))), then x <- x + s2 N2b(ff(N2(x))); N: RMS norm with one number as weight.
// The mixer is softmax attention (biases, rotation, query / key norms, a sink, optionally mixed heads and values that
// are the keys), optionally with a gated linear attention beside it that reads the same input.
void StackExecutor::layer_run_sandwich(int ri, int B, hipStream_t s) {
  const RunDesc& r = runs.at(ri);
  const LayerDesc& L = layers[r.layer];
  const int E = cfg.E, f32 = cfg.f32, taps = cfg.canon_taps;
  const int n1 = L.heads * L.vdim, n2 = L.r_heads * L.r_vdim;
  const long long gla_floats = (long long)L.r_heads * L.r_dim * L.r_vdim;  // the slot: [state matrix | input window]
  StepRows R{B, in.pos, in.slot, in.q_len, in.q_seq, in.block_table, in.max_blocks, in.bs};
  {
    CanonParams C{ws.resid, L.norm_w, cfg.eps, E, taps, L.canon, r.state ? r.state + gla_floats : nullptr, r.state_stride, ws.hn, ws.h,
                  f32};
    scalar_norm_conv(C, R, s);
  }
  {  // every matrix that reads the mixer's input, in one product
    GemmParams g{ws.h, E, L.w_in, B, L.n_in, E, ws.proj, ws.ld_proj, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(g, s);
  }
  {
    QkPrepParams Q{ws.proj, ws.ld_proj, L.off_q, L.off_k, L.off_v, L.in_b, L.heads, L.kv_heads, L.dim, L.vdim, L.rot_dims,
                   L.inv_freq64, L.qk_norm, L.q_norm, L.k_norm, cfg.eps, L.v_from_k, r.kc, r.vc, f32};
    qk_prepare(Q, R, s);
    AttnParams A{ws.proj, ws.ld_proj, L.off_q, L.off_k, L.off_v, L.heads, L.kv_heads, L.dim, L.vdim, L.scale, 0.f, 0.f, 1, r.kc, r.vc,
                 ws.a, ws.ld_a, f32, n_splits, ws.split_ws, ws.split_ws_floats, 0, 0, L.sink, 0, nullptr, 0};
    if (L.talk) {  // every query head's weights on every key/value head's values, in float32; then the heads are mixed
      A.vheads = L.kv_heads;
      A.out32 = ws.cbuf;
      A.ld_out32 = ws.ld_cbuf;
    }
    if (B > SMALL_B && n_tiles > 0 && tiles && flash_prefill_supported(A))
      flash_prefill(A, R, tiles, n_tiles, s);  // prompt portions: query tiles on the matrix cores
    else
      attention(A, R, s);
    if (L.talk) talk_mix(ws.cbuf, ws.ld_cbuf, B, L.heads, L.kv_heads, L.vdim, L.talk, ws.a, ws.ld_a, f32, s);
  }
  const size_t esz = f32 ? 4 : 2;
  void* a2 = (char*)ws.a + (size_t)n1 * esz;  // the second mixer's outputs sit beside the attention's
  if (L.r_heads) {
    GlaParams G{ws.proj, ws.ld_proj, L.off_rq, L.off_rk, L.off_rv, L.off_g, L.off_a1, L.r_heads, L.r_dim, L.r_vdim, L.r_rank, L.a2,
                L.a2_b, L.r_tau, L.gnorm, cfg.eps, r.state, r.state_stride, a2, ws.ld_a, f32};
    if (B > SMALL_B && n_chunks > 0 && ws.ret.U && ws.ret.Sin && ws.lna && ws.ld_coef >= L.r_heads * L.r_dim &&
        ws.ret.u_stride >= gla_floats && gla_chunk_supported(L.r_dim, L.r_vdim)) {
      GlaChunkWs W{ws.ret.chunks, n_chunks, ws.ret.max_chunks, ws.ret.U, ws.ret.Sin, ws.ret.u_stride, ws.lna, ws.ld_coef, nullptr, 0};
      gla_chunked(G, R, W, s);  // prompt portions: chunks in parallel around a scan over the chunk states
    } else {
      gla(G, R, s);
    }
  }
  const bool has_ff = L.ff_dense != 0;
  const float* g_next = has_ff ? L.norm2_w : nullptr;
  void* h_next = has_ff ? ws.h : nullptr;  // the updated rows leave normed for the feed-forward in the same launch
  if (L.r_heads && B <= 8) {  // decode steps: both output projections, their scales and the bias in one launch
    gemv_pair(ws.a, ws.ld_a, L.w_o, n1, L.o_b, L.left_scale, a2, ws.ld_a, L.w_o2, n2, L.right_scale, B, E, ws.y, E, f32, s);
    sandwich_add(ws.resid, ws.y, nullptr, 1.f, nullptr, 0.f, B, E, L.norm_b, L.ls1, cfg.eps, g_next, h_next, f32, s);
  } else {
    GemmParams o{ws.a, ws.ld_a, L.w_o, B, E, n1, ws.y, E, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(o, s);
    if (L.r_heads) {
      GemmParams o2{a2, ws.ld_a, L.w_o2, B, E, n2, ws.y2, E, EPI_STORE, 0.f, nullptr, 0.f, f32};
      gemm(o2, s);
    }
    sandwich_add(ws.resid, ws.y, L.o_b, L.r_heads ? L.left_scale : 1.f, L.r_heads ? ws.y2 : nullptr, L.right_scale, B, E, L.norm_b,
                 L.ls1, cfg.eps, g_next, h_next, f32, s);
  }
  if (!has_ff) return;
  if (B <= 8) {  // decode steps: gate / up projection and activation in one launch
    gemv_glu(ws.h, E, L.w_ff, E, L.ff, B, ws.hmid, ws.ld_hmid, f32, s);
  } else {
    GemmParams g{ws.h, E, L.w_ff, B, L.n_ff, E, ws.proj, ws.ld_proj, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(g, s);
    geglu_tanh_cast(ws.proj, ws.ld_proj, B, L.ff, ws.hmid, ws.ld_hmid, f32, s);
  }
  {
    GemmParams d{ws.hmid, ws.ld_hmid, L.w_dense_down, B, E, L.ff, ws.y, E, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(d, s);
  }
  sandwich_add(ws.resid, ws.y, nullptr, 1.f, nullptr, 0.f, B, E, L.norm2_b, L.ls2, cfg.eps, nullptr, nullptr, f32, s);
}

// x <- x + mixer(N1(x)), then x <- x + ff(N2(x)); N: RMS norm with a weight vector. A pass of a repeated span opens with
// x <- W_in [x; x0]. Mixers: attention inside a sliding window with two differential maps per head and an
// element-wise gate; attention inside a sliding window with adjacent-pair rotation and scores mixed across the heads
// before the softmax; latent attention with one gate per head.
void StackExecutor::layer_run_prenorm(int ri, int B, hipStream_t s) {
  const RunDesc& r = runs.at(ri);
  const LayerDesc& L = layers[r.layer];
  const int E = cfg.E, f32 = cfg.f32, n_out = L.heads * L.vdim;
  if (r.opens_pass) {
    concat_cast(ws.resid, ws.x0, B, E, ws.cat, f32, s);
    GemmParams g{ws.cat, 2 * E, loop_in, B, E, 2 * E, ws.resid, E, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(g, s);
  }
  StepRows R{B, in.pos, in.slot, in.q_len, in.q_seq, in.block_table, in.max_blocks, in.bs};
  const bool fused_in = gemv_ln_supported(B, E, f32);
  // differential attention: a K row of a key/value head holds its two maps side by side, so the K/V store sees heads
  // of 2 * dim
  AttnParams St{ws.proj, ws.ld_proj, L.off_q, L.off_k, L.off_v, L.heads, L.kv_heads, 2 * L.dim, L.vdim, L.scale, 0.f, 0.f, 1,
                r.kc, r.vc, ws.a, ws.ld_a, f32};
  if (fused_in) {  // decode steps: norm + every matrix that reads the mixer's input (+ that K/V store) in one launch
    gemv_ln(ws.resid, E, L.norm_w, nullptr, cfg.eps, L.w_in, B, L.n_in, ws.proj, ws.ld_proj, ws.h,
            L.kind == 0 && L.maps == 2 ? &St : nullptr, &R, f32, s);
  } else {
    rms_norm_cast(ws.resid, nullptr, B, E, L.norm_w, cfg.eps, ws.h, f32, s);
    GemmParams g{ws.h, E, L.w_in, B, L.n_in, E, ws.proj, ws.ld_proj, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(g, s);
  }
  const bool tiled = B > SMALL_B && n_tiles > 0 && tiles;
  // a window bounds the keys of a decode step: no need to share them among blocks
  const int splits = L.window > 0 && L.window <= 1024 ? 1 : n_splits;
  if (L.kind == 2) {
    const int C = L.kv_rank, W = C + L.rot_dim;
    LatentParams P{ws.proj, ws.ld_proj, L.off_q, L.off_k, L.off_g, L.heads, L.dim, L.rot_dim, C, L.vdim, L.rot_dims,
                   L.inv_freq64, L.dkv_norm, cfg.eps, L.w_uk, L.w_uvT, L.w_ukT, L.w_uv, r.kc, ws.cbuf, ws.ld_cbuf, ws.lat, ws.ld_lat, ws.a,
                   ws.ld_a, f32, 1};
    latent_prepare(P, R, s);
    AttnParams A{ws.cbuf, ws.ld_cbuf, 0, 0, 0, L.heads, 1, W, C, L.scale, 0.f, 0.f, 1, r.kc, r.kc, ws.lat, ws.ld_lat, f32,
                 n_splits, ws.split_ws, ws.split_ws_floats, W, W, nullptr};
    if (tiled && flash_prefill_supported(A))
      flash_prefill(A, R, tiles, n_tiles, s);
    else
      attention(A, R, s);
    latent_expand(P, B, s);
  } else if (L.maps == 2) {
    // the 2 * heads query maps are heads of their own
    if (!fused_in) attn_prepare(St, R, s);
    AttnParams A{ws.proj, ws.ld_proj, L.off_q, L.off_k, L.off_v, 2 * L.heads, L.kv_heads, L.dim, L.vdim, L.scale, 0.f, 0.f, 1, r.kc,
                 r.vc, ws.a, ws.ld_a, f32, splits, ws.split_ws, ws.split_ws_floats, 2 * L.dim, 0, nullptr, 0, ws.cbuf, ws.ld_cbuf,
                 L.window, 2, 0};
    if (tiled && flash_prefill_supported(A))
      flash_prefill(A, R, tiles, n_tiles, s);
    else
      attention(A, R, s);
    diff_combine(ws.cbuf, ws.ld_cbuf, B, L.heads, L.vdim, L.lam, L.diff, cfg.eps, ws.proj + L.off_g, ws.ld_proj, ws.a, ws.ld_a, f32, s);
  } else {
    RotFoldParams F{ws.proj, ws.ld_proj, L.off_q, L.off_k, L.off_v, L.heads, L.kv_heads, L.dim, L.vdim, L.rot_dims, L.inv_freq64,
                    L.talk, r.kc, r.vc, ws.cbuf, ws.ld_cbuf, f32};
    rotate_fold(F, R, s);
    // one key row per token serves every head: its width is all key/value heads' keys, the folded queries match it
    AttnParams A{ws.cbuf, ws.ld_cbuf, 0, 0, 0, L.heads, L.kv_heads, L.kv_heads * L.dim, L.vdim, L.scale, 0.f, 0.f, 1, r.kc, r.vc, ws.a,
                 ws.ld_a, f32, splits, ws.split_ws, ws.split_ws_floats, 0, 0, nullptr, 0, nullptr, 0, L.window, 1, 1};
    if (tiled && flash_prefill_supported(A))
      flash_prefill(A, R, tiles, n_tiles, s);
    else
      attention(A, R, s);
  }
  {
    GemmParams o{ws.a, ws.ld_a, L.w_o, B, E, n_out, ws.resid, E, EPI_RESID, 1.f, nullptr, 0.f, f32};
    gemm(o, s);
  }
  if (!L.ff_dense && !L.experts) return;
  if (L.experts && fused_in) {  // decode steps: norm + router in one launch (the normed rows leave for the experts)
    gemv_ln(ws.resid, E, L.norm2_w, nullptr, cfg.eps, L.w_ff, B, L.n_ff, ws.proj, ws.ld_proj, ws.h, nullptr, nullptr, f32, s);
  } else {
    rms_norm_cast(ws.resid, nullptr, B, E, L.norm2_w, cfg.eps, ws.h, f32, s);
  }
  if (L.ff_dense) {
    if (B <= 8) {  // decode steps: gate / up projection and activation in one launch
      gemv_relu_glu(ws.h, E, L.w_ff, E, L.ff, B, ws.hmid, ws.ld_hmid, f32, s);
    } else {
      GemmParams g{ws.h, E, L.w_ff, B, L.n_ff, E, ws.proj, ws.ld_proj, EPI_STORE, 0.f, nullptr, 0.f, f32};
      gemm(g, s);
      relu_glu_cast(ws.proj, ws.ld_proj, B, L.ff, ws.hmid, ws.ld_hmid, f32, s);
    }
    GemmParams d{ws.hmid, ws.ld_hmid, L.w_dense_down, B, E, L.ff, ws.resid, E, EPI_RESID, 1.f, nullptr, 0.f, f32};
    gemm(d, s);
    return;
  }
  if (!fused_in) {
    GemmParams g{ws.h, E, L.w_ff, B, L.n_ff, E, ws.proj, ws.ld_proj, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(g, s);
  }
  // the experts' weighted outputs are added straight into the stream (y = the stream, y_add)
  MoeParams M{ws.proj, ws.ld_proj, L.off_router, 0, 0, 0, B, E, L.experts, L.top, L.ff, 0, nullptr, ws.h, L.w_gu, L.w_down, nullptr,
              ws.eids, ws.ew, ws.ld_top, ws.sgate, ws.hmid, ws.ld_hmid, ws.resid, f32, 0, L.group_count, L.group_keep, ws.idw, 1,
              L.route_scale};
  if (B <= SMALL_B && moe_route_sigmoid_fused_supported(M)) {  // decode steps: routing + activations in one launch
    moe_route_sigmoid_experts(M, s);
    moe_down(M, s);
    return;
  }
  moe_route_sigmoid(M, s);
  if (B > SMALL_B && ws.moe.gu && moe_grouped_supported(M)) {
    moe_grouped(M, ws.moe, s);  // rows sorted by expert, one matrix-core product per expert tile
  } else {
    moe_experts(M, s);
    moe_down(M, s);
  }
}

void StackExecutor::layer_run(int ri, int B, hipStream_t s) {
  if (cfg.block == 3) {
    layer_run_prenorm(ri, B, s);
    return;
  }
  if (cfg.block == 1) {
    layer_run_postnorm(ri, B, s);
    return;
  }
  if (cfg.block == 2) {
    layer_run_sandwich(ri, B, s);
    return;
  }
  const RunDesc& r = runs.at(ri);
  const LayerDesc& L = layers[r.layer];
  const int E = cfg.E, f32 = cfg.f32;
  if (r.opens_pass) {
    concat_cast(ws.resid, ws.x0, B, E, ws.cat, f32, s);
    GemmParams g{ws.cat, 2 * E, loop_in, B, E, 2 * E, ws.resid, E, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(g, s);
  }
  StepRows R{B, in.pos, in.slot, in.q_len, in.q_seq, in.block_table, in.max_blocks, in.bs};
  AttnParams A{ws.proj, ws.ld_proj, L.off_q, L.off_k, L.off_v, L.heads, L.kv_heads, L.dim, L.vdim, L.scale, L.softcap,
               L.qtemp_coef, L.qtemp_every, r.kc, r.vc, ws.a, ws.ld_a, f32, n_splits, ws.split_ws, ws.split_ws_floats};
  const bool fused_in = gemv_ln_supported(B, E, f32);
  if (fused_in) {  // decode steps: norm + input projection (+ query temperature and K/V store) in one launch
    gemv_ln(ws.resid, E, L.norm_w, L.norm_b, cfg.eps, L.w_in, B, L.n_in, ws.proj, ws.ld_proj, ws.h, L.kind == 0 ? &A : nullptr,
            &R, f32, s);
  } else {
    layer_norm_cast(ws.resid, nullptr, B, E, L.norm_w, L.norm_b, cfg.eps, ws.h, f32, s);
    // every matrix that reads the normed activations, in one product
    GemmParams g{ws.h, E, L.w_in, B, L.n_in, E, ws.proj, ws.ld_proj, EPI_STORE, 0.f, nullptr, 0.f, f32};
    gemm(g, s);
  }
  if (L.kind == 0) {
    if (!fused_in) attn_prepare(A, R, s);
    if (B > SMALL_B && n_tiles > 0 && tiles && flash_prefill_supported(A))
      flash_prefill(A, R, tiles, n_tiles, s);  // prompt portions: query tiles on the matrix cores
    else
      attention(A, R, s);
  } else {
    RetParams P{ws.proj, ws.ld_proj, L.off_q, L.off_k, L.off_v, L.off_g, L.heads, L.dim, L.vdim, L.rot_dims, L.inv_freq,
                L.decay, r.state, cfg.eps, ws.a, ws.ld_a, f32};
    // prompt portions in chunks (the host bound this step's chunk table); else token by token in one launch
    if (B > SMALL_B && n_chunks > 0 && ws.ret.U && ws.ret.ld_o >= L.heads * L.vdim &&
        ws.ret.u_stride >= (long long)L.heads * L.dim * L.vdim && retention_chunk_supported(L.dim, L.vdim)) {
      RetChunkWs W = ws.ret;
      W.nchunks = n_chunks;
      retention_chunked(P, R, W, s);
    } else
      retention(P, R, s);
  }
  const float* ff = nullptr;
  if (L.experts) {
    MoeParams M{ws.proj, ws.ld_proj, L.off_router, L.off_sg, L.off_sgate, L.off_sup, B, E, L.experts, L.top, L.ff,
                L.shared_ff, L.router_b, ws.h, L.w_gu, L.w_down, L.sh_down, ws.eids, ws.ew, ws.ld_top, ws.sgate, ws.hmid,
                ws.ld_hmid, ws.y, f32};
    if (B <= SMALL_B) {  // decode steps: two launches end the layer (residual update included)
      moe_fused_small(M, ws.a, ws.ld_a, L.w_o, L.heads * L.vdim, ws.resid, cfg.residual_mult, s);
      return;
    }
    moe_route(M, s);
    if (ws.moe.gu && moe_grouped_supported(M)) {
      moe_grouped(M, ws.moe, s);  // rows sorted by expert, one matrix-core product per expert tile
    } else {
      moe_experts(M, s);          // every pair streams its expert's rows once
      moe_down(M, s);
    }
    ff = ws.y;
  }
  // x <- x + m * (mixer output projection + feed-forward)
  GemmParams o{ws.a, ws.ld_a, L.w_o, B, E, L.heads * L.vdim, ws.resid, E, EPI_RESID, cfg.residual_mult, ff, 0.f, f32};
  gemm(o, s);
}

void StackExecutor::head(int n_logits, bool use_idx, hipStream_t s) {
  if (n_logits <= 0) return;
  if (cfg.block == 3) {  // an RMS norm with a weight vector; plain logits
    rms_norm_cast(ws.resid, use_idx ? in.logit_idx : nullptr, n_logits, cfg.E, final_w, cfg.eps, ws.lrows, cfg.f32, s);
    GemmParams g{ws.lrows, cfg.E, head_w, n_logits, cfg.V, cfg.E, in.logits, in.ld_logits, EPI_STORE, 0.f, nullptr, 0.f, cfg.f32};
    gemm(g, s);
    return;
  }
  if (cfg.block == 2) {  // an RMS norm with one number as its weight, and a plain factor on the logits
    scalar_norm_cast(ws.resid, use_idx ? in.logit_idx : nullptr, n_logits, cfg.E, final_w, cfg.eps, ws.lrows, cfg.f32, s);
    GemmParams g{ws.lrows, cfg.E, head_w, n_logits, cfg.V, cfg.E, in.logits, in.ld_logits, EPI_SCALE, cfg.logit_scale, nullptr,
                 0.f, cfg.f32};
    gemm(g, s);
    return;
  }
  layer_norm_cast(ws.resid, use_idx ? in.logit_idx : nullptr, n_logits, cfg.E, final_w, final_b, cfg.eps, ws.lrows, cfg.f32,
                  s);
  GemmParams g{ws.lrows, cfg.E, head_w, n_logits, cfg.V, cfg.E, in.logits, in.ld_logits, EPI_SOFTCAP, 0.f, nullptr,
               cfg.logit_softcap, cfg.f32};
  gemm(g, s);
}

void StackExecutor::forward(int B, int n_logits, bool use_idx, hipStream_t s) {
  embed(B, s);
  for (int ri = 0; ri < (int)runs.size(); ++ri) layer_run(ri, B, s);
  head(n_logits, use_idx, s);
}

}  // namespace stack
}  // namespace omx
