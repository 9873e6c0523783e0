// Host-visible interface of the kernels of layer-list models (stack_kernels.hip): heterogeneous layers
// with a float32 residual stream, matrices and K/V pools in bfloat16 or float32 (`f32` flag of every call),
// paged softmax attention with capped scores and a query temperature, retention with a per-sequence state
// matrix, and a routed feed-forward with a gated shared expert. Plain C++ types only.
#pragma once
#include <hip/hip_runtime_api.h>
#include <stdint.h>

namespace omx {
namespace stack {

enum { EPI_STORE = 0, EPI_RESID = 1, EPI_SOFTCAP = 2, EPI_SCALE = 3 };

// C = epi(A . W^T): A [M][K] (row stride lda) and W [N][K] in the matrix dtype, float32 accumulation.
//   EPI_STORE:   C[m][n] = acc                                    (C float32, row stride ldc)
//   EPI_RESID:   C[m][n] += mult * (acc + (add ? add[m][n] : 0))  (C = the residual stream; add stride ldc)
//   EPI_SOFTCAP: C[m][n] = cap ? cap * tanh(acc / cap) : acc
//   EPI_SCALE:   C[m][n] = mult * acc
struct GemmParams {
  const void* A;
  int lda;
  const void* W;
  int M, N, K;
  float* C;
  int ldc;
  int epi;
  float mult;        // EPI_RESID
  const float* add;  // EPI_RESID (or null)
  float cap;         // EPI_SOFTCAP
  int f32;           // matrices are float32 (else bfloat16)
};
void gemm(const GemmParams& P, hipStream_t s);
// which kernel gemm() takes for these sizes: 0 wave-per-row GEMV (M <= 8), 1 matrix-core tile (bfloat16),
// 2 FMA tile (float32, or a K that the vector loads do not cover)
int gemm_path(int M, int N, int K, int f32);
void set_gemm_mfma(int on);  // 0: bfloat16 tiles also take the FMA kernel (A/B and tests)

// resid[r] = x0[r] = table[tokens[r]] * scale
void embed(const void* table, const int* tokens, int B, int E, int V, float* resid, float* x0, float scale, int f32,
           hipStream_t s);
// out[r] = layer_norm(x[idx ? idx[r] : r]) * w + b, written in the matrix dtype
void layer_norm_cast(const float* x, const int* idx, int rows, int E, const float* w, const float* b, float eps,
                     void* out, int f32, hipStream_t s);
// out[r] = [x[r]; x0[r]] in the matrix dtype, row stride 2E
void concat_cast(const float* x, const float* x0, int rows, int E, void* out, int f32, hipStream_t s);

struct StepRows {       // per-row step inputs (device arrays of B ints)
  int B;
  const int* pos;
  const int* slot;      // flat cache slot (block * bs + offset)
  const int* q_len;     // visible keys (pos + 1)
  const int* q_seq;     // block-table row = state slot
  const int* block_table;
  int max_blocks, bs;
};

struct AttnParams {
  float* proj;          // [B][ld] float32: q at off_q (scaled in place), k at off_k, v at off_v
  int ld, off_q, off_k, off_v;
  int H, G, D, Dv;
  float scale, softcap, qtemp_coef;
  int qtemp_every;
  void* kc;             // [blocks][G][bs][D]
  void* vc;             // [blocks][G][bs][Dv]
  void* out;            // [B][ld_out] matrix dtype, head-major
  int ld_out;
  int f32;
  // decode steps over long contexts: nsplit blocks per (row, head) share the keys and leave partials
  // {maximum, sum, output} in split_ws, a second launch merges them (nsplit <= 1: one block finishes the row)
  int nsplit;
  float* split_ws;
  long long split_ws_floats;
  // pools whose rows are wider than the head (0: D and Dv). With kc == vc and ldk == ldv the first Dv elements
  // of a cached row are its value too (latent attention: one row per token serves every head)
  int ldk, ldv;
  const float* sink;    // [H] or null: exp(sink[h]) joins the softmax denominator (no key, no value, not scaled)
  // vheads = G: every query head meets the values of EVERY key/value head, output "head" h * G + c holds query head
  // h's weights on the values of key/value head c (what a mixing of the heads' weights needs); 0 or 1: its own only
  int vheads;
  float* out32;         // non-null: the outputs leave in float32 here (row stride ld_out32) instead of `out`
  int ld_out32;
  int window;           // > 0: a row sees only its last `window` keys (itself included)
  // maps = M > 1: H counts M query maps per head, laid out [head][map]; a K row of key/value head g holds the M key maps
  // side by side (row stride ldk >= M * D) and query map h reads elements (h % M) * D ...; all maps of a head meet the
  // same values. Output "head" h is query map h.
  int maps;
  // kshared: the K pool has ONE head whose row (D wide) serves every query head, while the V pool keeps its G heads
  // (query head h meets the values of head h / (H / G)): scores that are sums over all key/value heads
  int kshared;
};
// q *= 1 + coef * ln(floor((pos + 1) / every) + 1); k, v of every row stored at its slot
void attn_prepare(const AttnParams& P, const StepRows& R, hipStream_t s);
// softmax(cap(q . k * scale)) v over the first q_len keys of the row's sequence
void attention(const AttnParams& P, const StepRows& R, hipStream_t s);

// prompt portions on the matrix cores (bfloat16, head sizes 64 / 96 / 128 with dim == vdim): `tiles` is a device
// table the host builds from the step's rows, per tile {first row, rows <= 32}, rows of one sequence in order
void flash_prefill(const AttnParams& P, const StepRows& R, const int* tiles, int ntiles, hipStream_t s);
bool flash_prefill_supported(const AttnParams& P);
constexpr int FLASH_TILE_ROWS = 32;

// decode steps (M <= 8 rows that fit LDS): C = layer_norm(x) . W^T in one launch (nb null: the norm is an RMS norm with
// weight nw, x / sqrt(mean(x^2) + eps) * nw); the normed rows also go to hout
// (matrix dtype). With A (an attention layer): q outputs get the row's query temperature, k and v outputs are
// also stored at the row's cache slot, so no attn_prepare follows.
void gemv_ln(const float* x, int E, const float* nw, const float* nb, float eps, const void* W, int M, int N, float* C,
             int ldc, void* hout, const AttnParams* A, const StepRows* R, int f32, hipStream_t s);
bool gemv_ln_supported(int M, int E, int f32);

struct RetParams {
  const float* proj;    // [B][ld] float32: q, k, v, g
  int ld, off_q, off_k, off_v, off_g;
  int H, D, Dv;
  int rot_dims;         // rotate-half pairs (i, i + rot_dims / 2) on q and k
  const float* inv_freq;  // [rot_dims / 2]
  const float* decay;   // [H]
  float* state;         // [slots][H][D][Dv] float32
  float eps;
  void* out;            // [B][ld_out] matrix dtype: unit_rms(o) * silu(g)
  int ld_out;
  int f32;
};
// rows of one sequence are contiguous and in position order; each sequence's state advances through them
void retention(const RetParams& P, const StepRows& R, hipStream_t s);
bool retention_supported(int D, int Dv);          // the state-in-registers kernel covers these head sizes
bool retention_general_supported(int D, int Dv);  // the state-in-memory kernel covers the rest, up to 1024
// the same recurrence in chunks (prompt portions), chunks in parallel around a scan over each sequence's chunk
// states; `chunks` is a device table the host builds from the step's rows: per chunk {first row, rows (at most
// retention_chunk_rows()), state slot, flags (1 = first chunk of its sequence's rows, 2 = last)}, a sequence's
// chunks in row order. The un-normalised o goes through obuf [B][ld_o]; U and Sin hold one state per chunk.
struct RetChunkWs {
  const int* chunks;
  int nchunks, max_chunks;
  float* U;
  float* Sin;
  long long u_stride;   // floats between chunks in U and Sin (>= heads * dim * vdim)
  float* obuf;
  int ld_o;
};
void retention_chunked(const RetParams& P, const StepRows& R, const RetChunkWs& W, hipStream_t s);
int retention_chunk_rows();
bool retention_chunk_supported(int D, int Dv);

struct MoeParams {
  const float* proj;    // [B][ld]: router logits at off_router, shared: scalar gate, gate rows, up rows
  int ld, off_router, off_sg, off_sgate, off_sup;
  int B, E, X, top, F, Fs;
  const float* router_b;
  const void* h;        // [B][E] matrix dtype (the normed activations)
  const void* w_gu;     // [X][2F][E]
  const void* w_down;   // [X][E][F]
  const void* sh_down;  // [E][Fs]
  int* eids;            // [B][ld_top]
  float* ew;
  int ld_top;
  float* sgate;         // [B]
  void* hmid;           // [B][ld_hmid] matrix dtype: top x F expert activations, then Fs shared
  int ld_hmid;
  float* y;             // [B][E] float32 feed-forward output
  int f32;
  // score router (moe_route_scores): the last `identity` of the X + identity router outputs return their input;
  // router_b is the choice correction; idw [B] receives the summed weight of the chosen identity outputs
  int identity, group_count, group_keep;
  float* idw;
  int y_add;            // moe_down / moe_grouped: y += the feed-forward's output (y = the residual stream) instead of y =
  float route_scale;    // sigmoid router (moe_route_sigmoid): factor on the normalised weights
};
void moe_route(const MoeParams& P, hipStream_t s);   // top-k ids + softmax weights, shared gate and activation
// softmax over all router outputs, choice by score + correction inside the best expert groups, weights = the
// chosen scores (not renormalised); leaves eids / ew / sgate (= 1) / the shared activation as moe_route does, so
// moe_experts, moe_down and moe_grouped follow unchanged
void moe_route_scores(const MoeParams& P, hipStream_t s);
// a few rows (decode steps): the same routing and the routed and shared activations (moe_experts' work) in one launch
void moe_route_scores_experts(const MoeParams& P, hipStream_t s);
bool moe_route_scores_fused_supported(const MoeParams& P);
void moe_experts(const MoeParams& P, hipStream_t s); // gate/up + activation of the routed experts -> hmid
void moe_down(const MoeParams& P, hipStream_t s);    // y = sum_j w_j down_j(hmid_j) + sgate * shared_down(hmid_s)
// a few rows (decode steps): routing + routed and shared activations in one launch, then the experts' down
// projections, the mixer's output projection (a [B][lda] . w_o [E][Ko]) and the residual update
// x += mult * (...) in a second one
void moe_fused_small(const MoeParams& P, const void* a, int lda, const void* w_o, int Ko, float* x, float mult,
                     hipStream_t s);
constexpr int MOE_MAX_TOP = 16;
// prompt portions (bfloat16): after moe_route, the (row, expert) pairs are sorted by expert and every expert's
// rows go through the matrix-core product together; y as moe_down leaves it
struct MoeGroupWs {
  int* rank;     // [max_pairs]
  int* srow;     // [max_pairs] sorted position -> pair
  int* inv;      // [max_pairs] pair -> sorted position
  int* tiles;    // [max_tiles][3]
  int* ntiles;   // [1]
  float* gu;     // [max_pairs][2F]
  void* hs;      // [max_pairs][F] matrix dtype
  float* ds;     // [max_pairs][E]
  int max_pairs, max_tiles;
};
void moe_grouped(const MoeParams& P, const MoeGroupWs& W, hipStream_t s);
bool moe_grouped_supported(const MoeParams& P);

// ---- layers whose norm sits on the sublayer's output (stack_mixers.hip)
// out = x in the matrix dtype (the sublayers read the stream itself)
void cast_rows(const float* x, int rows, int E, void* out, int f32, hipStream_t s);
// x[r] += layer_norm(y[r] + (idw ? idw[r] * x[r] : 0)) * w + b; hout (or null): the updated rows in the matrix dtype
void post_norm_add(float* x, const float* y, int rows, int E, const float* w, const float* b, float eps, const float* idw,
                   void* hout, int f32, hipStream_t s);

struct LatentParams {
  const float* proj;    // [B][ld] float32: per head [D plain | R rotated] queries at off_q, [C latent | R key part]
  int ld, off_q, off_k, off_g;  // at off_k, the output gate's pre-activations [H * Dv] at off_g
  int H, D, R, C, Dv;
  int rot_dims;         // adjacent pairs (2i, 2i + 1), i < rot_dims / 2, of the rotated part turn
  const double* inv_freq;  // [rot_dims / 2]
  const float* norm_w;  // [C] weight of the latent's RMS norm
  float eps;
  const void* w_uk;     // [H * D][C]
  const void* w_uvT;    // [H][C][Dv]
  const void* w_ukT;    // [H][C][D]   (or null) the layouts the few-row kernels read
  const void* w_uv;     // [H * Dv][C] (or null)
  void* cache;          // [blocks][1][bs][C + R] matrix dtype
  float* qa;            // [B][ld_qa]: per head [W_uk_h^T q_plain | rotated q part] (the attention's queries)
  int ld_qa;
  const void* lat;      // [B][ld_lat] matrix dtype: the attention's outputs in latent space, per head C
  int ld_lat;
  void* out;            // [B][ld_out] matrix dtype: (W_uv_h lat_h) * sigmoid(g), head-major
  int ld_out;
  int f32;
  int gate_heads;       // 1: the gate is one number per head ([H] at off_g) instead of one per output element
};
void latent_prepare(const LatentParams& P, const StepRows& R, hipStream_t s);
void latent_expand(const LatentParams& P, int B, hipStream_t s);
bool latent_supported(int D, int R, int C, int Dv);

struct ConvParams {
  const float* proj;    // [B][ld] float32: the convolution's inputs at off_in
  int ld, off_in;
  int ch, taps;
  const float* w;       // [ch][taps], the last tap is the current token's
  const float* bias;    // [ch]
  float* state;         // slot s: state + s * state_stride = [taps - 1][ch], the sequence's last inputs
  long long state_stride;
  float* out;           // [B][ld_out] float32: silu(conv)
  int ld_out;
};
void conv_silu(const ConvParams& P, const StepRows& R, hipStream_t s);

enum { SCAN_MLSTM = 0, SCAN_SSD = 1 };
struct ScanParams {
  int mode;
  const float* proj;    // [B][ld] float32
  int ld;
  const float* conv;    // SCAN_SSD: [B][ld_conv] the convolution's output (q, k, v live there)
  int ld_conv;
  int off_q, off_k, off_v;  // G groups of D (q, k), H heads of Dv (v)
  int off_i, off_f;     // SCAN_MLSTM: gate pre-activations [H] in proj; SCAN_SSD: off_i = dt [H] in proj
  int off_g;            // SCAN_SSD: z [H * Dv] in proj
  int H, G, D, Dv;
  const float* i_b;     // SCAN_MLSTM [H]
  const float* f_b;
  float cap;
  const float* dt_bias; // SCAN_SSD [H]
  const float* a_log;
  const float* d_skip;
  float* state;         // slot s: state + s * state_stride = S [H][D][Dv] (| n [H][D] | m [H] for SCAN_MLSTM)
  long long state_stride;
  float* y;             // [B][ld_y] float32
  int ld_y;
};
void gated_scan(const ScanParams& P, const StepRows& R, hipStream_t s);
bool gated_scan_supported(int mode, int D, int Dv);
// the same recurrence in chunks (prompt portions) over the host-built chunk table of the chunked retention
// ({first row, rows <= gated_chunk_rows(), state slot, flags}); U and Sin hold one state per chunk
// ([H][D][Dv (+ 1 for the mLSTM's normaliser)]), coef [B][H][3] the rows' {ln a, b, m}, ctot [chunks][H] the chunks'
// summed ln a, raw [B][ld_raw] the mLSTM's outputs before their division ([H][Dv + 1]). SCAN_SSD leaves P.y as
// gated_scan does; SCAN_MLSTM goes on to the finished mixer output `out` (division, per-head unit RMS, norm_w, the
// sigmoid gate at P.off_g), matrix dtype.
struct ScanChunkWs {
  const int* chunks;
  int nchunks, max_chunks;
  float* U;
  float* Sin;
  long long u_stride;
  float* coef;
  float* ctot;
  float* raw;
  int ld_raw;
};
void gated_scan_chunked(const ScanParams& P, const StepRows& R, const ScanChunkWs& W, const float* norm_w, float eps, void* out,
                        int ld_out, int f32, hipStream_t s);
int gated_chunk_rows();
bool gated_chunk_supported(int mode, int D, int Dv);
// out = y / rms(y over each of `groups` equal parts) * w * (gate ? sigmoid(gate) : 1), matrix dtype
void group_rms_cast(const float* y, int ld_y, int rows, int n, int groups, const float* w, float eps, const float* gate,
                    int ld_gate, void* out, int ld_out, int f32, hipStream_t s);
// out = relu(z)^2, matrix dtype
void relu2_cast(const float* z, int ld, int rows, int F, void* out, int ld_out, int f32, hipStream_t s);

// ---- layers with scalar-weight RMS norms before and after both sublayers (stack_sandwich.hip)
// hn[r] = x[r] / rms(x[r]) * g[0] (float32); out[r] = hn[r] + conv(hn)[r] in the matrix dtype, where conv is a causal
// per-channel convolution over the rows of r's sequence (w [E][taps], the last tap is the current token's) that
// continues from the sequence's carried window (slot s: window + s * stride = [taps - 1][E], oldest first), which
// is advanced past the step's rows. taps == 1: a per-channel factor on the current token, no window.
constexpr int CANON_MAX_TAPS = 8;
struct CanonParams {
  const float* x;
  const float* g;
  float eps;
  int E, taps;
  const float* w;
  float* window;
  long long stride;
  float* hn;            // [B][E]
  void* out;            // [B][E] matrix dtype
  int f32;
};
void scalar_norm_conv(const CanonParams& P, const StepRows& R, hipStream_t s);
// out[r] = x[idx ? idx[r] : r] / rms * g[0], matrix dtype
void scalar_norm_cast(const float* x, const int* idx, int rows, int E, const float* g, float eps, void* out, int f32,
                      hipStream_t s);

enum { QK_NORM_NONE = 0, QK_NORM_WEIGHT_FIRST = 1, QK_NORM_UNIT_LAST = 2 };
struct QkPrepParams {
  float* proj;          // [B][ld] float32: q at off_q (finished in place), k at off_k, v at off_v
  int ld, off_q, off_k, off_v;
  const float* bias;    // indexed like proj's columns, or null
  int H, G, D, Dv;
  int rot_dims;         // rotate-half pairs (i, i + rot_dims / 2) of every head turn by pos * inv_freq[i]
  const double* inv_freq;
  int qk_norm;          // QK_NORM_WEIGHT_FIRST: rms norm * weight before the rotation; QK_NORM_UNIT_LAST: unit rms after
  const float* q_norm;  // [D]
  const float* k_norm;
  float eps;
  int v_from_k;         // the value row is the key as projected (bias added, before norm and rotation); Dv == D
  void* kc;             // [blocks][G][bs][D]
  void* vc;             // [blocks][G][bs][Dv]
  int f32;
};
void qk_prepare(const QkPrepParams& P, const StepRows& R, hipStream_t s);
// out[b][h] = sum_g talk[h][g] * o32[b][g * G + kv(h)] (vectors of Dv): the mixed weights of head h on the values of
// its own key/value head, from the attention's outputs of every (query head, value head) pair
void talk_mix(const float* o32, int ld_o, int B, int H, int G, int Dv, const float* talk, void* out, int ld_out, int f32,
              hipStream_t s);

// gated linear attention: S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T (q_t D^(-1/2)), with
// alpha = sigmoid(z)^(1 / tau), z = a2 . a1_t + a2_b per key channel; out = rms_norm(o per head) * norm_w * silu(g)
struct GlaParams {
  const float* proj;    // [B][ld] float32
  int ld, off_q, off_k, off_v, off_g, off_a1;
  int H, D, Dv, rank;
  const void* a2;       // [H * D][rank] matrix dtype
  const float* a2_b;    // [H * D]
  float tau;
  const float* norm_w;  // [Dv]
  float eps;
  float* state;         // slot s: state + s * state_stride = S [H][D][Dv] float32
  long long state_stride;
  void* out;            // [B][ld_out] matrix dtype, head-major
  int ld_out;
  int f32;
};
void gla(const GlaParams& P, const StepRows& R, hipStream_t s);
bool gla_supported(int D, int Dv);          // the state-in-registers kernel covers these head sizes
bool gla_general_supported(int D, int Dv);  // the state-in-memory kernel covers the rest, up to 256
// the same in chunks (prompt portions) over the host-built chunk table of the chunked retention; lna [B][H * D] and
// U / Sin (one state per chunk) are scratch, raw [B][ld_raw] receives o before its norm
struct GlaChunkWs {
  const int* chunks;
  int nchunks, max_chunks;
  float* U;
  float* Sin;
  long long u_stride;
  float* lna;
  int ld_lna;
  float* raw;
  int ld_raw;
};
void gla_chunked(const GlaParams& P, const StepRows& R, const GlaChunkWs& W, hipStream_t s);
bool gla_chunk_supported(int D, int Dv);

// x[r] += ls * (v / rms(v) * g[0]) with v = sa * (y[r] + bias) + (y2 ? sb * y2[r] : 0); with g_next and hout the
// updated row also leaves normed, x_new / rms(x_new) * g_next[0], in the matrix dtype (the next sublayer's operand)
void sandwich_add(float* x, const float* y, const float* bias, float sa, const float* y2, float sb, int rows, int E,
                  const float* g, const float* ls, float eps, const float* g_next, void* hout, int f32, hipStream_t s);
// C[m][n] = sa * (A1[m] . W1[n] + bias[n]) + sb * (A2[m] . W2[n]): two output projections of a few rows (M <= 8) in one launch
void gemv_pair(const void* A1, int lda1, const void* W1, int K1, const float* bias, float sa, const void* A2, int lda2,
               const void* W2, int K2, float sb, int M, int N, float* C, int ldc, int f32, hipStream_t s);
// out[m][k] = gelu_tanh(A[m] . W[k]) * (A[m] . W[F + k]), matrix dtype: the gate / up projection of a few rows (M <= 8) with
// its activation in one launch (W [2F][K]: gate rows, then up rows)
void gemv_glu(const void* A, int lda, const void* W, int K, int F, int M, void* out, int ld_out, int f32, hipStream_t s);
// out = gelu_tanh(z[:, :F]) * z[:, F:2F], matrix dtype
void geglu_tanh_cast(const float* z, int ld, int rows, int F, void* out, int ld_out, int f32, hipStream_t s);


// ---- layers with RMS norms (weight vectors) on the inputs of both sublayers (stack_prenorm.hip)
// out[r] = x[idx ? idx[r] : r] / rms * w, matrix dtype
void rms_norm_cast(const float* x, const int* idx, int rows, int E, const float* w, float eps, void* out, int f32, hipStream_t s);
// differential attention: o32 [B][ld_o] holds per head the two maps' outputs side by side ([H][2][Dv], float32);
// out[b][h] = (a1 - lam a2) / rms over Dv * (1 - diff) * sigmoid(gate[b][h * Dv ...]) (gate null: no gate), matrix dtype
void diff_combine(const float* o32, int ld_o, int B, int H, int Dv, float lam, float diff, float eps, const float* gate, int ld_gate,
                  void* out, int ld_out, int f32, hipStream_t s);
// attention whose scores are mixed across the heads before the softmax, score_h = sum_g mix[h][g] (q_g . k_c(g)):
// q and k turn in adjacent pairs (2i, 2i + 1), i < rot_dims / 2, by pos * inv_freq[i]; the K pool's row of a token is
// [k_0 | ... | k_(G-1)] (one head, G * D wide), the V pool is [blocks][G][bs][Dv]; the queries leave folded through the
// mixing matrix, qf[b][h] = [sum_(g of head c) mix[h][g] q_g, for c < G], so that attention over the shared key row
// with H query heads of width G * D gives the mixed scores
struct RotFoldParams {
  const float* proj;    // [B][ld] float32: q [H][D] at off_q, k [G][D] at off_k, v [G][Dv] at off_v
  int ld, off_q, off_k, off_v;
  int H, G, D, Dv;
  int rot_dims;
  const double* inv_freq;  // [rot_dims / 2]
  const float* mix;     // [H][H]
  void* kc;             // [blocks][1][bs][G * D]
  void* vc;             // [blocks][G][bs][Dv]
  float* qf;            // [B][ld_qf]: [H][G * D]
  int ld_qf;
  int f32;
};
void rotate_fold(const RotFoldParams& P, const StepRows& R, hipStream_t s);
bool rotate_fold_supported(int H, int G, int D);
// out = relu(z[:, :F]) * z[:, F:2F], matrix dtype
void relu_glu_cast(const float* z, int ld, int rows, int F, void* out, int ld_out, int f32, hipStream_t s);
// out[m][k] = relu(A[m] . W[k]) * (A[m] . W[F + k]), matrix dtype: gate / up projection of a few rows (M <= 16) + activation
void gemv_relu_glu(const void* A, int lda, const void* W, int K, int F, int M, void* out, int ld_out, int f32, hipStream_t s);
// sigmoid scores; a group of neighbours ranks by the sum of its two largest scores, only the best group_keep groups
// stay; the `top` largest scores, divided by their sum, times route_scale -> eids / ew, as moe_route leaves them, so
// moe_experts, moe_down and moe_grouped follow unchanged (no shared expert, no router bias)
void moe_route_sigmoid(const MoeParams& P, hipStream_t s);
// a few rows (decode steps): the same routing and the routed activations (moe_experts' work) in one launch
void moe_route_sigmoid_experts(const MoeParams& P, hipStream_t s);
bool moe_route_sigmoid_fused_supported(const MoeParams& P);

}  // namespace stack
}  // namespace omx
