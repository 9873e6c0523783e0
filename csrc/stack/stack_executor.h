// Step executor of layer-list models: the launch sequence of one step over B rows (any mix of prompt
// portions and single decode tokens; rows of a sequence contiguous and in position order). Python owns
// the device memory and hands raw pointers in; the executor only enqueues kernels on a stream, so a whole
// step is capturable into one hipGraph.
#pragma once
#include <hip/hip_runtime_api.h>

#include <vector>

#include "stack_ops.h"

namespace omx {
namespace stack {

struct StackConfig {
  int E = 0, V = 0;
  float eps = 1e-5f, residual_mult = 1.f, logit_softcap = 0.f;
  int f32 = 0;
  int max_B = 0, max_seqs = 0;
  int block = 0;            // 0: one norm, mixer and feed-forward in parallel; 1: norms on the sublayers' outputs;
                            // 2: scalar-weight RMS norms before and after both sublayers; 3: RMS norms (weight vectors) on
                            // the inputs of both sublayers
  float embed_scale = 1.f;
  float logit_scale = 1.f;  // block 2: logits = head x * logit_scale
  int canon_taps = 1;       // block 2: taps of the convolution added to the mixer's input (1: the current token only)
};

struct LayerDesc {
  int kind = 0;  // 0 attention, 1 retention, 2 latent attention, 3 mLSTM, 4 Mamba-2
  int heads = 0, kv_heads = 0, dim = 0, vdim = 0;
  float scale = 1.f, softcap = 0.f, qtemp_coef = 0.f;
  int qtemp_every = 1, rot_dims = 0;
  int n_in = 0, off_q = 0, off_k = 0, off_v = 0, off_g = 0, off_router = 0, off_sg = 0, off_sgate = 0, off_sup = 0;
  const float* norm_w = nullptr;
  const float* norm_b = nullptr;
  const void* w_in = nullptr;   // [n_in][E]
  const void* w_o = nullptr;    // [E][heads * vdim]
  const float* decay = nullptr;
  const float* inv_freq = nullptr;
  int experts = 0, top = 0, ff = 0, shared_ff = 0;  // experts == 0: no feed-forward
  const float* router_b = nullptr;
  const void* w_gu = nullptr;
  const void* w_down = nullptr;
  const void* sh_down = nullptr;
  // layers with norms on the sublayers' outputs
  const float* norm2_w = nullptr;   // the feed-forward's output norm
  const float* norm2_b = nullptr;
  const void* w_ff = nullptr;       // [n_ff][E]: router | shared gate | shared up, or the dense up projection
  int n_ff = 0;
  int ff_dense = 0;                 // 1: W_down relu(W_up h)^2 with `ff` hidden units
  const void* w_dense_down = nullptr;
  int identity = 0, group_count = 1, group_keep = 1;  // score router
  int rot_dim = 0, kv_rank = 0;     // latent attention
  const double* inv_freq64 = nullptr;
  const float* dkv_norm = nullptr;
  const void* w_uk = nullptr;
  const void* w_uvT = nullptr;
  const void* w_ukT = nullptr;
  const void* w_uv = nullptr;
  const float* sink = nullptr;
  float gate_cap = 0.f;             // mLSTM
  int off_i = 0, off_f = 0;
  const float* i_b = nullptr;
  const float* f_b = nullptr;
  const float* mnorm = nullptr;     // weight of the mixer's own output norm (mLSTM, Mamba-2)
  int state = 0, groups = 1, conv = 1, norm_groups = 1;  // Mamba-2
  int off_conv = 0, off_dt = 0;
  const float* conv_w = nullptr;
  const float* conv_b = nullptr;
  const float* dt_bias = nullptr;
  const float* a_log = nullptr;
  const float* d_skip = nullptr;
  // layers with scalar-weight norms around both sublayers: norm_w / norm_b and norm2_w / norm2_b hold the single
  // weights of the norms before / after the mixer and the feed-forward
  const float* in_b = nullptr;      // [n_in] biases of the stacked input projection (zero where there is none)
  const float* o_b = nullptr;       // [E] bias of the attention's output projection, or null
  const float* ls1 = nullptr;       // [E] per-channel scale of the mixer's result
  const float* ls2 = nullptr;       // [E] of the feed-forward's
  const float* canon = nullptr;     // [E][taps]
  int qk_norm = 0, v_from_k = 0;
  const float* q_norm = nullptr;
  const float* k_norm = nullptr;
  const float* talk = nullptr;      // [heads][heads] mixing of the heads' attention weights, or null
  // a gated linear attention that reads the same input; the layer's result is left_scale * attention + right_scale * it
  int r_heads = 0, r_dim = 0, r_vdim = 0, r_rank = 0;
  float r_tau = 1.f, left_scale = 1.f, right_scale = 1.f;
  int off_rq = 0, off_rk = 0, off_rv = 0, off_a1 = 0;
  const void* a2 = nullptr;
  const float* a2_b = nullptr;
  const float* gnorm = nullptr;
  const void* w_o2 = nullptr;       // [E][r_heads * r_vdim]
  // layers with RMS norms on the sublayers' inputs: norm_w / norm2_w are the weight vectors; ff_dense == 3 is the gated
  // dense feed-forward with a relu gate; experts use the sigmoid router
  int window = 0;                   // sliding window of the attention (0: none)
  int maps = 1;                     // 2: differential attention (two query / key maps per head)
  float diff = 0.f, lam = 0.f;      // o = (a1 - lam a2) / rms * (1 - diff)
  int gate = 0;                     // 1: element-wise sigmoid output gate at off_g, 2: one gate per head
  int score_talk = 0;               // the heads' scores are mixed by `talk` before the softmax
  float route_scale = 1.f;
};

struct RunDesc {   // one execution of a layer: its own cache
  int layer = 0;
  int opens_pass = 0;  // x <- W_in [x; x0] first
  void* kc = nullptr;
  void* vc = nullptr;
  float* state = nullptr;
  long long state_stride = 0;  // floats per slot (mLSTM, Mamba-2: the slot's whole state)
};

struct StackWorkspace {
  float* resid = nullptr;  // [max_B][E]
  float* x0 = nullptr;     // [max_B][E]
  void* h = nullptr;       // [max_B][E] matrix dtype
  void* cat = nullptr;     // [max_B][2E] matrix dtype
  float* proj = nullptr;   // [max_B][ld_proj]
  int ld_proj = 0;
  void* a = nullptr;       // [max_B][ld_a] matrix dtype (mixer output before the output projection)
  int ld_a = 0;
  void* hmid = nullptr;
  int ld_hmid = 0;
  float* y = nullptr;      // [max_B][E] feed-forward output
  int* eids = nullptr;
  float* ew = nullptr;
  int ld_top = 0;
  float* sgate = nullptr;
  void* lrows = nullptr;   // [max_B][E] matrix dtype: normed rows for the head
  float* split_ws = nullptr;  // decode attention over long contexts: per-split partials
  long long split_ws_floats = 0;
  float* cbuf = nullptr;   // [max_B][ld_cbuf] float32: latent attention's folded queries, the convolution's output
  int ld_cbuf = 0;
  void* lat = nullptr;     // [max_B][ld_lat] matrix dtype: attention outputs in latent space
  int ld_lat = 0;
  float* idw = nullptr;    // [max_B] weight of the chosen identity experts
  float* coef = nullptr;   // [max_B][ld_coef] chunked gated scan: per (row, head) {ln a, b, m}
  int ld_coef = 0;
  float* ctot = nullptr;   // [max chunks][ld_coef / 3] the chunks' summed ln a per head
  float* hn = nullptr;     // [max_B][E] float32: normed rows before the input convolution (block 2)
  float* y2 = nullptr;     // [max_B][E] float32: the second mixer's projected output (block 2)
  float* lna = nullptr;    // chunked gated linear attention: the rows' running log decays (= coef)
  MoeGroupWs moe{};        // grouped routed feed-forward (prompt portions, bfloat16); gu == null: unused
  RetChunkWs ret{};        // chunked retention (prompt portions): chunk table, per-chunk states, o before its norm
};

struct StackInputs {
  const int* tokens = nullptr;
  const int* pos = nullptr;
  const int* slot = nullptr;
  const int* q_len = nullptr;
  const int* q_seq = nullptr;
  const int* block_table = nullptr;
  int max_blocks = 0, bs = 16;
  float* logits = nullptr;
  int ld_logits = 0;
  const int* logit_idx = nullptr;
};

constexpr int SMALL_B = 16;  // steps of at most this many rows take the decode kernels

class StackExecutor {
 public:
  StackConfig cfg;
  std::vector<LayerDesc> layers;
  std::vector<RunDesc> runs;
  const void* embed_w = nullptr;
  const void* loop_in = nullptr;
  const float* final_w = nullptr;
  const float* final_b = nullptr;
  const void* head_w = nullptr;
  StackWorkspace ws;
  StackInputs in;
  const int* tiles = nullptr;  // attention query tiles of the NEXT step {first row, rows}, n_tiles of them (0: none)
  int n_tiles = 0, max_tiles = 0;
  int n_splits = 1;        // blocks per (row, head) of the NEXT steps' decode attention (long contexts)
  bool h_ready = false;    // ws.h holds the stream's rows in the matrix dtype (layers with output norms)
  int n_chunks = 0;        // chunks in ws.ret.chunks for the NEXT step (0: none bound, retention runs token by token)

  void validate() const;  // throws when a size does not fit the kernels or a pointer is missing
  void embed(int B, hipStream_t s);
  void layer_run(int ri, int B, hipStream_t s);
  void layer_run_postnorm(int ri, int B, hipStream_t s);
  void layer_run_sandwich(int ri, int B, hipStream_t s);
  void layer_run_prenorm(int ri, int B, hipStream_t s);
  void head(int n_logits, bool use_idx, hipStream_t s);
  void forward(int B, int n_logits, bool use_idx, hipStream_t s);
};

}  // namespace stack
}  // namespace omx
