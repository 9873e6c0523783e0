// Python bindings of the stack executor's module (`ollama_operator_amd/_stack`): the executor, the matrix
// product on its own (kernel tests), and the sampler shared with the main module. Torch-header-free:
// device pointers and streams cross as integers.
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <stdexcept>

#include "../bind_sampling.h"
#include "stack_executor.h"

namespace py = pybind11;
using namespace omx::stack;

template <class T>
static inline T* Pp(uintptr_t p) { return reinterpret_cast<T*>(p); }
static inline hipStream_t S(uintptr_t s) { return reinterpret_cast<hipStream_t>(s); }
static uintptr_t ptr(const py::dict& d, const char* k) { return d.contains(k) ? d[k].cast<uintptr_t>() : 0; }
static int geti(const py::dict& d, const char* k, int dflt = 0) { return d.contains(k) ? d[k].cast<int>() : dflt; }
static float getf(const py::dict& d, const char* k, float dflt = 0.f) { return d.contains(k) ? d[k].cast<float>() : dflt; }

enum { ST_FORWARD = 0, ST_EMBED = 1, ST_RUN = 2, ST_HEAD = 3 };

PYBIND11_MODULE(_stack, m) {
  m.doc() = "gfx950 kernels and step executor of layer-list models";
  omx::bind_sampling(m);
  m.attr("ST_FORWARD") = (int)ST_FORWARD;
  m.attr("ST_EMBED") = (int)ST_EMBED;
  m.attr("ST_RUN") = (int)ST_RUN;
  m.attr("ST_HEAD") = (int)ST_HEAD;
  m.def("gemm", [](py::dict d, uintptr_t stream) {
    GemmParams P{};
    P.A = Pp<const void>(ptr(d, "A"));
    P.lda = geti(d, "lda");
    P.W = Pp<const void>(ptr(d, "W"));
    P.M = geti(d, "M");
    P.N = geti(d, "N");
    P.K = geti(d, "K");
    P.C = Pp<float>(ptr(d, "C"));
    P.ldc = geti(d, "ldc");
    P.epi = geti(d, "epi");
    P.mult = getf(d, "mult", 1.f);
    P.add = Pp<const float>(ptr(d, "add"));
    P.cap = getf(d, "cap");
    P.f32 = geti(d, "f32");
    gemm(P, S(stream));
  });
  m.def("gemm_path", &gemm_path);
  m.def("set_gemm_mfma", &set_gemm_mfma);
  m.def("retention_supported", &retention_supported);
  m.def("gated_scan_supported", &gated_scan_supported);
  m.def("latent_supported", &latent_supported);
  m.def("gla_supported", &gla_supported);
  m.def("gla_chunk_supported", &gla_chunk_supported);
  m.def("gated_chunk_rows", &gated_chunk_rows);
  m.def("retention_chunk_rows", &retention_chunk_rows);
  m.attr("FLASH_TILE_ROWS") = (int)FLASH_TILE_ROWS;

  py::class_<StackExecutor>(m, "Executor")
      .def(py::init<>())
      .def("configure", [](StackExecutor& e, py::dict c) {
        e.cfg.E = geti(c, "E");
        e.cfg.V = geti(c, "V");
        e.cfg.eps = getf(c, "eps", 1e-5f);
        e.cfg.residual_mult = getf(c, "residual_mult", 1.f);
        e.cfg.logit_softcap = getf(c, "logit_softcap");
        e.cfg.f32 = geti(c, "f32");
        e.cfg.max_B = geti(c, "max_B");
        e.cfg.max_seqs = geti(c, "max_seqs");
        e.cfg.block = geti(c, "block");
        e.cfg.embed_scale = getf(c, "embed_scale", 1.f);
        e.cfg.logit_scale = getf(c, "logit_scale", 1.f);
        e.cfg.canon_taps = geti(c, "canon_taps", 1);
      })
      .def("set_globals", [](StackExecutor& e, py::dict d) {
        e.embed_w = Pp<const void>(ptr(d, "embed"));
        e.loop_in = Pp<const void>(ptr(d, "loop_in"));
        e.final_w = Pp<const float>(ptr(d, "final_w"));
        e.final_b = Pp<const float>(ptr(d, "final_b"));
        e.head_w = Pp<const void>(ptr(d, "head"));
      })
      .def("set_layer", [](StackExecutor& e, int i, py::dict d) {
        if (i < 0) throw std::runtime_error("bad layer index");
        if ((int)e.layers.size() <= i) e.layers.resize(i + 1);
        LayerDesc& L = e.layers[i];
        L = LayerDesc{};
        L.kind = geti(d, "kind");
        L.heads = geti(d, "heads");
        L.kv_heads = geti(d, "kv_heads");
        L.dim = geti(d, "dim");
        L.vdim = geti(d, "vdim");
        L.scale = getf(d, "scale", 1.f);
        L.softcap = getf(d, "softcap");
        L.qtemp_coef = getf(d, "qtemp_coef");
        L.qtemp_every = geti(d, "qtemp_every", 1);
        L.rot_dims = geti(d, "rot_dims");
        L.n_in = geti(d, "n_in");
        L.off_q = geti(d, "off_q");
        L.off_k = geti(d, "off_k");
        L.off_v = geti(d, "off_v");
        L.off_g = geti(d, "off_g");
        L.off_router = geti(d, "off_router");
        L.off_sg = geti(d, "off_sg");
        L.off_sgate = geti(d, "off_sgate");
        L.off_sup = geti(d, "off_sup");
        L.norm_w = Pp<const float>(ptr(d, "norm_w"));
        L.norm_b = Pp<const float>(ptr(d, "norm_b"));
        L.w_in = Pp<const void>(ptr(d, "w_in"));
        L.w_o = Pp<const void>(ptr(d, "w_o"));
        L.decay = Pp<const float>(ptr(d, "decay"));
        L.inv_freq = Pp<const float>(ptr(d, "inv_freq"));
        L.experts = geti(d, "experts");
        L.top = geti(d, "top");
        L.ff = geti(d, "ff");
        L.shared_ff = geti(d, "shared_ff");
        L.router_b = Pp<const float>(ptr(d, "router_b"));
        L.w_gu = Pp<const void>(ptr(d, "w_gu"));
        L.w_down = Pp<const void>(ptr(d, "w_down"));
        L.sh_down = Pp<const void>(ptr(d, "sh_down"));
        L.norm2_w = Pp<const float>(ptr(d, "norm2_w"));
        L.norm2_b = Pp<const float>(ptr(d, "norm2_b"));
        L.w_ff = Pp<const void>(ptr(d, "w_ff"));
        L.n_ff = geti(d, "n_ff");
        L.ff_dense = geti(d, "ff_dense");
        L.w_dense_down = Pp<const void>(ptr(d, "w_dense_down"));
        L.identity = geti(d, "identity");
        L.group_count = geti(d, "group_count", 1);
        L.group_keep = geti(d, "group_keep", 1);
        L.rot_dim = geti(d, "rot_dim");
        L.kv_rank = geti(d, "kv_rank");
        L.inv_freq64 = Pp<const double>(ptr(d, "inv_freq64"));
        L.dkv_norm = Pp<const float>(ptr(d, "dkv_norm"));
        L.w_uk = Pp<const void>(ptr(d, "w_uk"));
        L.w_uvT = Pp<const void>(ptr(d, "w_uvT"));
        L.w_ukT = Pp<const void>(ptr(d, "w_ukT"));
        L.w_uv = Pp<const void>(ptr(d, "w_uv"));
        L.sink = Pp<const float>(ptr(d, "sink"));
        L.gate_cap = getf(d, "gate_cap");
        L.off_i = geti(d, "off_i");
        L.off_f = geti(d, "off_f");
        L.i_b = Pp<const float>(ptr(d, "i_b"));
        L.f_b = Pp<const float>(ptr(d, "f_b"));
        L.mnorm = Pp<const float>(ptr(d, "mnorm"));
        L.state = geti(d, "state");
        L.groups = geti(d, "groups", 1);
        L.conv = geti(d, "conv", 1);
        L.norm_groups = geti(d, "norm_groups", 1);
        L.off_conv = geti(d, "off_conv");
        L.off_dt = geti(d, "off_dt");
        L.conv_w = Pp<const float>(ptr(d, "conv_w"));
        L.conv_b = Pp<const float>(ptr(d, "conv_b"));
        L.dt_bias = Pp<const float>(ptr(d, "dt_bias"));
        L.a_log = Pp<const float>(ptr(d, "a_log"));
        L.d_skip = Pp<const float>(ptr(d, "d_skip"));
        L.in_b = Pp<const float>(ptr(d, "in_b"));
        L.o_b = Pp<const float>(ptr(d, "o_b"));
        L.ls1 = Pp<const float>(ptr(d, "ls1"));
        L.ls2 = Pp<const float>(ptr(d, "ls2"));
        L.canon = Pp<const float>(ptr(d, "canon"));
        L.qk_norm = geti(d, "qk_norm");
        L.v_from_k = geti(d, "v_from_k");
        L.q_norm = Pp<const float>(ptr(d, "q_norm"));
        L.k_norm = Pp<const float>(ptr(d, "k_norm"));
        L.talk = Pp<const float>(ptr(d, "talk"));
        L.r_heads = geti(d, "r_heads");
        L.r_dim = geti(d, "r_dim");
        L.r_vdim = geti(d, "r_vdim");
        L.r_rank = geti(d, "r_rank");
        L.r_tau = getf(d, "r_tau", 1.f);
        L.left_scale = getf(d, "left_scale", 1.f);
        L.right_scale = getf(d, "right_scale", 1.f);
        L.off_rq = geti(d, "off_rq");
        L.off_rk = geti(d, "off_rk");
        L.off_rv = geti(d, "off_rv");
        L.off_a1 = geti(d, "off_a1");
        L.a2 = Pp<const void>(ptr(d, "a2"));
        L.a2_b = Pp<const float>(ptr(d, "a2_b"));
        L.gnorm = Pp<const float>(ptr(d, "gnorm"));
        L.w_o2 = Pp<const void>(ptr(d, "w_o2"));
        L.window = geti(d, "window");
        L.maps = geti(d, "maps", 1);
        L.diff = getf(d, "diff");
        L.lam = getf(d, "lam");
        L.gate = geti(d, "gate");
        L.score_talk = geti(d, "score_talk");
        L.route_scale = getf(d, "route_scale", 1.f);
        if (L.qtemp_every <= 0) throw std::runtime_error("q_temp.every must be positive");
      })
      .def("set_runs", [](StackExecutor& e, std::vector<py::dict> runs) {
        e.runs.clear();
        for (auto& d : runs) {
          RunDesc r;
          r.layer = geti(d, "layer");
          r.opens_pass = geti(d, "opens_pass");
          r.kc = Pp<void>(ptr(d, "kc"));
          r.vc = Pp<void>(ptr(d, "vc"));
          r.state = Pp<float>(ptr(d, "state"));
          r.state_stride = d.contains("state_stride") ? d["state_stride"].cast<long long>() : 0;
          e.runs.push_back(r);
        }
      })
      .def("set_workspace", [](StackExecutor& e, py::dict d) {
        StackWorkspace& w = e.ws;
        w.resid = Pp<float>(ptr(d, "resid"));
        w.x0 = Pp<float>(ptr(d, "x0"));
        w.h = Pp<void>(ptr(d, "h"));
        w.cat = Pp<void>(ptr(d, "cat"));
        w.proj = Pp<float>(ptr(d, "proj"));
        w.ld_proj = geti(d, "ld_proj");
        w.a = Pp<void>(ptr(d, "a"));
        w.ld_a = geti(d, "ld_a");
        w.hmid = Pp<void>(ptr(d, "hmid"));
        w.ld_hmid = geti(d, "ld_hmid");
        w.y = Pp<float>(ptr(d, "y"));
        w.eids = Pp<int>(ptr(d, "eids"));
        w.ew = Pp<float>(ptr(d, "ew"));
        w.ld_top = geti(d, "ld_top");
        w.sgate = Pp<float>(ptr(d, "sgate"));
        w.lrows = Pp<void>(ptr(d, "lrows"));
        w.split_ws = Pp<float>(ptr(d, "split_ws"));
        w.split_ws_floats = d.contains("split_ws_floats") ? d["split_ws_floats"].cast<long long>() : 0;
        w.ret.chunks = Pp<const int>(ptr(d, "ret_chunks"));
        w.ret.max_chunks = geti(d, "ret_max_chunks");
        w.ret.U = Pp<float>(ptr(d, "ret_u"));
        w.ret.Sin = Pp<float>(ptr(d, "ret_sin"));
        w.ret.u_stride = d.contains("ret_u_stride") ? d["ret_u_stride"].cast<long long>() : 0;
        w.ret.obuf = Pp<float>(ptr(d, "obuf"));
        w.moe.rank = Pp<int>(ptr(d, "moe_rank"));
        w.moe.srow = Pp<int>(ptr(d, "moe_srow"));
        w.moe.inv = Pp<int>(ptr(d, "moe_inv"));
        w.moe.tiles = Pp<int>(ptr(d, "moe_tiles"));
        w.moe.ntiles = Pp<int>(ptr(d, "moe_ntiles"));
        w.moe.gu = Pp<float>(ptr(d, "moe_gu"));
        w.moe.hs = Pp<void>(ptr(d, "moe_hs"));
        w.moe.ds = Pp<float>(ptr(d, "moe_ds"));
        w.moe.max_pairs = geti(d, "moe_max_pairs");
        w.moe.max_tiles = geti(d, "moe_max_tiles");
        w.ret.ld_o = geti(d, "ld_obuf");
        w.cbuf = Pp<float>(ptr(d, "cbuf"));
        w.ld_cbuf = geti(d, "ld_cbuf");
        w.lat = Pp<void>(ptr(d, "lat"));
        w.ld_lat = geti(d, "ld_lat");
        w.idw = Pp<float>(ptr(d, "idw"));
        w.coef = Pp<float>(ptr(d, "coef"));
        w.ld_coef = geti(d, "ld_coef");
        w.ctot = Pp<float>(ptr(d, "ctot"));
        w.hn = Pp<float>(ptr(d, "hn"));
        w.y2 = Pp<float>(ptr(d, "y2"));
        w.lna = w.coef;
      })
      .def("set_inputs", [](StackExecutor& e, py::dict d) {
        StackInputs& in = e.in;
        in.tokens = Pp<const int>(ptr(d, "tokens"));
        in.pos = Pp<const int>(ptr(d, "pos"));
        in.slot = Pp<const int>(ptr(d, "slot"));
        in.q_len = Pp<const int>(ptr(d, "q_len"));
        in.q_seq = Pp<const int>(ptr(d, "q_seq"));
        in.block_table = Pp<const int>(ptr(d, "block_table"));
        in.max_blocks = geti(d, "max_blocks");
        in.bs = geti(d, "bs", 16);
        in.logits = Pp<float>(ptr(d, "logits"));
        in.ld_logits = geti(d, "ld_logits");
        in.logit_idx = Pp<const int>(ptr(d, "logit_idx"));
        if (in.bs <= 0 || in.max_blocks <= 0) throw std::runtime_error("bad block geometry");
        e.validate();
      })
      .def("bind_tiles", [](StackExecutor& e, uintptr_t table, int max_tiles) {
        e.tiles = Pp<const int>(table);
        e.max_tiles = max_tiles;
      })
      .def("set_tiles", [](StackExecutor& e, int n) {
        if (n < 0 || n > e.max_tiles) throw std::runtime_error("stack executor: tile count outside the table");
        e.n_tiles = n;
      })
      .def("set_splits", [](StackExecutor& e, int n) {
        if (n < 1 || n > 64) throw std::runtime_error("stack executor: splits outside 1..64");
        e.n_splits = n;
      })
      .def("set_chunks", [](StackExecutor& e, int n) {
        if (n < 0 || n > e.ws.ret.max_chunks) throw std::runtime_error("stack executor: chunk count outside the table");
        e.n_chunks = n;
      })
      .def("step", [](StackExecutor& e, int stage, int idx, int B, int n_logits, bool use_idx, uintptr_t stream) {
        if (B <= 0 || B > e.cfg.max_B || n_logits < 0 || n_logits > e.cfg.max_B)
          throw std::runtime_error("stack executor: rows outside 1..max_B");
        if (use_idx && !e.in.logit_idx) throw std::runtime_error("stack executor: no logit index bound");
        hipStream_t s = S(stream);
        switch (stage) {
          case ST_FORWARD: e.forward(B, n_logits, use_idx, s); break;
          case ST_EMBED: e.embed(B, s); break;
          case ST_RUN:
            if (idx < 0 || idx >= (int)e.runs.size()) throw std::runtime_error("stack executor: bad run index");
            e.layer_run(idx, B, s);
            break;
          case ST_HEAD: e.head(n_logits, use_idx, s); break;
          default: throw std::runtime_error("stack executor: unknown stage");
        }
      });
}
