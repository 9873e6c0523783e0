// Kernels of layers with RMS norms (weight vectors) on the inputs of both sublayers: the norm itself, the
// finishing of differential attention (two softmax maps per head over the same values), the preparation of
// attention whose scores are mixed across the heads before the softmax (rotation + the queries folded through
// the mixing matrix), a gated dense feed-forward with a relu gate, and a sigmoid router with ranked groups.
// float32 for norms, angles, gates and router; `T` is the matrix dtype (bfloat16 or float32).
#include "stack_device.h"
#include "stack_ops.h"

#include <algorithm>

namespace omx {
namespace stack {

// ------------------------------------------------------------------------------------------------ RMS norm
// out[r] = x[row] / sqrt(mean(x[row]^2) + eps) * w, one block per row
template <typename T>
__global__ __launch_bounds__(256) void rms_norm_cast_kernel(const float* __restrict__ x, const int* __restrict__ idx, int E,
                                                            const float* __restrict__ w, float eps, T* __restrict__ out) {
  __shared__ float red[4];
  const long long r = blockIdx.x;
  const float* xr = x + (idx ? (long long)idx[r] : r) * E;
  float ss = 0.f;
  for (int c = threadIdx.x; c < E; c += 256) ss += xr[c] * xr[c];
  const float inv = 1.f / sqrtf(block_sum256(ss, red) / (float)E + eps);
  for (int c = threadIdx.x; c < E; c += 256) st(out + r * E + c, xr[c] * inv * w[c]);
}
void rms_norm_cast(const float* x, const int* idx, int rows, int E, const float* w, float eps, void* out, int f32, hipStream_t s) {
  check(rows > 0 && E > 0 && x && w && out, "rms_norm_cast: bad operands");
  if (f32)
    hipLaunchKernelGGL(rms_norm_cast_kernel<float>, dim3(rows), dim3(256), 0, s, x, idx, E, w, eps, (float*)out);
  else
    hipLaunchKernelGGL(rms_norm_cast_kernel<bf16>, dim3(rows), dim3(256), 0, s, x, idx, E, w, eps, (bf16*)out);
  launched("rms_norm_cast");
}

// ------------------------------------------------------------------------------------------------ differential attention
// One wave per (row, head): o = a1 - lam a2 over the head's Dv values (a1, a2: the two maps' outputs, float32, side
// by side), o / sqrt(mean(o^2) + eps) * (1 - diff) * sigmoid(gate), written in the matrix dtype.
template <typename T>
__global__ __launch_bounds__(256) void diff_combine_kernel(const float* __restrict__ o32, int ld_o, int B, int H, int Dv, float lam,
                                                           float diff, float eps, const float* __restrict__ gate, int ld_gate,
                                                           T* __restrict__ out, int ld_out) {
  const int lane = threadIdx.x & 63;
  const long long item = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= (long long)B * H) return;
  const long long b = item / H;
  const int h = (int)(item % H);
  const float* a1 = o32 + b * ld_o + (long long)2 * h * Dv;
  const float* a2 = a1 + Dv;
  float o[4], ss = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int d = lane + 64 * c;
    o[c] = d < Dv ? a1[d] - lam * a2[d] : 0.f;
    ss += o[c] * o[c];
  }
  const float f = (1.f - diff) / sqrtf(wave_sum(ss) / (float)Dv + eps);
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int d = lane + 64 * c;
    if (d < Dv) st(out + b * ld_out + h * Dv + d, o[c] * f * (gate ? sigmoidf(gate[b * ld_gate + h * Dv + d]) : 1.f));
  }
}
void diff_combine(const float* o32, int ld_o, int B, int H, int Dv, float lam, float diff, float eps, const float* gate, int ld_gate,
                  void* out, int ld_out, int f32, hipStream_t s) {
  check(B > 0 && o32 && out && H > 0 && Dv > 0 && Dv <= 256 && ld_o >= 2 * H * Dv && ld_out >= H * Dv,
        "diff_combine: bad operands (value size up to 256)");
  const dim3 grid((unsigned)(((long long)B * H + 3) / 4));
  if (f32)
    hipLaunchKernelGGL(diff_combine_kernel<float>, grid, dim3(256), 0, s, o32, ld_o, B, H, Dv, lam, diff, eps, gate, ld_gate,
                       (float*)out, ld_out);
  else
    hipLaunchKernelGGL(diff_combine_kernel<bf16>, grid, dim3(256), 0, s, o32, ld_o, B, H, Dv, lam, diff, eps, gate, ld_gate,
                       (bf16*)out, ld_out);
  launched("diff_combine");
}

// ------------------------------------------------------------------------------------------------ rotation + folded queries
// One block per (row, slice of the folded queries). The block rotates the row's H query heads into LDS (pairs
// (2i, 2i + 1), angle pos * inv_freq[i] reduced in float64); block slice 0 also rotates the G keys into the row's
// slot of the K pool, whose row holds the G keys side by side, and stores the values. Then
//   qf[h][c][d] = sum over the heads g = c * per + j of key/value head c of mix[h][g] * q_rot[g][d],
// so that qf[h] . [k_0 | ... | k_(G-1)] = sum_g mix[h][g] (q_g . k_c(g)): the mixed score of head h.
template <typename T>
__global__ __launch_bounds__(256) void rotate_fold_kernel(RotFoldParams P, StepRows R) {
  extern __shared__ float lds[];
  const int half = P.rot_dims / 2, D = P.D, H = P.H, G = P.G, per = H / G;
  float* cs = lds;            // [half]
  float* sn = lds + half;     // [half]
  float* qr = lds + 2 * half; // [H * D]
  const int b = blockIdx.x;
  const float* row = P.proj + (long long)b * P.ld;
  const int pos = R.pos[b];
  for (int i = threadIdx.x; i < half; i += 256) {
    const double ang = (double)pos * P.inv_freq[i];
    const float red = (float)(ang - 6.283185307179586 * rint(ang * 0.15915494309189535));
    cs[i] = cosf(red);
    sn[i] = sinf(red);
  }
  __syncthreads();
  auto rotated = [&](int col, int idx) {  // element idx of a stack of heads that starts at column col
    const int d = idx % D;
    const float x = row[col + idx];
    if (d >= 2 * half) return x;
    const float y = row[col + (idx ^ 1)];
    return (d & 1) ? x * cs[d >> 1] + y * sn[d >> 1] : x * cs[d >> 1] - y * sn[d >> 1];
  };
  for (int i = threadIdx.x; i < H * D; i += 256) qr[i] = rotated(P.off_q, i);
  if (blockIdx.y == 0) {
    const int slot = R.slot[b];
    const long long blk = slot / R.bs, off = slot % R.bs;
    T* kc = (T*)P.kc + (blk * R.bs + off) * (long long)(G * D);
    for (int i = threadIdx.x; i < G * D; i += 256) st(kc + i, rotated(P.off_k, i));
    T* vc = (T*)P.vc;
    for (int i = threadIdx.x; i < G * P.Dv; i += 256) {
      const int g = i / P.Dv, d = i % P.Dv;
      st(vc + ((blk * G + g) * R.bs + off) * P.Dv + d, row[P.off_v + i]);
    }
  }
  __syncthreads();
  float* qf = P.qf + (long long)b * P.ld_qf;
  const int n = H * G * D;
  for (int i = blockIdx.y * 256 + threadIdx.x; i < n; i += 256 * gridDim.y) {
    const int h = i / (G * D), c = (i / D) % G, d = i % D;
    const float* mx = P.mix + h * H + c * per;
    const float* q = qr + (c * per) * D + d;
    float acc = 0.f;
    for (int j = 0; j < per; ++j) acc += mx[j] * q[j * D];
    qf[i] = acc;
  }
}
bool rotate_fold_supported(int H, int G, int D) {
  return H > 0 && G > 0 && H % G == 0 && D > 0 && (long long)(H + 1) * D <= 12288 && (long long)G * D <= 1024;
}
void rotate_fold(const RotFoldParams& P, const StepRows& R, hipStream_t s) {
  check(R.B > 0 && P.proj && P.kc && P.vc && P.qf && P.mix && rotate_fold_supported(P.H, P.G, P.D) && P.Dv > 0 && P.rot_dims >= 0 &&
            P.rot_dims % 2 == 0 && P.rot_dims <= P.D && (P.rot_dims == 0 || P.inv_freq) && P.ld_qf >= P.H * P.G * P.D,
        "rotate_fold: bad operands (heads * dim up to 12288, key/value heads * dim up to 1024)");
  const int n = P.H * P.G * P.D;
  const dim3 grid(R.B, R.B <= 64 ? std::max(1, std::min(16, n / 1024)) : 1);  // few rows: the fold shared among blocks
  const size_t lds = (size_t)(P.rot_dims + P.H * P.D) * sizeof(float);
  if (P.f32)
    hipLaunchKernelGGL(rotate_fold_kernel<float>, grid, dim3(256), lds, s, P, R);
  else
    hipLaunchKernelGGL(rotate_fold_kernel<bf16>, grid, dim3(256), lds, s, P, R);
  launched("rotate_fold");
}

// ------------------------------------------------------------------------------------------------ gated dense feed-forward
// out = relu(z[:, :F]) * z[:, F:2F], matrix dtype
template <typename T>
__global__ __launch_bounds__(256) void relu_glu_kernel(const float* __restrict__ z, int ld, int rows, int F, T* __restrict__ out,
                                                       int ld_out) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long long)rows * F) return;
  const long long r = i / F;
  const int f = (int)(i % F);
  st(out + r * ld_out + f, fmaxf(z[r * ld + f], 0.f) * z[r * ld + F + f]);
}
void relu_glu_cast(const float* z, int ld, int rows, int F, void* out, int ld_out, int f32, hipStream_t s) {
  check(rows > 0 && F > 0 && z && out && ld >= 2 * F && ld_out >= F, "relu_glu_cast: bad operands");
  const long long n = (long long)rows * F;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (f32)
    hipLaunchKernelGGL(relu_glu_kernel<float>, grid, dim3(256), 0, s, z, ld, rows, F, (float*)out, ld_out);
  else
    hipLaunchKernelGGL(relu_glu_kernel<bf16>, grid, dim3(256), 0, s, z, ld, rows, F, (bf16*)out, ld_out);
  launched("relu_glu_cast");
}
// out[m][k] = relu(A[m] . W[k]) * (A[m] . W[F + k]), matrix dtype: the gate / up projection of a few rows with its
// activation in one launch (W [2F][K]: gate rows, then up rows); one wave per hidden unit takes both rows
template <typename T>
__global__ __launch_bounds__(256) void gemv_relu_glu_kernel(const T* __restrict__ A, int lda, const T* __restrict__ W, int K, int F,
                                                            int M, T* __restrict__ out, int ld_out, int vec) {
  const int lane = threadIdx.x & 63;
  const int f = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (f >= F) return;
  const T* wg = W + (long long)f * K;
  const T* wu = W + (long long)(F + f) * K;
  for (int m = 0; m < M; ++m) {
    const T* x = A + (long long)m * lda;
    const float g = wave_dot<T>(wg, x, K, lane, vec != 0), u = wave_dot<T>(wu, x, K, lane, vec != 0);
    if (lane == 0) st(out + (long long)m * ld_out + f, fmaxf(g, 0.f) * u);
  }
}
void gemv_relu_glu(const void* A, int lda, const void* W, int K, int F, int M, void* out, int ld_out, int f32, hipStream_t s) {
  check(M > 0 && M <= 16 && A && W && out && K > 0 && F > 0 && ld_out >= F, "gemv_relu_glu: bad operands (up to 16 rows)");
  const dim3 grid((F + 3) / 4);
  if (f32)
    hipLaunchKernelGGL(gemv_relu_glu_kernel<float>, grid, dim3(256), 0, s, (const float*)A, lda, (const float*)W, K, F, M, (float*)out,
                       ld_out, (int)(vec_ok<float>(A, lda, K) && vec_ok<float>(W, K, K)));
  else
    hipLaunchKernelGGL(gemv_relu_glu_kernel<bf16>, grid, dim3(256), 0, s, (const bf16*)A, lda, (const bf16*)W, K, F, M, (bf16*)out,
                       ld_out, (int)(vec_ok<bf16>(A, lda, K) && vec_ok<bf16>(W, K, K)));
  launched("gemv_relu_glu");
}

// ------------------------------------------------------------------------------------------------ sigmoid router
// Per row: s = sigmoid of the X router logits. The experts form group_count groups of neighbours; a group ranks by
// the sum of its two largest scores and only experts of the best group_keep groups can be chosen; the `top` largest
// scores among them are taken (ties: the lower index), divided by their sum (+ 1e-20) and multiplied by route_scale.
// One wave per row with an expert per lane (X <= 64); lane q < top ends up holding the q-th choice.
__device__ __forceinline__ void route_sigmoid_wave(const MoeParams& P, const float* row, int lane, int& who_q, float& w_q) {
  const bool has = lane < P.X;
  const float sc = has ? sigmoidf(row[P.off_router + lane]) : -INFINITY;
  float ch = sc;
  if (P.group_count > 1) {
    const int per = P.X / P.group_count, mine = has ? lane / per : -1;
    // this lane's group's rank: every lane walks its own group's scores (the groups are neighbours, so one lane
    // exchange per member) and keeps the two largest
    const int base = has ? mine * per : lane;
    float m1 = -INFINITY, m2 = -INFINITY;
    for (int i = 0; i < per; ++i) {
      const float v = __shfl(sc, has ? base + i : lane, 64);
      if (v > m1) {
        m2 = m1;
        m1 = v;
      } else if (v > m2) {
        m2 = v;
      }
    }
    float gs = has ? m1 + (m2 == -INFINITY ? 0.f : m2) : -INFINITY;
    bool kept = false;
    for (int q = 0; q < P.group_keep; ++q) {
      const float best = wave_max(gs);
      const int who = max(0, __ffsll((unsigned long long)__ballot(gs == best && has)) - 1);  // lowest lane of the best group
      if (mine == who / per) {
        kept = true;
        gs = -INFINITY;
      }
    }
    if (!kept) ch = -INFINITY;
  }
  who_q = 0;
  w_q = 0.f;
  for (int q = 0; q < P.top; ++q) {
    const float mx = wave_max(ch);
    // non-finite logits (a fault upstream) compare unequal to everything: expert 0 then, never an index of -1
    const int who = max(0, __ffsll((unsigned long long)__ballot(ch == mx && has)) - 1);
    if (lane == q) {
      who_q = who;
      w_q = mx;
    }
    if (lane == who) ch = -INFINITY;
  }
  const float sum = wave_sum(lane < P.top ? w_q : 0.f) + 1e-20f;
  w_q = w_q / sum * P.route_scale;
}
// the same by one thread, for up to 256 experts (sc: X floats of scratch)
__device__ void route_sigmoid_serial(const MoeParams& P, const float* row, float* sc, int* ids, float* wts) {
  for (int e = 0; e < P.X; ++e) sc[e] = sigmoidf(row[P.off_router + e]);
  if (P.group_count > 1) {
    const int per = P.X / P.group_count;
    unsigned long long kept = 0ull;
    for (int q = 0; q < P.group_keep; ++q) {
      int best = -1;
      float bv = -INFINITY;
      for (int gi = 0; gi < P.group_count; ++gi) {
        if (kept >> gi & 1ull) continue;
        float m1 = -INFINITY, m2 = -INFINITY;
        for (int e = gi * per; e < (gi + 1) * per; ++e) {
          const float v = sc[e];
          if (v > m1) {
            m2 = m1;
            m1 = v;
          } else if (v > m2) {
            m2 = v;
          }
        }
        const float gs = m1 + (m2 == -INFINITY ? 0.f : m2);
        if (best < 0 || gs > bv) {
          best = gi;
          bv = gs;
        }
      }
      kept |= 1ull << best;
    }
    for (int gi = 0; gi < P.group_count; ++gi)
      if (!(kept >> gi & 1ull))
        for (int e = gi * per; e < (gi + 1) * per; ++e) sc[e] = -1.f;  // a score is positive: never chosen before a kept one
  }
  float sum = 1e-20f;
  for (int jj = 0; jj < P.top; ++jj) {
    int best = 0;
    float bv = -INFINITY;
    for (int e = 0; e < P.X; ++e)
      if (sc[e] > bv) {
        best = e;
        bv = sc[e];
      }
    sc[best] = -2.f;
    ids[jj] = best;
    wts[jj] = bv;
    sum += bv;
  }
  for (int jj = 0; jj < P.top; ++jj) wts[jj] = wts[jj] / sum * P.route_scale;
}
constexpr int ROUTE_SIG_MAX = 256;
__global__ __launch_bounds__(256) void moe_route_sigmoid_kernel(MoeParams P) {
  __shared__ float sc[4][ROUTE_SIG_MAX];
  __shared__ int ids[4][MOE_MAX_TOP];
  __shared__ float wts[4][MOE_MAX_TOP];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int b = blockIdx.x * 4 + wv;
  if (b >= P.B) return;
  const float* row = P.proj + (long long)b * P.ld;
  if (P.X <= 64) {
    int who;
    float w;
    route_sigmoid_wave(P, row, lane, who, w);
    if (lane < P.top) {
      P.eids[(long long)b * P.ld_top + lane] = who;
      P.ew[(long long)b * P.ld_top + lane] = w;
    }
  } else if (lane == 0) {
    route_sigmoid_serial(P, row, sc[wv], ids[wv], wts[wv]);
    for (int q = 0; q < P.top; ++q) {
      P.eids[(long long)b * P.ld_top + q] = ids[wv][q];
      P.ew[(long long)b * P.ld_top + q] = wts[wv][q];
    }
  }
}
static void check_route_sigmoid(const MoeParams& P) {
  check(P.B > 0 && P.proj && P.eids && P.ew && P.X > 0 && P.X <= ROUTE_SIG_MAX && P.top > 0 && P.top <= MOE_MAX_TOP && P.top <= P.X &&
            P.ld_top >= P.top && P.group_count >= 1 && P.group_count <= 64 && P.X % P.group_count == 0 && P.group_keep >= 1 &&
            P.group_keep <= P.group_count && P.group_keep * (P.X / P.group_count) >= P.top && P.Fs == 0 && P.identity == 0,
        "sigmoid router: operands or sizes (up to 256 experts in up to 64 groups, top <= 16)");
}
void moe_route_sigmoid(const MoeParams& P, hipStream_t s) {
  check_route_sigmoid(P);
  hipLaunchKernelGGL(moe_route_sigmoid_kernel, dim3((P.B + 3) / 4), dim3(256), 0, s, P);
  launched("moe_route_sigmoid");
}
// ---- a few rows (decode steps): routing and the routed activations in one launch. Grid (ff units / 4, row x top);
// every wave routes its row itself (a few dozen operations) and takes hidden unit f of routed expert jj; block
// (0, row, 0) records ids and weights for the down projection.
template <typename T>
__global__ __launch_bounds__(256) void moe_route_sigmoid_experts_kernel(MoeParams P, int vec) {
  const int lane = threadIdx.x & 63;
  const int f = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int b = blockIdx.y / P.top, jj = blockIdx.y % P.top;
  const float* row = P.proj + (long long)b * P.ld;
  int who;
  float w;
  route_sigmoid_wave(P, row, lane, who, w);
  if (threadIdx.x < P.top && blockIdx.x == 0 && jj == 0) {
    P.eids[(long long)b * P.ld_top + lane] = who;
    P.ew[(long long)b * P.ld_top + lane] = w;
  }
  const int e = __shfl(who, jj, 64);
  if (f >= P.F) return;
  const T* x = (const T*)P.h + (long long)b * P.E;
  const T* wg = (const T*)P.w_gu + ((long long)e * 2 * P.F + f) * P.E;
  const T* wu = wg + (long long)P.F * P.E;
  const float gate = wave_dot<T>(wg, x, P.E, lane, vec != 0);
  const float up = wave_dot<T>(wu, x, P.E, lane, vec != 0);
  if (lane == 0) st((T*)P.hmid + (long long)b * P.ld_hmid + jj * P.F + f, silu(gate) * up);
}
bool moe_route_sigmoid_fused_supported(const MoeParams& P) { return P.X <= 64; }
void moe_route_sigmoid_experts(const MoeParams& P, hipStream_t s) {
  check_route_sigmoid(P);
  check(moe_route_sigmoid_fused_supported(P) && P.h && P.w_gu && P.hmid && P.F > 0 && P.ld_hmid >= P.top * P.F,
        "fused sigmoid router: operands or sizes (up to 64 experts)");
  const dim3 grid((P.F + 3) / 4, P.B * P.top);
  if (P.f32)
    hipLaunchKernelGGL(moe_route_sigmoid_experts_kernel<float>, grid, dim3(256), 0, s, P,
                       (int)(vec_ok<float>(P.h, P.E, P.E) && vec_ok<float>(P.w_gu, P.E, P.E)));
  else
    hipLaunchKernelGGL(moe_route_sigmoid_experts_kernel<bf16>, grid, dim3(256), 0, s, P,
                       (int)(vec_ok<bf16>(P.h, P.E, P.E) && vec_ok<bf16>(P.w_gu, P.E, P.E)));
  launched("moe_route_sigmoid_experts");
}

}  // namespace stack
}  // namespace omx
