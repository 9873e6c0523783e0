// gfx950 kernels of the layers with scalar-weight RMS norms before and after both sublayers (interface:
// stack_ops.h): the input norm with the short causal convolution that is added to the mixer's input and its
// carried window, the finishing of queries and keys (biases, RMS norms before or after a rotate-half rotation
// with float64 angles, the K/V store), the mixing of the heads' attention weights, gated linear attention with a
// per-channel decay (token by token with the state in registers, and in chunks for prompt portions), the
// norm + per-channel scale + residual update, and the gated feed-forward's activation.
// Everything but the matrix operands and the K/V pools is float32. Wave = 64 lanes.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>

#include "stack_device.h"
#include "stack_ops.h"

namespace omx {
namespace stack {

// ------------------------------------------------------------------------------------------------ input norm + convolution
// One block per row r. hn[r] = x[r] * g / rms(x[r]); out[r][c] = hn[r][c] + sum_j w[c][j] hn(p_r - (taps - 1) + j)[c].
// Inputs of earlier rows of the same step are recomputed from the stream with their own row's scale (the same
// operations in the same order as that row's block, so the value is the same bit for bit); inputs from before the
// step's first row of the sequence come from its carried window (the last taps - 1 normed rows, oldest first; zero
// for a new sequence). A sequence with a single row in the step advances its window there and then; for the others
// a second launch does, by the block of the sequence's LAST row, from hn.
template <typename T>
__global__ __launch_bounds__(256) void scalar_norm_conv_kernel(CanonParams P, StepRows R) {
  __shared__ float red[4];
  const int r = blockIdx.x, K = P.taps, E = P.E;
  const int seq = R.q_seq[r];
  int nb = 0;  // rows of the same sequence right before r, up to taps - 1
  while (nb < K - 1 && r - nb - 1 >= 0 && R.q_seq[r - nb - 1] == seq) ++nb;
  const bool alone = nb == 0 && !(r + 1 < R.B && R.q_seq[r + 1] == seq);
  const float g = P.g[0];
  float scale[CANON_MAX_TAPS];  // indexed by constants only (unrolled), so it lives in registers
#pragma unroll
  for (int k = 0; k < CANON_MAX_TAPS; ++k) {
    scale[k] = 0.f;
    if (k <= nb) {  // uniform over the block
      const float* xr = P.x + (long long)(r - k) * E;
      float ss = 0.f;
      for (int c = threadIdx.x; c < E; c += 256) ss += xr[c] * xr[c];
      scale[k] = g / sqrtf(block_sum256(ss, red) / (float)E + P.eps);
    }
  }
  float* win = P.window ? P.window + (long long)seq * P.stride : nullptr;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < E; c += 256 * gridDim.y) {
    const float cur = P.x[(long long)r * E + c] * scale[0];
    P.hn[(long long)r * E + c] = cur;
    float acc = cur;
#pragma unroll
    for (int back = CANON_MAX_TAPS - 1; back >= 0; --back) {  // oldest input first, as the taps are stored
      if (back < K) {
        const float v = back == 0 ? cur : back <= nb ? P.x[(long long)(r - back) * E + c] * scale[back]
                                                     : win[(long long)(K - 1 - (back - nb)) * E + c];
        acc += P.w[(long long)c * K + (K - 1 - back)] * v;
        if (alone && back > 0) win[(long long)(K - 1 - back) * E + c] = back == 1 ? cur : win[(long long)(K - back) * E + c];
      }
    }
    st((T*)P.out + (long long)r * E + c, acc);
  }
}
__global__ __launch_bounds__(256) void canon_window_kernel(CanonParams P, StepRows R) {
  const int r = blockIdx.x, K = P.taps, E = P.E;
  const int seq = R.q_seq[r];
  if (r + 1 < R.B && R.q_seq[r + 1] == seq) return;  // not the sequence's last row of this step
  if (!(r > 0 && R.q_seq[r - 1] == seq)) return;     // its only row: the first launch advanced the window
  int n = 1;  // rows of the sequence in this step, up to taps - 1
  while (n < K - 1 && r - n >= 0 && R.q_seq[r - n] == seq) ++n;
  float* win = P.window + (long long)seq * P.stride;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < E; c += 256 * gridDim.y)
    for (int sidx = 0; sidx < K - 1; ++sidx) {  // ascending: a thread never reads what it has overwritten
      const int back = K - 2 - sidx;
      win[(long long)sidx * E + c] = back < n ? P.hn[(long long)(r - back) * E + c] : win[(long long)(sidx + n) * E + c];
    }
}
void scalar_norm_conv(const CanonParams& P, const StepRows& R, hipStream_t s) {
  check(R.B > 0 && P.x && P.g && P.hn && P.out && P.E > 0 && P.taps >= 1 && P.taps <= CANON_MAX_TAPS && P.w &&
            (P.taps == 1 || P.window),
        "scalar_norm_conv: bad operands (at most 8 taps)");
  // few rows (decode steps): the channels are shared among several blocks per row (each sums the whole row itself)
  const dim3 grid(R.B, R.B <= 64 ? std::min(8, (P.E + 255) / 256) : 1);
  if (P.f32)
    hipLaunchKernelGGL(scalar_norm_conv_kernel<float>, grid, dim3(256), 0, s, P, R);
  else
    hipLaunchKernelGGL(scalar_norm_conv_kernel<bf16>, grid, dim3(256), 0, s, P, R);
  launched("scalar_norm_conv");
  if (P.taps > 1 && R.B > 1) {  // a single row is alone in its sequence
    hipLaunchKernelGGL(canon_window_kernel, dim3(R.B, (P.E + 1023) / 1024), dim3(256), 0, s, P, R);
    launched("canon_window");
  }
}

template <typename T>
__global__ __launch_bounds__(256) void scalar_norm_cast_kernel(const float* __restrict__ x, const int* __restrict__ idx, int E,
                                                               const float* __restrict__ g, float eps, T* __restrict__ out) {
  __shared__ float red[4];
  const long long r = blockIdx.x;
  const float* xr = x + (idx ? (long long)idx[r] : r) * E;
  float ss = 0.f;
  for (int c = threadIdx.x; c < E; c += 256) ss += xr[c] * xr[c];
  const float scale = g[0] / sqrtf(block_sum256(ss, red) / (float)E + eps);
  for (int c = threadIdx.x; c < E; c += 256) st(out + r * E + c, xr[c] * scale);
}
void scalar_norm_cast(const float* x, const int* idx, int rows, int E, const float* g, float eps, void* out, int f32,
                      hipStream_t s) {
  check(rows > 0 && E > 0 && x && g && out, "scalar_norm_cast: bad operands");
  if (f32)
    hipLaunchKernelGGL(scalar_norm_cast_kernel<float>, dim3(rows), dim3(256), 0, s, x, idx, E, g, eps, (float*)out);
  else
    hipLaunchKernelGGL(scalar_norm_cast_kernel<bf16>, dim3(rows), dim3(256), 0, s, x, idx, E, g, eps, (bf16*)out);
  launched("scalar_norm_cast");
}

// ------------------------------------------------------------------------------------------------ queries and keys
// One block per row; its four waves take the H query heads and G key heads in turn (a head per wave and turn,
// four elements per lane: D <= 256). Per head: + bias; (the key as it stands is the value row, if the values are
// the keys); RMS norm with a weight; rotation of the pairs (i, i + rot_dims / 2) by pos * inv_freq[i], the angle
// and its sine / cosine in float64; unit RMS. Queries go back to proj in place, keys to the row's cache slot.
// The value rows (+ bias) are stored by all threads at the end.
constexpr int QK_MAXD = 256;
template <typename T>
__global__ __launch_bounds__(256) void qk_prepare_kernel(QkPrepParams P, StepRows R) {
  __shared__ float cs[QK_MAXD / 2], sn[QK_MAXD / 2];
  __shared__ float stage[4][QK_MAXD];
  const int b = blockIdx.x, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  float* row = P.proj + (long long)b * P.ld;
  const int pos = R.pos[b], half = P.rot_dims / 2, D = P.D;
  for (int i = threadIdx.x; i < half; i += 256) {
    // the angle and its reduction to [-pi, pi] in float64 (a float32 angle at position 10^3 is off by 10^-4); the
    // sine and cosine of the reduced angle in float32
    const double ang = (double)pos * P.inv_freq[i];
    const float red = (float)(ang - 6.283185307179586 * rint(ang * 0.15915494309189535));
    cs[i] = cosf(red);
    sn[i] = sinf(red);
  }
  const int slot = R.slot[b];
  const long long blk = slot / R.bs, off = slot % R.bs;
  T* kc = (T*)P.kc;
  T* vc = (T*)P.vc;
  const int heads = P.H + P.G;
  // turns of four heads (a head per wave); with several blocks per row (gridDim.y) a block takes every gridDim.y-th
  // turn, and every wave of a block sees the same number of turns: block-wide barriers inside
  for (int h0 = 4 * blockIdx.y; h0 < heads; h0 += 4 * gridDim.y) {
    const int head = h0 + wv;
    const bool on = head < heads, isq = head < P.H;
    const int hh = isq ? head : head - P.H;
    const int col = isq ? P.off_q + hh * D : P.off_k + hh * D;
    float v[4];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int d = lane + 64 * c;
      v[c] = (on && d < D) ? row[col + d] + (P.bias ? P.bias[col + d] : 0.f) : 0.f;
      ss += v[c] * v[c];
    }
    if (on && !isq && P.v_from_k) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int d = lane + 64 * c;
        if (d < D) st(vc + ((blk * P.G + hh) * R.bs + off) * P.Dv + d, v[c]);
      }
    }
    if (P.qk_norm == QK_NORM_WEIGHT_FIRST) {
      const float inv = 1.f / sqrtf(wave_sum(ss) / (float)D + P.eps);
      const float* w = isq ? P.q_norm : P.k_norm;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int d = lane + 64 * c;
        if (d < D) v[c] *= inv * w[d];
      }
    }
    if (half > 0) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int d = lane + 64 * c;
        if (d < D) stage[wv][d] = v[c];
      }
      __syncthreads();
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int d = lane + 64 * c;
        if (d < half)
          v[c] = v[c] * cs[d] - stage[wv][d + half] * sn[d];
        else if (d < 2 * half)
          v[c] = v[c] * cs[d - half] + stage[wv][d - half] * sn[d - half];
      }
      __syncthreads();
    }
    if (P.qk_norm == QK_NORM_UNIT_LAST) {
      ss = 0.f;
#pragma unroll
      for (int c = 0; c < 4; ++c) ss += (lane + 64 * c < D) ? v[c] * v[c] : 0.f;
      const float inv = 1.f / sqrtf(wave_sum(ss) / (float)D + P.eps);
#pragma unroll
      for (int c = 0; c < 4; ++c) v[c] *= inv;
    }
    if (on) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int d = lane + 64 * c;
        if (d < D) {
          if (isq)
            row[col + d] = v[c];
          else
            st(kc + ((blk * P.G + hh) * R.bs + off) * D + d, v[c]);
        }
      }
    }
  }
  if (!P.v_from_k && blockIdx.y == gridDim.y - 1) {
    for (int i = threadIdx.x; i < P.G * P.Dv; i += 256) {
      const int g = i / P.Dv, d = i % P.Dv;
      st(vc + ((blk * P.G + g) * R.bs + off) * P.Dv + d, row[P.off_v + i] + (P.bias ? P.bias[P.off_v + i] : 0.f));
    }
  }
}
void qk_prepare(const QkPrepParams& P, const StepRows& R, hipStream_t s) {
  check(R.B > 0 && P.proj && P.kc && P.vc && P.H > 0 && P.G > 0 && P.D > 0 && P.D <= QK_MAXD && P.rot_dims >= 0 &&
            P.rot_dims % 2 == 0 && P.rot_dims <= P.D && (P.rot_dims == 0 || P.inv_freq) &&
            (P.qk_norm != QK_NORM_WEIGHT_FIRST || (P.q_norm && P.k_norm)) && (!P.v_from_k || P.Dv == P.D),
        "qk_prepare: bad operands (head size up to 256)");
  // few rows (decode steps): a block per turn of four heads, so a row's heads are finished side by side
  const int turns = (P.H + P.G + 3) / 4;
  const dim3 grid(R.B, R.B <= 64 ? turns : 1);
  if (P.f32)
    hipLaunchKernelGGL(qk_prepare_kernel<float>, grid, dim3(256), 0, s, P, R);
  else
    hipLaunchKernelGGL(qk_prepare_kernel<bf16>, grid, dim3(256), 0, s, P, R);
  launched("qk_prepare");
}

// ------------------------------------------------------------------------------------------------ mixed heads
template <typename T>
__global__ __launch_bounds__(256) void talk_mix_kernel(const float* __restrict__ o32, int ld_o, int H, int G, int Dv,
                                                       const float* __restrict__ talk, T* __restrict__ out, int ld_out) {
  const long long b = blockIdx.x;
  const float* src = o32 + b * ld_o;
  const int per = H / G;
  for (int i = blockIdx.y * 256 + threadIdx.x; i < H * Dv; i += 256 * gridDim.y) {
    const int h = i / Dv, d = i % Dv, c = h / per;
    float acc = 0.f;
    for (int g = 0; g < H; ++g) acc += talk[h * H + g] * src[(long long)(g * G + c) * Dv + d];
    st(out + b * ld_out + i, acc);
  }
}
void talk_mix(const float* o32, int ld_o, int B, int H, int G, int Dv, const float* talk, void* out, int ld_out, int f32,
              hipStream_t s) {
  check(B > 0 && o32 && talk && out && H > 0 && G > 0 && H % G == 0 && ld_o >= H * G * Dv && ld_out >= H * Dv,
        "talk_mix: bad operands");
  if (f32)
    hipLaunchKernelGGL(talk_mix_kernel<float>, dim3(B, (H * Dv + 255) / 256), dim3(256), 0, s, o32, ld_o, H, G, Dv, talk,
                       (float*)out, ld_out);
  else
    hipLaunchKernelGGL(talk_mix_kernel<bf16>, dim3(B, (H * Dv + 255) / 256), dim3(256), 0, s, o32, ld_o, H, G, Dv, talk,
                       (bf16*)out, ld_out);
  launched("talk_mix");
}

// ------------------------------------------------------------------------------------------------ gated linear attention
// S_t = diag(alpha_t) S_(t-1) + k_t v_t^T (S is D x Dv per head; the decay acts on the rows, one per key channel),
// o_t = S_t^T q_t, q scaled by D^(-1/2); ln alpha = logsigmoid(a2 . a1_t + a2_b) / tau.
// Token by token: one block per (sequence segment of the step, head), as the retention kernel: the block of the
// segment's first row walks its rows; thread (g, j) = (tid / Dv, tid % Dv) keeps S[i][j], i = g, g + NG, ..., in
// registers; o is a sum of NG partials per column; the head's RMS norm, its weight and the silu gate finish the row.
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }
template <typename T>
__device__ __forceinline__ void load8w(const T* p, float* out);
template <>
__device__ __forceinline__ void load8w<bf16>(const bf16* p, float* out) {
  const u32x4 a = *(const u32x4*)p;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    out[2 * i] = __uint_as_float(a[i] << 16);
    out[2 * i + 1] = __uint_as_float(a[i] & 0xffff0000u);
  }
}
template <>
__device__ __forceinline__ void load8w<float>(const float* p, float* out) {
  const f32x4 a = *(const f32x4*)p, b = *(const f32x4*)(p + 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    out[i] = a[i];
    out[4 + i] = b[i];
  }
}
// a1: the row's first decay factor (rank floats, global or LDS); vec: a2's rows allow 16-byte loads (rank % 8 == 0)
template <typename T>
__device__ __forceinline__ float gla_ln_alpha(const GlaParams& P, const float* a1, int ch, int vec) {
  const T* w = (const T*)P.a2 + (long long)ch * P.rank;
  float z = P.a2_b[ch];
  if (vec) {
    for (int i = 0; i < P.rank; i += 8) {
      float w8[8];
      load8w<T>(w + i, w8);
#pragma unroll
      for (int u = 0; u < 8; ++u) z += w8[u] * a1[i + u];
    }
  } else {
    for (int i = 0; i < P.rank; ++i) z += ld(w + i) * a1[i];
  }
  return log_sigmoid(z) / P.tau;
}
static inline int gla_vec(const GlaParams& P) { return P.rank % 8 == 0 && ((uintptr_t)P.a2 & 15) == 0; }
constexpr int GLA_MAX_RANK = 256;
template <typename T, int MAXI>
__global__ __launch_bounds__(256) void gla_kernel(GlaParams P, StepRows R, int vec) {
  __shared__ float qs[256], ks[256], as[256], vs[256], po[256], red[4];
  __shared__ float a1s[GLA_MAX_RANK];
  const int r0 = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int seq = R.q_seq[r0];
  if (r0 > 0 && R.q_seq[r0 - 1] == seq) return;  // not the first row of its segment (uniform per block)
  const int D = P.D, Dv = P.Dv;
  const int NG = 256 / Dv;
  const int g = tid / Dv, j = tid % Dv;
  const bool act = g < NG;
  float* S0 = P.state + (long long)seq * P.state_stride + (long long)h * D * Dv;
  float S[MAXI];
#pragma unroll
  for (int ii = 0; ii < MAXI; ++ii) {
    const int i = g + ii * NG;
    S[ii] = (act && i < D) ? S0[(long long)i * Dv + j] : 0.f;
  }
  const float qscale = 1.f / sqrtf((float)D);
  for (int r = r0; r < R.B && R.q_seq[r] == seq; ++r) {
    const float* row = P.proj + (long long)r * P.ld;
    if (tid < P.rank) a1s[tid] = row[P.off_a1 + tid];
    if (tid < D) {
      qs[tid] = row[P.off_q + h * D + tid] * qscale;
      ks[tid] = row[P.off_k + h * D + tid];
    }
    if (tid < Dv) vs[tid] = row[P.off_v + h * Dv + tid];
    __syncthreads();
    if (tid < D) as[tid] = expf(gla_ln_alpha<T>(P, a1s, h * D + tid, vec));
    __syncthreads();
    float part = 0.f;
    if (act) {
      const float vj = vs[j];
#pragma unroll
      for (int ii = 0; ii < MAXI; ++ii) {
        const int i = g + ii * NG;
        if (i < D) {
          S[ii] = as[i] * S[ii] + ks[i] * vj;
          part += S[ii] * qs[i];
        }
      }
    }
    po[tid] = part;
    __syncthreads();
    float o = 0.f;
    if (tid < Dv)
      for (int gg = 0; gg < NG; ++gg) o += po[gg * Dv + tid];
    const float ms = block_sum256(o * o, red) / (float)Dv;
    if (tid < Dv) {
      const float y = o / sqrtf(ms + P.eps) * P.norm_w[tid] * silu(row[P.off_g + h * Dv + tid]);
      st((T*)P.out + (long long)r * P.ld_out + h * Dv + tid, y);
    }
    __syncthreads();
  }
#pragma unroll
  for (int ii = 0; ii < MAXI; ++ii) {
    const int i = g + ii * NG;
    if (act && i < D) S0[(long long)i * Dv + j] = S[ii];
  }
}
bool gla_supported(int D, int Dv) {
  if (D <= 0 || Dv <= 0 || D > 256 || Dv > 256) return false;
  const int ng = 256 / Dv;
  return (D + ng - 1) / ng <= 64;
}
template <typename T>
static void launch_gla(const GlaParams& P, const StepRows& R, hipStream_t s) {
  const int ng = 256 / P.Dv, ni = (P.D + ng - 1) / ng;
  const dim3 grid(R.B, P.H);
  if (ni <= 8)
    hipLaunchKernelGGL((gla_kernel<T, 8>), grid, dim3(256), 0, s, P, R, gla_vec(P));
  else if (ni <= 16)
    hipLaunchKernelGGL((gla_kernel<T, 16>), grid, dim3(256), 0, s, P, R, gla_vec(P));
  else if (ni <= 32)
    hipLaunchKernelGGL((gla_kernel<T, 32>), grid, dim3(256), 0, s, P, R, gla_vec(P));
  else
    hipLaunchKernelGGL((gla_kernel<T, 64>), grid, dim3(256), 0, s, P, R, gla_vec(P));
}
// Heads whose state the registers do not hold: the same walk with the state in memory. Thread j owns column j of the
// state (Dv <= 256 columns), reads and writes it row by row (coalesced over j) and sums its output on the way.
template <typename T>
__global__ __launch_bounds__(256) void gla_general_kernel(GlaParams P, StepRows R, int vec) {
  __shared__ float qs[256], ks[256], as[256], red[4];
  __shared__ float a1s[GLA_MAX_RANK];
  const int r0 = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int seq = R.q_seq[r0];
  if (r0 > 0 && R.q_seq[r0 - 1] == seq) return;  // not the first row of its segment (uniform per block)
  const int D = P.D, Dv = P.Dv;
  float* S0 = P.state + (long long)seq * P.state_stride + (long long)h * D * Dv;
  const float qscale = 1.f / sqrtf((float)D);
  for (int r = r0; r < R.B && R.q_seq[r] == seq; ++r) {
    const float* row = P.proj + (long long)r * P.ld;
    __syncthreads();
    if (tid < P.rank) a1s[tid] = row[P.off_a1 + tid];
    if (tid < D) {
      qs[tid] = row[P.off_q + h * D + tid] * qscale;
      ks[tid] = row[P.off_k + h * D + tid];
    }
    __syncthreads();
    if (tid < D) as[tid] = expf(gla_ln_alpha<T>(P, a1s, h * D + tid, vec));
    __syncthreads();
    float o = 0.f;
    if (tid < Dv) {
      const float vj = row[P.off_v + h * Dv + tid];
      for (int i = 0; i < D; ++i) {
        const float sv = as[i] * S0[(long long)i * Dv + tid] + ks[i] * vj;
        S0[(long long)i * Dv + tid] = sv;
        o += sv * qs[i];
      }
    }
    const float ms = block_sum256(o * o, red) / (float)Dv;
    if (tid < Dv) {
      const float y = o / sqrtf(ms + P.eps) * P.norm_w[tid] * silu(row[P.off_g + h * Dv + tid]);
      st((T*)P.out + (long long)r * P.ld_out + h * Dv + tid, y);
    }
  }
}
bool gla_general_supported(int D, int Dv) { return D > 0 && Dv > 0 && D <= 256 && Dv <= 256; }
static void check_gla(const GlaParams& P, const StepRows& R) {
  check(R.B > 0 && P.proj && P.state && P.out && P.a2 && P.a2_b && P.norm_w && P.H > 0 && P.rank > 0 && P.rank <= GLA_MAX_RANK &&
            P.tau > 0.f &&
            gla_general_supported(P.D, P.Dv),
        "gated linear attention: operands or head sizes (key and value size <= 256)");
}
void gla(const GlaParams& P, const StepRows& R, hipStream_t s) {
  check_gla(P, R);
  if (!gla_supported(P.D, P.Dv)) {
    if (P.f32)
      hipLaunchKernelGGL(gla_general_kernel<float>, dim3(R.B, P.H), dim3(256), 0, s, P, R, gla_vec(P));
    else
      hipLaunchKernelGGL(gla_general_kernel<bf16>, dim3(R.B, P.H), dim3(256), 0, s, P, R, gla_vec(P));
    launched("gla_general");
    return;
  }
  if (P.f32)
    launch_gla<float>(P, R, s);
  else
    launch_gla<bf16>(P, R, s);
  launched("gla");
}

// ---- prompt portions: the same recurrence in chunks of GC tokens over the host-built chunk table
// {first row, rows, state slot, flags}. With l_s = ln alpha_s (a vector over the key channels) and
// L_t = l_0 + ... + l_t inside a chunk of n tokens that starts from state S,
//   A[t][s] = sum_d q_t[d] k_s[d] exp(L_t[d] - L_s[d]) for s <= t,   o_t = S^T (q_t * exp(L_t)) + sum_s A[t][s] v_s,
//   U = sum_s (k_s * exp(L_(n-1) - L_s)) v_s^T,                        S <- diag(exp(L_(n-1))) S + U.
// Every exponent is <= 0, so nothing overflows whatever the decay; all float32 on the vector ALUs.
//   0. gla_lna_kernel: ln alpha of every (row, channel), then its running sum inside each chunk (in place)
//   1. gla_u_kernel: every chunk's U, chunks in parallel
//   2. gla_chunk_scan_kernel: the scan over each sequence's chunks, one thread per state element
//   3. gla_out_kernel: every chunk's outputs from its incoming state, in parallel, with the norm and the gate
constexpr int GC = 32;
constexpr int GLA_CD = 128;  // largest key size of the chunked form
// LDS floats of the output kernel: q, k and the running log decays [GC][D + 1] each, A [GC][GC + 1], v [GC][Dv]
static inline long long gla_out_lds(int D, int Dv) { return 3LL * GC * (D + 1) + GC * (GC + 1) + (long long)GC * Dv; }
bool gla_chunk_supported(int D, int Dv) {
  return D > 0 && D <= GLA_CD && Dv > 0 && Dv <= 256 && gla_out_lds(D, Dv) * 4 <= 64 * 1024;
}
template <typename T>
__global__ __launch_bounds__(256) void gla_lna_kernel(GlaParams P, int B, float* __restrict__ lna, int ld_lna, int vec) {
  __shared__ float a1s[GLA_MAX_RANK];
  const int r = blockIdx.x;
  const float* row = P.proj + (long long)r * P.ld;
  if (threadIdx.x < P.rank) a1s[threadIdx.x] = row[P.off_a1 + threadIdx.x];
  __syncthreads();
  for (int ch = threadIdx.x; ch < P.H * P.D; ch += 256) lna[(long long)r * ld_lna + ch] = gla_ln_alpha<T>(P, a1s, ch, vec);
}
__global__ __launch_bounds__(256) void gla_cum_kernel(const int* __restrict__ chunks, int HD, float* __restrict__ lna,
                                                      int ld_lna) {
  const int r0 = chunks[4 * blockIdx.x], n = chunks[4 * blockIdx.x + 1];
  for (int ch = threadIdx.x; ch < HD; ch += 256) {
    float acc = 0.f;
    for (int t = 0; t < n; ++t) {
      acc += lna[(long long)(r0 + t) * ld_lna + ch];
      lna[(long long)(r0 + t) * ld_lna + ch] = acc;
    }
  }
}
// U[i][j] = sum_s k_s[i] exp(L_end[i] - L_s[i]) v_s[j]: one block per (chunk, head), thread (g, j) as above
__global__ __launch_bounds__(256) void gla_u_kernel(GlaParams P, const int* __restrict__ chunks, const float* __restrict__ lna,
                                                    int ld_lna, float* __restrict__ U, long long u_stride) {
  __shared__ float kd[GC][GLA_CD];
  __shared__ float vs[GC][256];
  const int c = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int r0 = chunks[4 * c], n = chunks[4 * c + 1];
  const int D = P.D, Dv = P.Dv, NG = 256 / Dv;
  for (int i = tid; i < n * D; i += 256) {
    const int t = i / D, d = i % D;
    const float Lend = lna[(long long)(r0 + n - 1) * ld_lna + h * D + d], Lt = lna[(long long)(r0 + t) * ld_lna + h * D + d];
    kd[t][d] = P.proj[(long long)(r0 + t) * P.ld + P.off_k + h * D + d] * expf(Lend - Lt);
  }
  for (int i = tid; i < n * Dv; i += 256)
    vs[i / Dv][i % Dv] = P.proj[(long long)(r0 + i / Dv) * P.ld + P.off_v + h * Dv + i % Dv];
  __syncthreads();
  const int g = tid / Dv, j = tid % Dv;
  if (g >= NG) return;
  float* out = U + (long long)c * u_stride + (long long)h * D * Dv;
  for (int i = g; i < D; i += NG) {
    float acc = 0.f;
    for (int t = 0; t < n; ++t) acc += kd[t][i] * vs[t][j];
    out[(long long)i * Dv + j] = acc;
  }
}
// Sin[c] = the state a chunk starts from; the sequence's state after its last chunk goes back to the slot. One thread
// per state element walks every chunk of the step (a sequence's chunks are consecutive in the table)
__global__ __launch_bounds__(256) void gla_chunk_scan_kernel(GlaParams P, const int* __restrict__ chunks, int nchunks,
                                                             const float* __restrict__ lna, int ld_lna,
                                                             const float* __restrict__ U, float* __restrict__ Sin,
                                                             long long u_stride) {
  const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
  if (e >= (long long)P.H * P.D * P.Dv) return;
  const int hd = (int)(e / P.Dv);  // head * D + key channel
  float S = 0.f;
  for (int c = 0; c < nchunks; ++c) {  // the table's entries are the same for every thread: scalar loads
    const int last = chunks[4 * c] + chunks[4 * c + 1] - 1, slot = chunks[4 * c + 2], flags = chunks[4 * c + 3];
    float* st_e = P.state + (long long)slot * P.state_stride + e;
    if (flags & 1) S = *st_e;
    Sin[c * u_stride + e] = S;
    S = expf(lna[(long long)last * ld_lna + hd]) * S + U[c * u_stride + e];
    if (flags & 2) *st_e = S;
  }
}
// outputs of one chunk and head: A is built in LDS first (the exponentials are per pair and channel)
template <typename T, int RT>  // RT >= ceil(GC / NG): rows of a column that one thread sums
__global__ __launch_bounds__(256) void gla_out_kernel(GlaParams P, const int* __restrict__ chunks, const float* __restrict__ lna,
                                                      int ld_lna, const float* __restrict__ Sin, long long u_stride) {
  extern __shared__ float lds[];
  const int c = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int r0 = chunks[4 * c], n = chunks[4 * c + 1];
  const int D = P.D, Dv = P.Dv, NG = 256 / Dv, D1 = D + 1;
  float* qd = lds;                 // [GC][D + 1]
  float* kk = qd + GC * D1;        // [GC][D + 1]
  float* Lc = kk + GC * D1;        // [GC][D + 1]
  float* A = Lc + GC * D1;         // [GC][GC + 1]
  float* vs = A + GC * (GC + 1);   // [GC][Dv]
  const float qscale = 1.f / sqrtf((float)D);
  for (int i = tid; i < n * D; i += 256) {
    const int t = i / D, d = i % D;
    const float* row = P.proj + (long long)(r0 + t) * P.ld;
    qd[t * D1 + d] = row[P.off_q + h * D + d] * qscale;
    kk[t * D1 + d] = row[P.off_k + h * D + d];
    Lc[t * D1 + d] = lna[(long long)(r0 + t) * ld_lna + h * D + d];
  }
  for (int i = tid; i < n * Dv; i += 256) vs[i] = P.proj[(long long)(r0 + i / Dv) * P.ld + P.off_v + h * Dv + i % Dv];
  __syncthreads();
  for (int p = tid; p < GC * GC; p += 256) {  // A[t][s], s <= t < n; zero elsewhere
    const int t = p / GC, sidx = p % GC;
    float acc = 0.f;
    if (sidx <= t && t < n)
      for (int d = 0; d < D; ++d)  // exponents <= 0; exp2 on the transcendental unit (1 ulp)
        acc += qd[t * D1 + d] * kk[sidx * D1 + d] * __builtin_amdgcn_exp2f((Lc[t * D1 + d] - Lc[sidx * D1 + d]) * 1.44269504088896341f);
    A[t * (GC + 1) + sidx] = acc;
  }
  __syncthreads();
  for (int i = tid; i < n * D; i += 256) {  // q_t * exp(L_t) meets the incoming state
    const int t = i / D, d = i % D;
    qd[t * D1 + d] *= expf(Lc[t * D1 + d]);
  }
  __syncthreads();
  // O = (Q * exp(L)) S + A V: thread (g, j) owns column j of rows t = g, g + NG, ... (up to GC / NG of them) and sums
  // them whole, the state's column read once per key channel; the rows then meet in LDS for their norms
  const int g = tid / Dv, j = tid % Dv;
  const float* S = Sin + (long long)c * u_stride + (long long)h * D * Dv;
  float acc[RT];
#pragma unroll
  for (int k = 0; k < RT; ++k) acc[k] = 0.f;
  if (g < NG) {
    for (int i0 = 0; i0 < D; i0 += 8) {  // eight loads of the state's column in flight at a time
      float sv[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) sv[u] = i0 + u < D ? S[(long long)(i0 + u) * Dv + j] : 0.f;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (i0 + u < D) {
#pragma unroll
          for (int k = 0; k < RT; ++k) {
            const int t = min(g + k * NG, GC - 1);  // rows past the chunk's end: computed, never stored
            acc[k] += sv[u] * qd[t * D1 + i0 + u];
          }
        }
      }
    }
    for (int sidx = 0; sidx < n; ++sidx) {
      const float vv = vs[sidx * Dv + j];
#pragma unroll
      for (int k = 0; k < RT; ++k) {
        const int t = min(g + k * NG, GC - 1);
        acc[k] += A[t * (GC + 1) + sidx] * vv;  // A is zero above the diagonal and in rows past the chunk's end
      }
    }
  }
  __syncthreads();  // every thread is done with vs: the rows' outputs take its place
  float* ob = vs;   // [GC][Dv]
  if (g < NG) {
#pragma unroll
    for (int k = 0; k < RT; ++k) {
      const int t = g + k * NG;
      if (t < n) ob[t * Dv + j] = acc[k];
    }
  }
  __syncthreads();
  const int lane = tid & 63, wv = tid >> 6;
  for (int t = wv; t < n; t += 4) {  // a wave per row: the head's RMS norm, its weight, the gate
    float ss = 0.f;
    for (int d = lane; d < Dv; d += 64) ss += ob[t * Dv + d] * ob[t * Dv + d];
    const float inv = 1.f / sqrtf(wave_sum(ss) / (float)Dv + P.eps);
    for (int d = lane; d < Dv; d += 64) {
      const float y = ob[t * Dv + d] * inv * P.norm_w[d] * silu(P.proj[(long long)(r0 + t) * P.ld + P.off_g + h * Dv + d]);
      st((T*)P.out + (long long)(r0 + t) * P.ld_out + h * Dv + d, y);
    }
  }
}
void gla_chunked(const GlaParams& P, const StepRows& R, const GlaChunkWs& W, hipStream_t s) {
  check_gla(P, R);
  check(gla_chunk_supported(P.D, P.Dv) && W.chunks && W.nchunks > 0 && W.nchunks <= W.max_chunks && W.U && W.Sin && W.lna &&
            W.ld_lna >= P.H * P.D && W.u_stride >= (long long)P.H * P.D * P.Dv,
        "chunked gated linear attention: operands");
  const int HD = P.H * P.D;
  const long long per = (long long)HD * P.Dv;
  const dim3 cg(W.nchunks, P.H);
  if (P.f32)
    hipLaunchKernelGGL(gla_lna_kernel<float>, dim3(R.B), dim3(256), 0, s, P, R.B, W.lna, W.ld_lna, gla_vec(P));
  else
    hipLaunchKernelGGL(gla_lna_kernel<bf16>, dim3(R.B), dim3(256), 0, s, P, R.B, W.lna, W.ld_lna, gla_vec(P));
  hipLaunchKernelGGL(gla_cum_kernel, dim3(W.nchunks), dim3(256), 0, s, W.chunks, HD, W.lna, W.ld_lna);
  hipLaunchKernelGGL(gla_u_kernel, cg, dim3(256), 0, s, P, W.chunks, W.lna, W.ld_lna, W.U, W.u_stride);
  hipLaunchKernelGGL(gla_chunk_scan_kernel, dim3((unsigned)((per + 255) / 256)), dim3(256), 0, s, P, W.chunks,
                     W.nchunks, W.lna, W.ld_lna, W.U, W.Sin, W.u_stride);
  const size_t lds = (size_t)gla_out_lds(P.D, P.Dv) * sizeof(float);
  const int ng = 256 / P.Dv, rt = (GC + ng - 1) / ng;
#define GLA_OUT(TT, RT) hipLaunchKernelGGL((gla_out_kernel<TT, RT>), cg, dim3(256), lds, s, P, W.chunks, W.lna, W.ld_lna, W.Sin, W.u_stride)
  if (P.f32) {
    if (rt <= 8) GLA_OUT(float, 8); else if (rt <= 16) GLA_OUT(float, 16); else GLA_OUT(float, 32);
  } else {
    if (rt <= 8) GLA_OUT(bf16, 8); else if (rt <= 16) GLA_OUT(bf16, 16); else GLA_OUT(bf16, 32);
  }
#undef GLA_OUT
  launched("gla_chunked");
}

// ------------------------------------------------------------------------------------------------ norm + scale + residual
// v = sa * (y + bias) + sb * y2; x += ls * (v / rms(v) * g). With g_next the updated row also leaves normed in the
// matrix dtype. The row is read again for every pass: it is a few kilobytes and stays in the cache.
template <typename T>
__global__ __launch_bounds__(256) void sandwich_add_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                           const float* __restrict__ bias, float sa,
                                                           const float* __restrict__ y2, float sb, int E,
                                                           const float* __restrict__ g, const float* __restrict__ ls, float eps,
                                                           const float* __restrict__ g_next, T* __restrict__ hout) {
  __shared__ float red[4];
  const long long r = blockIdx.x;
  float* xr = x + r * E;
  const float* yr = y + r * E;
  const float* zr = y2 ? y2 + r * E : nullptr;
  auto val = [&](int i) { return sa * (yr[i] + (bias ? bias[i] : 0.f)) + (zr ? sb * zr[i] : 0.f); };
  float ss = 0.f;
  for (int i = threadIdx.x; i < E; i += 256) {
    const float v = val(i);
    ss += v * v;
  }
  const float scale = g[0] / sqrtf(block_sum256(ss, red) / (float)E + eps);
  float s2 = 0.f;
  for (int i = threadIdx.x; i < E; i += 256) {
    const float o = xr[i] + ls[i] * (val(i) * scale);
    xr[i] = o;
    s2 += o * o;
  }
  if (!hout) return;
  const float sn = g_next[0] / sqrtf(block_sum256(s2, red) / (float)E + eps);
  for (int i = threadIdx.x; i < E; i += 256) st(hout + r * E + i, xr[i] * sn);
}
// the same with the row held in registers (widths up to 256 * SW_REG): x, y and y2 are read once
constexpr int SW_REG = 16;
template <typename T>
__global__ __launch_bounds__(256) void sandwich_add_reg_kernel(float* __restrict__ x, const float* __restrict__ y,
                                                               const float* __restrict__ bias, float sa,
                                                               const float* __restrict__ y2, float sb, int E,
                                                               const float* __restrict__ g, const float* __restrict__ ls,
                                                               float eps, const float* __restrict__ g_next, T* __restrict__ hout) {
  __shared__ float red[4];
  const long long r = blockIdx.x;
  float* xr = x + r * E;
  const float* yr = y + r * E;
  const float* zr = y2 ? y2 + r * E : nullptr;
  float v[SW_REG], xv[SW_REG], lv[SW_REG];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < SW_REG; ++k) {
    const int i = threadIdx.x + 256 * k;
    v[k] = xv[k] = lv[k] = 0.f;
    if (i < E) {
      v[k] = sa * (yr[i] + (bias ? bias[i] : 0.f)) + (zr ? sb * zr[i] : 0.f);
      xv[k] = xr[i];
      lv[k] = ls[i];
    }
    ss += v[k] * v[k];
  }
  const float scale = g[0] / sqrtf(block_sum256(ss, red) / (float)E + eps);
  float s2 = 0.f;
#pragma unroll
  for (int k = 0; k < SW_REG; ++k) {
    const int i = threadIdx.x + 256 * k;
    xv[k] = xv[k] + lv[k] * (v[k] * scale);
    if (i < E) xr[i] = xv[k];
    s2 += xv[k] * xv[k];
  }
  if (!hout) return;
  const float sn = g_next[0] / sqrtf(block_sum256(s2, red) / (float)E + eps);
#pragma unroll
  for (int k = 0; k < SW_REG; ++k) {
    const int i = threadIdx.x + 256 * k;
    if (i < E) st(hout + r * E + i, xv[k] * sn);
  }
}
void sandwich_add(float* x, const float* y, const float* bias, float sa, const float* y2, float sb, int rows, int E,
                  const float* g, const float* ls, float eps, const float* g_next, void* hout, int f32, hipStream_t s) {
  check(rows > 0 && E > 0 && x && y && g && ls && (!hout || g_next), "sandwich_add: bad operands");
  if (E <= 256 * SW_REG) {
    if (f32)
      hipLaunchKernelGGL(sandwich_add_reg_kernel<float>, dim3(rows), dim3(256), 0, s, x, y, bias, sa, y2, sb, E, g, ls, eps,
                         g_next, (float*)hout);
    else
      hipLaunchKernelGGL(sandwich_add_reg_kernel<bf16>, dim3(rows), dim3(256), 0, s, x, y, bias, sa, y2, sb, E, g, ls, eps,
                         g_next, (bf16*)hout);
    launched("sandwich_add");
    return;
  }
  if (f32)
    hipLaunchKernelGGL(sandwich_add_kernel<float>, dim3(rows), dim3(256), 0, s, x, y, bias, sa, y2, sb, E, g, ls, eps, g_next,
                       (float*)hout);
  else
    hipLaunchKernelGGL(sandwich_add_kernel<bf16>, dim3(rows), dim3(256), 0, s, x, y, bias, sa, y2, sb, E, g, ls, eps, g_next,
                       (bf16*)hout);
  launched("sandwich_add");
}

// ------------------------------------------------------------------------------------------------ two output projections
// C[m][n] = sa * (A1[m] . W1[n] + bias[n]) + sb * (A2[m] . W2[n]) for a few rows (decode steps): one wave per output,
// both weight rows streamed once per activation row.
template <typename T>
__global__ __launch_bounds__(256) void gemv_pair_kernel(const T* __restrict__ A1, int lda1, const T* __restrict__ W1, int K1,
                                                        const float* __restrict__ bias, float sa, const T* __restrict__ A2,
                                                        int lda2, const T* __restrict__ W2, int K2, float sb, int M, int N,
                                                        float* __restrict__ C, int ldc, int v1, int v2) {
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= N) return;
  const float b = bias ? bias[n] : 0.f;
  for (int m = 0; m < M; ++m) {
    const float d1 = wave_dot<T>(W1 + (long long)n * K1, A1 + (long long)m * lda1, K1, lane, v1);
    const float d2 = wave_dot<T>(W2 + (long long)n * K2, A2 + (long long)m * lda2, K2, lane, v2);
    if (lane == 0) C[(long long)m * ldc + n] = sa * (d1 + b) + sb * d2;
  }
}
void gemv_pair(const void* A1, int lda1, const void* W1, int K1, const float* bias, float sa, const void* A2, int lda2,
               const void* W2, int K2, float sb, int M, int N, float* C, int ldc, int f32, hipStream_t s) {
  check(M > 0 && M <= 8 && N > 0 && K1 > 0 && K2 > 0 && A1 && W1 && A2 && W2 && C && lda1 >= K1 && lda2 >= K2 && ldc >= N,
        "gemv_pair: bad operands (at most 8 rows)");
  const dim3 grid((N + 3) / 4);
  if (f32)
    hipLaunchKernelGGL(gemv_pair_kernel<float>, grid, dim3(256), 0, s, (const float*)A1, lda1, (const float*)W1, K1, bias, sa,
                       (const float*)A2, lda2, (const float*)W2, K2, sb, M, N, C, ldc,
                       (int)(vec_ok<float>(A1, lda1, K1) && vec_ok<float>(W1, K1, K1)),
                       (int)(vec_ok<float>(A2, lda2, K2) && vec_ok<float>(W2, K2, K2)));
  else
    hipLaunchKernelGGL(gemv_pair_kernel<bf16>, grid, dim3(256), 0, s, (const bf16*)A1, lda1, (const bf16*)W1, K1, bias, sa,
                       (const bf16*)A2, lda2, (const bf16*)W2, K2, sb, M, N, C, ldc,
                       (int)(vec_ok<bf16>(A1, lda1, K1) && vec_ok<bf16>(W1, K1, K1)),
                       (int)(vec_ok<bf16>(A2, lda2, K2) && vec_ok<bf16>(W2, K2, K2)));
  launched("gemv_pair");
}

// ------------------------------------------------------------------------------------------------ gate / up projection + activation
// out[m][k] = gelu_tanh(A[m] . W[k]) * (A[m] . W[F + k]) for a few rows (decode steps): one wave per hidden unit takes
// its gate row and its up row, so the activation leaves with the product and needs no launch of its own.
__device__ __forceinline__ float geglu_tanh(float a, float u) {
  const float t = tanhf(0.7978845608028654f * (a + 0.044715f * a * a * a));
  return 0.5f * a * (1.f + t) * u;
}
template <typename T>
__global__ __launch_bounds__(256) void gemv_glu_kernel(const T* __restrict__ A, int lda, const T* __restrict__ W, int K, int F,
                                                       int M, T* __restrict__ out, int ld_out, int vec) {
  const int lane = threadIdx.x & 63;
  const int k = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (k >= F) return;
  for (int m = 0; m < M; ++m) {
    const float g = wave_dot<T>(W + (long long)k * K, A + (long long)m * lda, K, lane, vec);
    const float u = wave_dot<T>(W + (long long)(F + k) * K, A + (long long)m * lda, K, lane, vec);
    if (lane == 0) st(out + (long long)m * ld_out + k, geglu_tanh(g, u));
  }
}
void gemv_glu(const void* A, int lda, const void* W, int K, int F, int M, void* out, int ld_out, int f32, hipStream_t s) {
  check(M > 0 && M <= 8 && K > 0 && F > 0 && A && W && out && lda >= K && ld_out >= F, "gemv_glu: bad operands (at most 8 rows)");
  const dim3 grid((F + 3) / 4);
  if (f32)
    hipLaunchKernelGGL(gemv_glu_kernel<float>, grid, dim3(256), 0, s, (const float*)A, lda, (const float*)W, K, F, M, (float*)out,
                       ld_out, (int)(vec_ok<float>(A, lda, K) && vec_ok<float>(W, K, K)));
  else
    hipLaunchKernelGGL(gemv_glu_kernel<bf16>, grid, dim3(256), 0, s, (const bf16*)A, lda, (const bf16*)W, K, F, M, (bf16*)out,
                       ld_out, (int)(vec_ok<bf16>(A, lda, K) && vec_ok<bf16>(W, K, K)));
  launched("gemv_glu");
}

// ------------------------------------------------------------------------------------------------ gated activation
template <typename T>
__global__ __launch_bounds__(256) void geglu_tanh_kernel(const float* __restrict__ z, int ld, int rows, int F,
                                                         T* __restrict__ out, int ld_out) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long long)rows * F) return;
  const long long r = i / F;
  const int c = (int)(i % F);
  st(out + r * ld_out + c, geglu_tanh(z[r * ld + c], z[r * ld + F + c]));
}
void geglu_tanh_cast(const float* z, int ld, int rows, int F, void* out, int ld_out, int f32, hipStream_t s) {
  check(rows > 0 && F > 0 && z && out && ld >= 2 * F && ld_out >= F, "geglu_tanh_cast: bad operands");
  const dim3 grid((unsigned)(((long long)rows * F + 255) / 256));
  if (f32)
    hipLaunchKernelGGL(geglu_tanh_kernel<float>, grid, dim3(256), 0, s, z, ld, rows, F, (float*)out, ld_out);
  else
    hipLaunchKernelGGL(geglu_tanh_kernel<bf16>, grid, dim3(256), 0, s, z, ld, rows, F, (bf16*)out, ld_out);
  launched("geglu_tanh_cast");
}

}  // namespace stack
}  // namespace omx
