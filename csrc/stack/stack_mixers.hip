// gfx950 kernels of the layers whose norm sits on the sublayer's output (interface: stack_ops.h): the cast of
// the stream into the matrix dtype, the post-norm residual update, latent attention's cache row / folded
// queries / value expansion, the short causal convolution with its carried inputs, the gated state scan that
// serves the mLSTM matrix memory and the Mamba-2 state space layer, the grouped RMS norm of their outputs,
// the dense feed-forward's activation and the score router with expert groups and identity experts.
// Everything but the matrix operands and the cached latent is float32. Wave = 64 lanes.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>

#include "stack_device.h"
#include "stack_ops.h"

namespace omx {
namespace stack {

// ------------------------------------------------------------------------------------------------ cast
template <typename T>
__global__ __launch_bounds__(256) void cast_rows_kernel(const float* __restrict__ x, long long n, T* __restrict__ out) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) st(out + i, x[i]);
}
void cast_rows(const float* x, int rows, int E, void* out, int f32, hipStream_t s) {
  check(rows > 0 && E > 0 && x && out, "cast_rows: bad operands");
  const long long n = (long long)rows * E;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (f32)
    hipLaunchKernelGGL(cast_rows_kernel<float>, grid, dim3(256), 0, s, x, n, (float*)out);
  else
    hipLaunchKernelGGL(cast_rows_kernel<bf16>, grid, dim3(256), 0, s, x, n, (bf16*)out);
  launched("cast_rows");
}

// ------------------------------------------------------------------------------------------------ post-norm residual
// x[r] += layer_norm(y[r] + (idw ? idw[r] * x[r] : 0)) * w + b; the variance is the mean of the squared deviations.
// With hout the updated row also leaves in the matrix dtype (the next sublayer's operand).
template <typename T>
__global__ __launch_bounds__(256) void post_norm_add_kernel(float* __restrict__ x, const float* __restrict__ y, int E,
                                                            const float* __restrict__ w, const float* __restrict__ b,
                                                            float eps, const float* __restrict__ idw, T* __restrict__ hout) {
  __shared__ float red[4];
  const long long r = blockIdx.x;
  float* xr = x + r * E;
  const float* yr = y + r * E;
  const float iw = idw ? idw[r] : 0.f;
  float sum = 0.f;
  for (int i = threadIdx.x; i < E; i += 256) sum += yr[i] + iw * xr[i];
  const float mean = block_sum256(sum, red) / (float)E;
  float sq = 0.f;
  for (int i = threadIdx.x; i < E; i += 256) {
    const float d = yr[i] + iw * xr[i] - mean;
    sq += d * d;
  }
  const float inv = 1.f / sqrtf(block_sum256(sq, red) / (float)E + eps);
  for (int i = threadIdx.x; i < E; i += 256) {
    const float v = xr[i] + ((yr[i] + iw * xr[i] - mean) * inv * w[i] + b[i]);
    xr[i] = v;
    if (hout) st(hout + r * E + i, v);
  }
}
// the same with the row held in registers (widths up to 256 * PN_REG): x and y are read once
constexpr int PN_REG = 16;
template <typename T>
__global__ __launch_bounds__(256) void post_norm_add_reg_kernel(float* __restrict__ x, const float* __restrict__ y, int E,
                                                                const float* __restrict__ w, const float* __restrict__ b,
                                                                float eps, const float* __restrict__ idw, T* __restrict__ hout) {
  __shared__ float red[4];
  const long long r = blockIdx.x;
  float* xr = x + r * E;
  const float* yr = y + r * E;
  const float iw = idw ? idw[r] : 0.f;
  float xv[PN_REG], v[PN_REG];
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < PN_REG; ++k) {
    const int i = threadIdx.x + 256 * k;
    xv[k] = i < E ? xr[i] : 0.f;
    v[k] = i < E ? yr[i] + iw * xv[k] : 0.f;
    sum += v[k];
  }
  const float mean = block_sum256(sum, red) / (float)E;
  float sq = 0.f;
#pragma unroll
  for (int k = 0; k < PN_REG; ++k) {
    const float d = threadIdx.x + 256 * k < E ? v[k] - mean : 0.f;
    sq += d * d;
  }
  const float inv = 1.f / sqrtf(block_sum256(sq, red) / (float)E + eps);
#pragma unroll
  for (int k = 0; k < PN_REG; ++k) {
    const int i = threadIdx.x + 256 * k;
    if (i < E) {
      const float o = xv[k] + ((v[k] - mean) * inv * w[i] + b[i]);
      xr[i] = o;
      if (hout) st(hout + r * E + i, o);
    }
  }
}
void post_norm_add(float* x, const float* y, int rows, int E, const float* w, const float* b, float eps, const float* idw,
                   void* hout, int f32, hipStream_t s) {
  check(rows > 0 && E > 0 && x && y && w && b, "post_norm_add: bad operands");
  if (E <= 256 * PN_REG) {
    if (f32)
      hipLaunchKernelGGL(post_norm_add_reg_kernel<float>, dim3(rows), dim3(256), 0, s, x, y, E, w, b, eps, idw, (float*)hout);
    else
      hipLaunchKernelGGL(post_norm_add_reg_kernel<bf16>, dim3(rows), dim3(256), 0, s, x, y, E, w, b, eps, idw, (bf16*)hout);
    launched("post_norm_add");
    return;
  }
  if (f32)
    hipLaunchKernelGGL(post_norm_add_kernel<float>, dim3(rows), dim3(256), 0, s, x, y, E, w, b, eps, idw, (float*)hout);
  else
    hipLaunchKernelGGL(post_norm_add_kernel<bf16>, dim3(rows), dim3(256), 0, s, x, y, E, w, b, eps, idw, (bf16*)hout);
  launched("post_norm_add");
}

// ------------------------------------------------------------------------------------------------ latent attention
// Keys and values of every head are linear maps of one latent c per token, so attention runs in latent space:
//   score_h(t, s) = (W_uk_h^T q_plain_h(t)) . c(s) + q_rot_h(t) . k_rot(s),   o_h(t) = W_uv_h sum_s p_h(t, s) c(s).
// The cached row of a token is [c | k_rot] (one row serves all heads, and its first C elements are the value).
// latent_prepare: grid (row groups of LAT_RB, H + 1). Blocks y < H fold LAT_RB queries of head y onto the latent
// (thread r owns output r: W_uk is read along its contiguous axis) and rotate their rotated part; blocks y == H
// write the rows' cache entries: c = rms_norm(first C outputs) * w, the last R outputs rotated.
// Rotation: dims (2i, 2i + 1), i < rot_dims / 2, turn by pos * inv_freq[i]; the angle and its sine / cosine are
// computed in float64 (a float32 angle at position 10^3 is already off by 10^-4).
constexpr int LAT_RB = 8;
constexpr int LAT_MAXD = 256, LAT_MAXC = 512;
__device__ __forceinline__ float rotate_pair_elem(const float* v, int j, int rot_dims, int pos, const double* inv_freq) {
  if (j >= rot_dims) return v[j];
  const double ang = (double)pos * inv_freq[j >> 1];
  const float c = (float)cos(ang), sn = (float)sin(ang);
  const float a = v[j & ~1], b = v[j | 1];
  return (j & 1) ? b * c + a * sn : a * c - b * sn;
}
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_kernel(LatentParams P, StepRows R) {
  __shared__ float qs[LAT_RB][LAT_MAXD];
  __shared__ float red[4];
  const int r0 = blockIdx.x * LAT_RB, h = blockIdx.y, tid = threadIdx.x;
  const int nr = min(LAT_RB, R.B - r0);
  const int C = P.C, Rr = P.R, D = P.D, W = C + Rr;
  if (h == P.H) {  // the rows' cache entries
    T* cache = (T*)P.cache;
    for (int i = 0; i < nr; ++i) {
      const int b = r0 + i;
      const float* dkv = P.proj + (long long)b * P.ld + P.off_k;
      float sq = 0.f;
      for (int c = tid; c < C; c += 256) sq += dkv[c] * dkv[c];
      const float inv = 1.f / sqrtf(block_sum256(sq, red) / (float)C + P.eps);
      T* dst = cache + (long long)R.slot[b] * W;
      for (int c = tid; c < C; c += 256) st(dst + c, dkv[c] * inv * P.norm_w[c]);
      for (int j = tid; j < Rr; j += 256) st(dst + C + j, rotate_pair_elem(dkv + C, j, P.rot_dims, R.pos[b], P.inv_freq));
    }
    return;
  }
  for (int idx = tid; idx < nr * D; idx += 256) {
    const int i = idx / D, d = idx % D;
    qs[i][d] = P.proj[(long long)(r0 + i) * P.ld + P.off_q + h * (D + Rr) + d];
  }
  __syncthreads();
  const T* wk = (const T*)P.w_uk + (long long)h * D * C;
  for (int c = tid; c < C; c += 256) {
    float acc[LAT_RB];
#pragma unroll
    for (int i = 0; i < LAT_RB; ++i) acc[i] = 0.f;
    for (int d = 0; d < D; ++d) {
      const float wv = ld(wk + (long long)d * C + c);
#pragma unroll
      for (int i = 0; i < LAT_RB; ++i) acc[i] += qs[i][d] * wv;
    }
#pragma unroll
    for (int i = 0; i < LAT_RB; ++i)
      if (i < nr) P.qa[(long long)(r0 + i) * P.ld_qa + h * W + c] = acc[i];
  }
  for (int idx = tid; idx < nr * Rr; idx += 256) {
    const int i = idx / Rr, j = idx % Rr, b = r0 + i;
    const float* qr = P.proj + (long long)b * P.ld + P.off_q + h * (D + Rr) + D;
    P.qa[(long long)b * P.ld_qa + h * W + C + j] = rotate_pair_elem(qr, j, P.rot_dims, R.pos[b], P.inv_freq);
  }
}
// out[b][h * Dv + j] = (sum_c W_uvT[h][c][j] lat[b][h * C + c]) * sigmoid(g[b][h * Dv + j]); grid (row groups, H,
// tiles of 64 columns). Thread (cg, jj) = (tid / 64, tid % 64) sums a quarter of the latent axis for column jj of the
// tile (W_uvT is read along its contiguous axis); the four quarters meet in LDS.
template <typename T>
__global__ __launch_bounds__(256) void latent_expand_kernel(LatentParams P, int B) {
  __shared__ float ls[LAT_RB][LAT_MAXC];
  __shared__ float part[4][LAT_RB][64];
  const int r0 = blockIdx.x * LAT_RB, h = blockIdx.y, tid = threadIdx.x;
  const int nr = min(LAT_RB, B - r0);
  const int C = P.C, Dv = P.Dv;
  for (int idx = tid; idx < nr * C; idx += 256) {
    const int i = idx / C, c = idx % C;
    ls[i][c] = ld((const T*)P.lat + (long long)(r0 + i) * P.ld_lat + h * C + c);
  }
  for (int idx = tid; idx < (LAT_RB - nr) * C; idx += 256) ls[nr + idx / C][idx % C] = 0.f;
  __syncthreads();
  const int cg = tid >> 6, jj = tid & 63, j = blockIdx.z * 64 + jj;
  const int per = (C + 3) / 4, c0 = cg * per, c1 = min(C, c0 + per);
  const T* wv = (const T*)P.w_uvT + (long long)h * C * Dv;
  float acc[LAT_RB];
#pragma unroll
  for (int i = 0; i < LAT_RB; ++i) acc[i] = 0.f;
  if (j < Dv) {
#pragma unroll 8
    for (int c = c0; c < c1; ++c) {
      const float w = ld(wv + (long long)c * Dv + j);
#pragma unroll
      for (int i = 0; i < LAT_RB; ++i) acc[i] += ls[i][c] * w;
    }
  }
#pragma unroll
  for (int i = 0; i < LAT_RB; ++i) part[cg][i][jj] = acc[i];
  __syncthreads();
  for (int idx = tid; idx < nr * 64; idx += 256) {
    const int i = idx >> 6, col = blockIdx.z * 64 + (idx & 63);
    if (col < Dv) {
      const float o = part[0][i][idx & 63] + part[1][i][idx & 63] + part[2][i][idx & 63] + part[3][i][idx & 63];
      const float g = P.proj[(long long)(r0 + i) * P.ld + P.off_g + (P.gate_heads ? h : h * Dv + col)];
      st((T*)P.out + (long long)(r0 + i) * P.ld_out + h * Dv + col, o * sigmoidf(g));
    }
  }
}
// ---- decode steps (a few rows): the fold and the expansion as wave-per-output-row products, so every weight row is
// one 16-byte load per lane and all of them are in flight at once (the row-group kernels above walk a weight column
// with dependent 2-byte loads: fine when 8 rows share them from cache, slow when one row streams them from memory).
// They read the other layouts of the two matrices: W_uk transposed per head [H][C][D], W_uv as stored [H * Dv][C].
template <typename T>
__device__ __forceinline__ float wave_dot_f32x(const T* __restrict__ w, const float* __restrict__ x, int K, int lane, bool vec) {
  float acc = 0.f;
  if (vec) {
    for (int k = lane * 8; k < K; k += 512) {
      float w8[8];
      if constexpr (sizeof(T) == 2) {
        const u32x4 a = *(const u32x4*)(w + k);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          w8[2 * i] = __uint_as_float(a[i] << 16);
          w8[2 * i + 1] = __uint_as_float(a[i] & 0xffff0000u);
        }
      } else {
        const f32x4 a = *(const f32x4*)(w + k), b = *(const f32x4*)(w + k + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          w8[i] = a[i];
          w8[4 + i] = b[i];
        }
      }
      const f32x4 xa = *(const f32x4*)(x + k), xb = *(const f32x4*)(x + k + 4);
      acc += w8[0] * xa[0] + w8[1] * xa[1] + w8[2] * xa[2] + w8[3] * xa[3] + w8[4] * xb[0] + w8[5] * xb[1] + w8[6] * xb[2] +
             w8[7] * xb[3];
    }
  } else {
    for (int k = lane; k < K; k += 64) acc += ld(w + k) * x[k];
  }
  return wave_sum(acc);
}
// blocks [0, nfold): wave (h, c) -> qa[b][h * W + c] = W_ukT[h][c][:] . q_plain_h(b) for every row b;
// blocks nfold + b: row b's cache entry and the rotated parts of its queries
template <typename T>
__global__ __launch_bounds__(256) void latent_prepare_small_kernel(LatentParams P, StepRows R, int nfold, int vec) {
  __shared__ float red[4];
  const int tid = threadIdx.x, lane = tid & 63;
  const int C = P.C, Rr = P.R, D = P.D, W = C + Rr;
  if ((int)blockIdx.x < nfold) {
    const int item = blockIdx.x * 4 + (tid >> 6);
    if (item >= P.H * C) return;
    const int h = item / C, c = item % C;
    const T* w = (const T*)P.w_ukT + (long long)item * D;
    for (int b = 0; b < R.B; ++b) {
      const float v = wave_dot_f32x<T>(w, P.proj + (long long)b * P.ld + P.off_q + h * (D + Rr), D, lane, vec != 0);
      if (lane == 0) P.qa[(long long)b * P.ld_qa + h * W + c] = v;
    }
    return;
  }
  const int b = blockIdx.x - nfold;
  const float* dkv = P.proj + (long long)b * P.ld + P.off_k;
  float sq = 0.f;
  for (int c = tid; c < C; c += 256) sq += dkv[c] * dkv[c];
  const float inv = 1.f / sqrtf(block_sum256(sq, red) / (float)C + P.eps);
  T* dst = (T*)P.cache + (long long)R.slot[b] * W;
  for (int c = tid; c < C; c += 256) st(dst + c, dkv[c] * inv * P.norm_w[c]);
  for (int j = tid; j < Rr; j += 256) st(dst + C + j, rotate_pair_elem(dkv + C, j, P.rot_dims, R.pos[b], P.inv_freq));
  for (int idx = tid; idx < P.H * Rr; idx += 256) {
    const int h = idx / Rr, j = idx % Rr;
    const float* qr = P.proj + (long long)b * P.ld + P.off_q + h * (D + Rr) + D;
    P.qa[(long long)b * P.ld_qa + h * W + C + j] = rotate_pair_elem(qr, j, P.rot_dims, R.pos[b], P.inv_freq);
  }
}
// wave (h, j) -> out[b][h * Dv + j] = (W_uv[h * Dv + j][:] . lat[b][h * C :]) * sigmoid(g[b][h * Dv + j]) for every row b
template <typename T>
__global__ __launch_bounds__(256) void latent_expand_small_kernel(LatentParams P, int B, int vec) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= P.H * P.Dv) return;
  const int h = item / P.Dv;
  const T* w = (const T*)P.w_uv + (long long)item * P.C;
  for (int b = 0; b < B; ++b) {
    const float v = wave_dot<T>(w, (const T*)P.lat + (long long)b * P.ld_lat + h * P.C, P.C, lane, vec != 0);
    if (lane == 0)
      st((T*)P.out + (long long)b * P.ld_out + item, v * sigmoidf(P.proj[(long long)b * P.ld + P.off_g + (P.gate_heads ? h : item)]));
  }
}
bool latent_supported(int D, int R, int C, int Dv) {
  // the latent is the attention's value (up to 256 wide); the cached row [latent | rotated part] is its key: up to 256 on
  // every attention kernel, up to 1024 on the block-per-(row, head) kernel alone
  return D > 0 && D <= LAT_MAXD && R >= 0 && C > 0 && C <= 256 && Dv > 0 && C + R <= 1024;
}
static void check_latent(const LatentParams& P) {
  check(P.proj && P.cache && P.qa && P.lat && P.out && P.w_uk && P.w_uvT && P.norm_w &&
            latent_supported(P.D, P.R, P.C, P.Dv) && P.rot_dims % 2 == 0 && P.rot_dims <= P.R && (P.rot_dims == 0 || P.inv_freq),
        "latent attention: operands or sizes (dim <= 256, kv_rank <= 256, kv_rank + rot_dim <= 1024)");
}
constexpr int LAT_SMALL = 8;  // steps of at most this many rows take the wave-per-output kernels
void latent_prepare(const LatentParams& P, const StepRows& R, hipStream_t s) {
  check_latent(P);
  if (R.B <= LAT_SMALL && P.w_ukT) {
    const int nfold = (P.H * P.C + 3) / 4;
    const int per = P.f32 ? 4 : 8;
    const int vec = P.D % 8 == 0 && (P.D + P.R) % 4 == 0 && P.off_q % 4 == 0 && P.ld % 4 == 0 && ((uintptr_t)P.proj & 15) == 0 &&
                    ((uintptr_t)P.w_ukT & 15) == 0 && P.D % per == 0;
    if (P.f32)
      hipLaunchKernelGGL(latent_prepare_small_kernel<float>, dim3(nfold + R.B), dim3(256), 0, s, P, R, nfold, vec);
    else
      hipLaunchKernelGGL(latent_prepare_small_kernel<bf16>, dim3(nfold + R.B), dim3(256), 0, s, P, R, nfold, vec);
    launched("latent_prepare_small");
    return;
  }
  const dim3 grid((R.B + LAT_RB - 1) / LAT_RB, P.H + 1);
  if (P.f32)
    hipLaunchKernelGGL(latent_prepare_kernel<float>, grid, dim3(256), 0, s, P, R);
  else
    hipLaunchKernelGGL(latent_prepare_kernel<bf16>, grid, dim3(256), 0, s, P, R);
  launched("latent_prepare");
}
void latent_expand(const LatentParams& P, int B, hipStream_t s) {
  check_latent(P);
  if (B <= LAT_SMALL && P.w_uv) {
    const dim3 grid((P.H * P.Dv + 3) / 4);
    if (P.f32) {
      const int vec = vec_ok<float>(P.w_uv, P.C, P.C) && vec_ok<float>(P.lat, P.ld_lat, P.C);
      hipLaunchKernelGGL(latent_expand_small_kernel<float>, grid, dim3(256), 0, s, P, B, vec);
    } else {
      const int vec = vec_ok<bf16>(P.w_uv, P.C, P.C) && vec_ok<bf16>(P.lat, P.ld_lat, P.C);
      hipLaunchKernelGGL(latent_expand_small_kernel<bf16>, grid, dim3(256), 0, s, P, B, vec);
    }
    launched("latent_expand_small");
    return;
  }
  const dim3 grid((B + LAT_RB - 1) / LAT_RB, P.H, (P.Dv + 63) / 64);
  if (P.f32)
    hipLaunchKernelGGL(latent_expand_kernel<float>, grid, dim3(256), 0, s, P, B);
  else
    hipLaunchKernelGGL(latent_expand_kernel<bf16>, grid, dim3(256), 0, s, P, B);
  launched("latent_expand");
}

// ------------------------------------------------------------------------------------------------ short convolution
// out[r][c] = silu(bias[c] + sum_j w[c][j] in(p_r - (taps - 1) + j)[c]): tap taps - 1 is the current token's.
// Inputs before the step's first row of the sequence come from its carried window (the last taps - 1 inputs,
// oldest first; zero for a new sequence). One block per row. A sequence with a single row in the step advances its
// window there and then; for the others a second launch does: the block of a sequence's LAST row of the step writes
// the window (ascending, so a thread never reads what it has overwritten).
__global__ __launch_bounds__(256) void conv_silu_kernel(ConvParams P, StepRows R) {
  const int r = blockIdx.x, K = P.taps;
  const int seq = R.q_seq[r];
  int nb = 0;  // rows of the same sequence right before r, up to taps - 1
  while (nb < K - 1 && r - nb - 1 >= 0 && R.q_seq[r - nb - 1] == seq) ++nb;
  // a sequence with ONE row in this step (a decode step): nobody else reads its window, so this block advances it
  const bool alone = nb == 0 && !(r + 1 < R.B && R.q_seq[r + 1] == seq);
  float* win = P.state + (long long)seq * P.state_stride;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < P.ch; c += 256 * gridDim.y) {
    float acc = P.bias[c];
    const float cur = P.proj[(long long)r * P.ld + P.off_in + c];
    for (int j = 0; j < K; ++j) {
      const int back = K - 1 - j;
      const float v = back == 0 ? cur : back <= nb ? P.proj[(long long)(r - back) * P.ld + P.off_in + c]
                                                   : win[(long long)(K - 1 - (back - nb)) * P.ch + c];
      acc += P.w[(long long)c * K + j] * v;
      if (alone && back > 0) win[(long long)(K - 1 - back) * P.ch + c] = back == 1 ? cur : win[(long long)(K - back) * P.ch + c];
    }
    P.out[(long long)r * P.ld_out + c] = silu(acc);
  }
}
__global__ __launch_bounds__(256) void conv_window_kernel(ConvParams P, StepRows R) {
  const int r = blockIdx.x, K = P.taps;
  const int seq = R.q_seq[r];
  if (r + 1 < R.B && R.q_seq[r + 1] == seq) return;  // not the sequence's last row of this step
  if (!(r > 0 && R.q_seq[r - 1] == seq)) return;     // its only row: the first launch advanced the window
  int n = 1;  // rows of the sequence in this step, up to taps - 1
  while (n < K - 1 && r - n >= 0 && R.q_seq[r - n] == seq) ++n;
  float* win = P.state + (long long)seq * P.state_stride;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < P.ch; c += 256 * gridDim.y)
    for (int sidx = 0; sidx < K - 1; ++sidx) {
      const int back = K - 2 - sidx;
      win[(long long)sidx * P.ch + c] = back < n ? P.proj[(long long)(r - back) * P.ld + P.off_in + c]
                                                 : win[(long long)(sidx + n) * P.ch + c];
    }
}
void conv_silu(const ConvParams& P, const StepRows& R, hipStream_t s) {
  check(R.B > 0 && P.proj && P.w && P.bias && P.out && P.ch > 0 && P.taps >= 1 && (P.taps == 1 || P.state),
        "conv_silu: bad operands");
  const dim3 grid(R.B, (P.ch + 255) / 256);  // a block per (row, 256 channels)
  hipLaunchKernelGGL(conv_silu_kernel, grid, dim3(256), 0, s, P, R);
  launched("conv_silu");
  if (P.taps > 1 && R.B > 1) {  // a single row is alone in its sequence
    hipLaunchKernelGGL(conv_window_kernel, grid, dim3(256), 0, s, P, R);
    launched("conv_window");
  }
}

// ------------------------------------------------------------------------------------------------ gated state scan
// S_t = a_t S_(t-1) + b_t k_t v_t^T (S is D x Dv per head), o_t = S_t^T q_t, with per-row scalars
//   SCAN_MLSTM: i = cap tanh((i_raw + i_b) / cap), f = logsigmoid(cap tanh((f_raw + f_b) / cap)),
//               m_t = max(f + m_(t-1), i), a = exp(f + m_(t-1) - m_t), b = exp(i - m_t); q scaled by D^(-1/2); a
//               normaliser n_t = a n_(t-1) + b k_t rides along, and
//               y = o / (max(|n_t . q|, exp(-m_t)) + 1e-6)
//   SCAN_SSD:   dt = softplus(dt_raw + dt_bias), a = exp(-exp(A_log) dt), b = dt; q = C_t, k = B_t of the head's
//               group, v = x_t (all three from the convolution's output); y = (o + D x_t) silu(z_t)
// One block per (sequence segment of the step, head), as the retention kernel: the block of the segment's first
// row walks its rows; thread (g, j) = (tid / Dv, tid % Dv) keeps S[i][j], i = g, g + NG, ..., in registers, so the
// update needs no exchange and o is a sum of NG partials per column; the mLSTM's normaliser sits with threads
// tid < D. The slot's state (S, then for the mLSTM n and m) is read once and written back once per step.
__device__ __forceinline__ float softplusf(float z) { return z > 20.f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float logsigmoidf(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }
template <int MODE, int MAXI>
__global__ __launch_bounds__(256) void gated_scan_kernel(ScanParams P, StepRows R) {
  __shared__ float qs[256], ks[256], vs[256], po[256], os[256], nred[4];
  const int r0 = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int seq = R.q_seq[r0];
  if (r0 > 0 && R.q_seq[r0 - 1] == seq) return;  // not the first row of its segment (uniform per block)
  const int D = P.D, Dv = P.Dv;
  const int NG = 256 / Dv;
  const int g = tid / Dv, j = tid % Dv;
  const bool act = g < NG;
  const int hg = h / (P.H / P.G);
  float* sbase = P.state + (long long)seq * P.state_stride;
  float* S0 = sbase + (long long)h * D * Dv;
  float* nvec = sbase + (long long)P.H * D * Dv + (long long)h * D;   // mLSTM only
  float* mptr = sbase + (long long)P.H * D * (Dv + 1) + h;            // mLSTM only
  float S[MAXI];
#pragma unroll
  for (int ii = 0; ii < MAXI; ++ii) {
    const int i = g + ii * NG;
    S[ii] = (act && i < D) ? S0[(long long)i * Dv + j] : 0.f;
  }
  // the mLSTM's normaliser n [D] lives with threads tid < D; its product with q is a sum over the block's waves
  float nreg = (MODE == SCAN_MLSTM && tid < D) ? nvec[tid] : 0.f;
  float m = MODE == SCAN_MLSTM ? *mptr : 0.f;
  const float qscale = MODE == SCAN_MLSTM ? 1.f / sqrtf((float)D) : 1.f;
  for (int r = r0; r < R.B && R.q_seq[r] == seq; ++r) {
    const float* row = P.proj + (long long)r * P.ld;
    const float* src = MODE == SCAN_MLSTM ? row : P.conv + (long long)r * P.ld_conv;
    float a, b;
    if (MODE == SCAN_MLSTM) {
      const float ig = P.cap * tanhf((row[P.off_i + h] + P.i_b[h]) / P.cap);
      const float fg = logsigmoidf(P.cap * tanhf((row[P.off_f + h] + P.f_b[h]) / P.cap));
      const float mn = fmaxf(fg + m, ig);
      a = expf(fg + m - mn);
      b = expf(ig - mn);
      m = mn;
    } else {
      const float dt = softplusf(row[P.off_i + h] + P.dt_bias[h]);
      a = expf(-expf(P.a_log[h]) * dt);
      b = dt;
    }
    float qv = 0.f, kv = 0.f;
    if (tid < D) {
      qv = src[P.off_q + hg * D + tid] * qscale;
      kv = src[P.off_k + hg * D + tid];
      qs[tid] = qv;
      ks[tid] = kv;
    }
    if (tid < Dv) vs[tid] = src[P.off_v + h * Dv + tid];
    if (MODE == SCAN_MLSTM) {
      nreg = a * nreg + b * kv;
      const float pn = wave_sum(nreg * qv);
      if ((tid & 63) == 0) nred[tid >> 6] = pn;
    }
    __syncthreads();
    float part = 0.f;
    if (act) {
      const float bv = b * vs[j];
#pragma unroll
      for (int ii = 0; ii < MAXI; ++ii) {
        const int i = g + ii * NG;
        if (i < D) {
          S[ii] = a * S[ii] + ks[i] * bv;
          part += S[ii] * qs[i];
        }
      }
    }
    po[tid] = part;
    __syncthreads();
    if (tid < Dv) {
      float o = 0.f;
      for (int gg = 0; gg < NG; ++gg) o += po[gg * Dv + tid];
      float y;
      if (MODE == SCAN_MLSTM)
        y = o / (fmaxf(fabsf(nred[0] + nred[1] + nred[2] + nred[3]), expf(-m)) + 1e-6f);
      else
        y = (o + P.d_skip[h] * vs[tid]) * silu(row[P.off_g + h * Dv + tid]);
      P.y[(long long)r * P.ld_y + h * Dv + tid] = y;
    }
    __syncthreads();
  }
#pragma unroll
  for (int ii = 0; ii < MAXI; ++ii) {
    const int i = g + ii * NG;
    if (act && i < D) S0[(long long)i * Dv + j] = S[ii];
  }
  if (MODE == SCAN_MLSTM) {
    if (tid < D) nvec[tid] = nreg;
    if (tid == 0) *mptr = m;
  }
}
bool gated_scan_supported(int mode, int D, int Dv) {
  (void)mode;
  if (D <= 0 || Dv <= 0 || D > 256 || Dv > 256) return false;
  const int ng = 256 / Dv;
  return (D + ng - 1) / ng <= 64;
}
template <int MODE>
static void launch_gated_scan(const ScanParams& P, const StepRows& R, hipStream_t s) {
  const int ng = 256 / P.Dv, ni = (P.D + ng - 1) / ng;
  const dim3 grid(R.B, P.H);
  if (ni <= 8)
    hipLaunchKernelGGL((gated_scan_kernel<MODE, 8>), grid, dim3(256), 0, s, P, R);
  else if (ni <= 16)
    hipLaunchKernelGGL((gated_scan_kernel<MODE, 16>), grid, dim3(256), 0, s, P, R);
  else if (ni <= 32)
    hipLaunchKernelGGL((gated_scan_kernel<MODE, 32>), grid, dim3(256), 0, s, P, R);
  else
    hipLaunchKernelGGL((gated_scan_kernel<MODE, 64>), grid, dim3(256), 0, s, P, R);
}
void gated_scan(const ScanParams& P, const StepRows& R, hipStream_t s) {
  check(R.B > 0 && P.proj && P.state && P.y && P.H > 0 && P.G > 0 && P.H % P.G == 0 && gated_scan_supported(P.mode, P.D, P.Dv),
        "gated scan: operands or head sizes (key and value size <= 256, state within the registers)");
  if (P.mode == SCAN_MLSTM) {
    check(P.i_b && P.f_b && P.cap > 0.f && P.G == P.H, "gated scan: mLSTM gate operands");
    launch_gated_scan<SCAN_MLSTM>(P, R, s);
  } else {
    check(P.conv && P.dt_bias && P.a_log && P.d_skip, "gated scan: state space operands");
    launch_gated_scan<SCAN_SSD>(P, R, s);
  }
  launched("gated_scan");
}

// ---- prompt portions: the same recurrence in chunks of SC tokens, as the chunked retention but with per-row decays.
// With l_s = ln a_s and L_t = l_0 + ... + l_t inside a chunk of n tokens that starts from state S,
//   A[t][s] = (q_t . k_s) exp(L_t - L_s) b_s for s <= t,   o_t = exp(L_t) S^T q_t + sum_s A[t][s] v_s,
//   U = sum_s exp(L_(n-1) - L_s) b_s k_s v_s^T,              S <- exp(L_(n-1)) S + U,
// all in float32 on the vector ALUs, over the host-built chunk table {first row, rows, state slot, flags}:
//   0. per (row, head) coefficients {l, b, m}: gated_coef_*                       (the mLSTM's running maximum is a
//      scan of x -> max(x + f, i), composed over a wave's 64 rows at a time)
//   1. every chunk's U and its total log decay, chunks in parallel                (gated_u_kernel)
//   2. the scan over each sequence's chunks, one thread per state element        (gated_chunk_scan_kernel)
//   3. every chunk's outputs from its incoming state, in parallel                (gated_out_kernel)
// The mLSTM's normaliser is column Dv of the state here too; its raw outputs [B][H][Dv + 1] are finished by
// mlstm_finish_kernel (the division, the per-head unit RMS, the norm's weight, the output gate).
constexpr int SC = 32;
int gated_chunk_rows() { return SC; }
bool gated_chunk_supported(int mode, int D, int Dv) { return D > 0 && D <= 128 && Dv > 0 && Dv + (mode == SCAN_MLSTM ? 1 : 0) <= 256; }

__global__ __launch_bounds__(256) void gated_coef_ssd_kernel(ScanParams P, int B, float* __restrict__ coef) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= B * P.H) return;
  const int r = idx / P.H, h = idx % P.H;
  const float dt = softplusf(P.proj[(long long)r * P.ld + P.off_i + h] + P.dt_bias[h]);
  coef[(long long)idx * 3] = -expf(P.a_log[h]) * dt;
  coef[(long long)idx * 3 + 1] = dt;
  coef[(long long)idx * 3 + 2] = 0.f;
}
// one wave per (sequence segment, head); lanes take 64 consecutive rows, the running maximum crosses them as the
// composition of the rows' maps x -> max(x + c, d): (c1, d1) then (c2, d2) = (c1 + c2, max(d1 + c2, d2))
__global__ __launch_bounds__(256) void gated_coef_mlstm_kernel(ScanParams P, StepRows R, float* __restrict__ coef) {
  const int r0 = blockIdx.x, lane = threadIdx.x & 63;
  const int h = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int seq = R.q_seq[r0];
  if (r0 > 0 && R.q_seq[r0 - 1] == seq) return;
  if (h >= P.H) return;
  float* mptr = P.state + (long long)seq * P.state_stride + (long long)P.H * P.D * (P.Dv + 1) + h;
  float m_in = *mptr;
  for (int t0 = r0; t0 < R.B; t0 += 64) {
    const int r = t0 + lane;
    const bool valid = r < R.B && R.q_seq[r] == seq;
    float c = 0.f, d = -INFINITY, ig = 0.f, fg = 0.f;
    if (valid) {
      const float* row = P.proj + (long long)r * P.ld;
      ig = P.cap * tanhf((row[P.off_i + h] + P.i_b[h]) / P.cap);
      fg = logsigmoidf(P.cap * tanhf((row[P.off_f + h] + P.f_b[h]) / P.cap));
      c = fg;
      d = ig;
    }
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {  // inclusive scan of the composed maps
      const float pc = __shfl_up(c, off, 64), pd = __shfl_up(d, off, 64);
      if (lane >= off) {
        d = fmaxf(pd + c, d);
        c = pc + c;
      }
    }
    const float m = fmaxf(m_in + c, d);                    // the running maximum after this lane's row
    float mp = __shfl_up(m, 1, 64);
    if (lane == 0) mp = m_in;
    if (valid) {
      float* o = coef + ((long long)r * P.H + h) * 3;
      o[0] = fg + mp - m;
      o[1] = expf(ig - m);
      o[2] = m;
    }
    const unsigned long long mask = __ballot(valid);
    const int cnt = __popcll(mask);
    if (cnt == 0) break;
    m_in = __shfl(m, cnt - 1, 64);
    if (cnt < 64) break;
  }
  if (lane == 0) *mptr = m_in;
}
// q (scaled for the mLSTM) and k rows of a chunk into LDS; rows past cn and dims past D zero
template <int MODE, int MAXD, bool WITH_Q>
__device__ __forceinline__ void stage_qk_gated(const ScanParams& P, int row0, int cn, int hg, float (*Qs)[MAXD],
                                               float (*Ks)[MAXD + 4]) {
  const float qscale = MODE == SCAN_MLSTM ? 1.f / sqrtf((float)P.D) : 1.f;
  for (int idx = threadIdx.x; idx < SC * MAXD; idx += 256) {
    const int c = idx / MAXD, d = idx % MAXD;
    float qv = 0.f, kv = 0.f;
    if (c < cn && d < P.D) {
      const float* src = MODE == SCAN_MLSTM ? P.proj + (long long)(row0 + c) * P.ld : P.conv + (long long)(row0 + c) * P.ld_conv;
      kv = src[P.off_k + hg * P.D + d];
      if (WITH_Q) qv = src[P.off_q + hg * P.D + d] * qscale;
    }
    if (WITH_Q) Qs[c][d] = qv;
    Ks[c][d] = kv;
  }
}
// value columns jb * 64 .. + 63 of a chunk's rows; the mLSTM's column Dv is 1 (the normaliser)
template <int MODE>
__device__ __forceinline__ void stage_v_gated(const ScanParams& P, int row0, int cn, int h, int jb, float (*Vs)[64]) {
  for (int idx = threadIdx.x; idx < SC * 64; idx += 256) {
    const int c = idx >> 6, col = jb * 64 + (idx & 63);
    float v = 0.f;
    if (c < cn) {
      const float* src = MODE == SCAN_MLSTM ? P.proj + (long long)(row0 + c) * P.ld : P.conv + (long long)(row0 + c) * P.ld_conv;
      if (col < P.Dv)
        v = src[P.off_v + h * P.Dv + col];
      else if (MODE == SCAN_MLSTM && col == P.Dv)
        v = 1.f;
    }
    Vs[c][idx & 63] = v;
  }
}
// Lc[t] = l_0 + ... + l_t and bw[t] = b_t of the chunk's rows (Lc past cn stays at its last value)
__device__ __forceinline__ void stage_coef(const ScanParams& P, const float* coef, int row0, int cn, int h, float* Lc, float* bw) {
  if (threadIdx.x < SC) {
    const int t = threadIdx.x;
    const float* c = coef + ((long long)(row0 + min(t, cn - 1)) * P.H + h) * 3;
    Lc[t] = t < cn ? c[0] : 0.f;
    bw[t] = t < cn ? c[1] : 0.f;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float acc = 0.f;
    for (int t = 0; t < SC; ++t) {
      acc += Lc[t];
      Lc[t] = acc;
    }
  }
  __syncthreads();
}
template <int MODE, int MAXD>
__global__ __launch_bounds__(256) void gated_u_kernel(ScanParams P, const int* __restrict__ chunks, const float* __restrict__ coef,
                                                      float* __restrict__ U, long long u_stride, float* __restrict__ ctot,
                                                      int NJ) {
  __shared__ __attribute__((aligned(16))) float Ks[SC][MAXD + 4];
  __shared__ float Vs[SC][64];
  __shared__ float Lc[SC], bw[SC];
  const int c = blockIdx.x, h = blockIdx.y / NJ, jb = blockIdx.y % NJ, tid = threadIdx.x;
  const int row0 = chunks[4 * c], cn = chunks[4 * c + 1];
  const int Dvp = P.Dv + (MODE == SCAN_MLSTM ? 1 : 0);
  const int j = tid & 63, g4 = tid >> 6, col = jb * 64 + j;
  stage_coef(P, coef, row0, cn, h, Lc, bw);
  stage_qk_gated<MODE, MAXD, false>(P, row0, cn, h / (P.H / P.G), nullptr, Ks);
  stage_v_gated<MODE>(P, row0, cn, h, jb, Vs);
  __syncthreads();
  if (jb == 0 && tid == 0) ctot[(long long)c * P.H + h] = Lc[cn - 1];
  float u[MAXD / 4];
#pragma unroll
  for (int ii = 0; ii < MAXD / 4; ++ii) u[ii] = 0.f;
  for (int sx = 0; sx < cn; ++sx) {
    const float vv = Vs[sx][j] * (expf(Lc[cn - 1] - Lc[sx]) * bw[sx]);
#pragma unroll
    for (int ii = 0; ii < MAXD / 4; ++ii) u[ii] += Ks[sx][g4 + 4 * ii] * vv;
  }
  if (col < Dvp) {
    float* out = U + c * u_stride + (long long)h * P.D * Dvp;
#pragma unroll
    for (int ii = 0; ii < MAXD / 4; ++ii) {
      const int i = g4 + 4 * ii;
      if (i < P.D) out[(long long)i * Dvp + col] = u[ii];
    }
  }
}
template <int MODE>
__global__ __launch_bounds__(256) void gated_chunk_scan_kernel(ScanParams P, const int* __restrict__ chunks, int nchunks,
                                                               const float* __restrict__ U, float* __restrict__ Sin,
                                                               long long u_stride, const float* __restrict__ ctot) {
  const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
  const int Dvp = P.Dv + (MODE == SCAN_MLSTM ? 1 : 0);
  const long long per_head = (long long)P.D * Dvp;
  if (e >= P.H * per_head) return;
  const int h = (int)(e / per_head), i = (int)(e % per_head) / Dvp, j = (int)(e % per_head) % Dvp;
  // where this element lives in a slot's state: S [H][D][Dv], then (mLSTM) the normaliser [H][D]
  const long long at = j < P.Dv ? ((long long)h * P.D + i) * P.Dv + j : (long long)P.H * P.D * P.Dv + (long long)h * P.D + i;
  float S = 0.f;
  for (int c = 0; c < nchunks; ++c) {
    const int slot = chunks[4 * c + 2], flags = chunks[4 * c + 3];
    float* st_e = P.state + (long long)slot * P.state_stride + at;
    if (flags & 1) S = *st_e;
    Sin[c * u_stride + e] = S;
    S = expf(ctot[(long long)c * P.H + h]) * S + U[c * u_stride + e];
    if (flags & 2) *st_e = S;
  }
}
template <int MODE, int MAXD>
__global__ __launch_bounds__(256) void gated_out_kernel(ScanParams P, const int* __restrict__ chunks, const float* __restrict__ coef,
                                                        const float* __restrict__ Sin, long long u_stride,
                                                        float* __restrict__ raw, int ld_raw, int NJ) {
  __shared__ __attribute__((aligned(16))) float Qs[SC][MAXD];
  __shared__ __attribute__((aligned(16))) float Ks[SC][MAXD + 4];
  __shared__ float Vs[SC][64];
  __shared__ float As[SC][SC + 1];
  __shared__ float Lc[SC], bw[SC];
  const int c = blockIdx.x, h = blockIdx.y / NJ, jb = blockIdx.y % NJ, tid = threadIdx.x;
  const int row0 = chunks[4 * c], cn = chunks[4 * c + 1];
  const int D = P.D, Dv = P.Dv;
  const int Dvp = Dv + (MODE == SCAN_MLSTM ? 1 : 0);
  const int j = tid & 63, g4 = tid >> 6, col = jb * 64 + j;
  const bool colok = col < Dvp;
  float S[MAXD];
  const float* sin_base = Sin + c * u_stride + (long long)h * D * Dvp;
#pragma unroll
  for (int i = 0; i < MAXD; ++i) S[i] = (colok && i < D) ? sin_base[(long long)i * Dvp + col] : 0.f;
  stage_coef(P, coef, row0, cn, h, Lc, bw);
  stage_qk_gated<MODE, MAXD, true>(P, row0, cn, h / (P.H / P.G), Qs, Ks);
  stage_v_gated<MODE>(P, row0, cn, h, jb, Vs);
  __syncthreads();
#pragma unroll
  for (int kx = 0; kx < SC * SC / 256; ++kx) {
    const int t = (tid >> 5) + 8 * kx, sx = tid & 31;
    float dot = 0.f;
    if (sx <= t && t < cn) {
#pragma unroll
      for (int i4 = 0; i4 < MAXD / 4; ++i4) {
        const f32x4 qa = *(const f32x4*)&Qs[t][4 * i4], kb = *(const f32x4*)&Ks[sx][4 * i4];
        dot += qa[0] * kb[0] + qa[1] * kb[1] + qa[2] * kb[2] + qa[3] * kb[3];
      }
      dot *= expf(Lc[t] - Lc[sx]) * bw[sx];
    }
    As[t][sx] = dot;
  }
  __syncthreads();
  for (int t = g4; t < cn; t += 4) {
    float inter = 0.f;
#pragma unroll
    for (int i4 = 0; i4 < MAXD / 4; ++i4) {
      const f32x4 qa = *(const f32x4*)&Qs[t][4 * i4];
      inter += qa[0] * S[4 * i4] + qa[1] * S[4 * i4 + 1] + qa[2] * S[4 * i4 + 2] + qa[3] * S[4 * i4 + 3];
    }
    float intra = 0.f;
#pragma unroll
    for (int sx = 0; sx < SC; ++sx) intra += As[t][sx] * Vs[sx][j];  // As is zero above the diagonal
    if (colok) {
      const float o = expf(Lc[t]) * inter + intra;
      const long long r = row0 + t;
      if (MODE == SCAN_MLSTM)
        raw[r * ld_raw + h * Dvp + col] = o;
      else
        P.y[r * P.ld_y + h * Dv + col] = (o + P.d_skip[h] * Vs[t][j]) * silu(P.proj[r * P.ld + P.off_g + h * Dv + col]);
    }
  }
}
// mLSTM: y = o / (max(|n . q|, exp(-m)) + 1e-6), divided by its root mean square over the head, times the norm's
// weight and the sigmoid output gate; one wave per (row, head)
template <typename T>
__global__ __launch_bounds__(256) void mlstm_finish_kernel(ScanParams P, int B, const float* __restrict__ raw, int ld_raw,
                                                           const float* __restrict__ coef, const float* __restrict__ w, float eps,
                                                           T* __restrict__ out, int ld_out) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= B * P.H) return;
  const int b = item / P.H, h = item % P.H, Dv = P.Dv;
  const float* o = raw + (long long)b * ld_raw + h * (Dv + 1);
  const float den = fmaxf(fabsf(o[Dv]), expf(-coef[(long long)item * 3 + 2])) + 1e-6f;
  float sq = 0.f;
  for (int jx = lane; jx < Dv; jx += 64) sq += (o[jx] / den) * (o[jx] / den);
  const float rs = 1.f / sqrtf(wave_sum(sq) / (float)Dv + eps);
  const float* gate = P.proj + (long long)b * P.ld + P.off_g + h * Dv;
  for (int jx = lane; jx < Dv; jx += 64)
    st(out + (long long)b * ld_out + h * Dv + jx, o[jx] / den * rs * w[h * Dv + jx] * sigmoidf(gate[jx]));
}
template <int MODE, int MAXD>
static void launch_gated_chunked(const ScanParams& P, const StepRows& R, const ScanChunkWs& W, hipStream_t s) {
  const int Dvp = P.Dv + (MODE == SCAN_MLSTM ? 1 : 0), NJ = (Dvp + 63) / 64;
  const dim3 grid(W.nchunks, P.H * NJ);
  hipLaunchKernelGGL((gated_u_kernel<MODE, MAXD>), grid, dim3(256), 0, s, P, W.chunks, W.coef, W.U, W.u_stride, W.ctot, NJ);
  launched("gated_u");
  const long long elems = (long long)P.H * P.D * Dvp;
  hipLaunchKernelGGL(gated_chunk_scan_kernel<MODE>, dim3((unsigned)((elems + 255) / 256)), dim3(256), 0, s, P, W.chunks, W.nchunks,
                     W.U, W.Sin, W.u_stride, W.ctot);
  launched("gated_chunk_scan");
  hipLaunchKernelGGL((gated_out_kernel<MODE, MAXD>), grid, dim3(256), 0, s, P, W.chunks, W.coef, W.Sin, W.u_stride, W.raw,
                     W.ld_raw, NJ);
  launched("gated_out");
}
void gated_scan_chunked(const ScanParams& P, const StepRows& R, const ScanChunkWs& W, const float* norm_w, float eps, void* out,
                        int ld_out, int f32, hipStream_t s) {
  const int Dvp = P.Dv + (P.mode == SCAN_MLSTM ? 1 : 0);
  check(R.B > 0 && P.proj && P.state && P.H > 0 && P.G > 0 && P.H % P.G == 0 && gated_chunk_supported(P.mode, P.D, P.Dv),
        "chunked gated scan: key size <= 128, value size <= 255");
  check(W.chunks && W.nchunks > 0 && W.nchunks <= W.max_chunks && W.U && W.Sin && W.coef && W.ctot &&
            W.u_stride >= (long long)P.H * P.D * Dvp,
        "chunked gated scan: chunk table or workspace");
  if (P.mode == SCAN_MLSTM) {
    check(P.i_b && P.f_b && P.cap > 0.f && P.G == P.H && W.raw && W.ld_raw >= P.H * Dvp && norm_w && out, "chunked mLSTM operands");
    hipLaunchKernelGGL(gated_coef_mlstm_kernel, dim3(R.B, (P.H + 3) / 4), dim3(256), 0, s, P, R, W.coef);
    launched("gated_coef_mlstm");
    if (P.D <= 64)
      launch_gated_chunked<SCAN_MLSTM, 64>(P, R, W, s);
    else
      launch_gated_chunked<SCAN_MLSTM, 128>(P, R, W, s);
    const dim3 g2((R.B * P.H + 3) / 4);
    if (f32)
      hipLaunchKernelGGL(mlstm_finish_kernel<float>, g2, dim3(256), 0, s, P, R.B, W.raw, W.ld_raw, W.coef, norm_w, eps, (float*)out,
                         ld_out);
    else
      hipLaunchKernelGGL(mlstm_finish_kernel<bf16>, g2, dim3(256), 0, s, P, R.B, W.raw, W.ld_raw, W.coef, norm_w, eps, (bf16*)out,
                         ld_out);
    launched("mlstm_finish");
  } else {
    check(P.conv && P.dt_bias && P.a_log && P.d_skip && P.y, "chunked state space operands");
    hipLaunchKernelGGL(gated_coef_ssd_kernel, dim3((R.B * P.H + 255) / 256), dim3(256), 0, s, P, R.B, W.coef);
    launched("gated_coef_ssd");
    if (P.D <= 64)
      launch_gated_chunked<SCAN_SSD, 64>(P, R, W, s);
    else
      launch_gated_chunked<SCAN_SSD, 128>(P, R, W, s);
  }
}

// ------------------------------------------------------------------------------------------------ grouped RMS norm
// out[r][i] = y[r][i] / sqrt(mean over i's part of y^2 + eps) * w[i] * (gate ? sigmoid(gate[r][i]) : 1), the row in
// `groups` equal parts; grid (rows, groups)
template <typename T>
__global__ __launch_bounds__(256) void group_rms_kernel(const float* __restrict__ y, int ld_y, int n, int groups,
                                                        const float* __restrict__ w, float eps, const float* __restrict__ gate,
                                                        int ld_gate, T* __restrict__ out, int ld_out) {
  __shared__ float red[4];
  const long long r = blockIdx.x;
  const int per = n / groups, i0 = blockIdx.y * per;
  const float* yr = y + r * ld_y + i0;
  float sq = 0.f;
  for (int i = threadIdx.x; i < per; i += 256) sq += yr[i] * yr[i];
  const float inv = 1.f / sqrtf(block_sum256(sq, red) / (float)per + eps);
  for (int i = threadIdx.x; i < per; i += 256) {
    float v = yr[i] * inv * w[i0 + i];
    if (gate) v *= sigmoidf(gate[r * ld_gate + i0 + i]);
    st(out + r * ld_out + i0 + i, v);
  }
}
void group_rms_cast(const float* y, int ld_y, int rows, int n, int groups, const float* w, float eps, const float* gate,
                    int ld_gate, void* out, int ld_out, int f32, hipStream_t s) {
  check(rows > 0 && n > 0 && groups > 0 && n % groups == 0 && y && w && out, "group_rms_cast: bad operands");
  const dim3 grid(rows, groups);
  if (f32)
    hipLaunchKernelGGL(group_rms_kernel<float>, grid, dim3(256), 0, s, y, ld_y, n, groups, w, eps, gate, ld_gate, (float*)out,
                       ld_out);
  else
    hipLaunchKernelGGL(group_rms_kernel<bf16>, grid, dim3(256), 0, s, y, ld_y, n, groups, w, eps, gate, ld_gate, (bf16*)out,
                       ld_out);
  launched("group_rms_cast");
}

// ------------------------------------------------------------------------------------------------ dense feed-forward
// out[r][f] = relu(z[r][f])^2 in the matrix dtype
template <typename T>
__global__ __launch_bounds__(256) void relu2_kernel(const float* __restrict__ z, int ld, int rows, int F, T* __restrict__ out,
                                                    int ld_out) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long long)rows * F) return;
  const long long r = i / F;
  const int f = (int)(i % F);
  const float v = fmaxf(z[r * ld + f], 0.f);
  st(out + r * ld_out + f, v * v);
}
void relu2_cast(const float* z, int ld, int rows, int F, void* out, int ld_out, int f32, hipStream_t s) {
  check(rows > 0 && F > 0 && z && out, "relu2_cast: bad operands");
  const long long n = (long long)rows * F;
  const dim3 grid((unsigned)((n + 255) / 256));
  if (f32)
    hipLaunchKernelGGL(relu2_kernel<float>, grid, dim3(256), 0, s, z, ld, rows, F, (float*)out, ld_out);
  else
    hipLaunchKernelGGL(relu2_kernel<bf16>, grid, dim3(256), 0, s, z, ld, rows, F, (bf16*)out, ld_out);
  launched("relu2_cast");
}

// ------------------------------------------------------------------------------------------------ score router
// Per row: s = softmax of the X + I router logits; choice = s + correction; the outputs form group_count groups of
// neighbours, a group ranks by its largest choice score and only outputs of the best group_keep groups can be
// chosen; the `top` largest choice scores among them are taken (ties: the lower index), weighted by their s (not
// renormalised). Outputs X .. X + I - 1 are identity experts: their weight is summed into idw[r] (the post-norm
// update adds idw * x) and their place in the expert list points at expert 0 with weight 0. The shared expert
// has no gate (sgate = 1); its activation silu(gate) * up is written behind the routed ones, as moe_route does.
constexpr int ROUTE_MAX = 256;
template <typename T>
__global__ __launch_bounds__(256) void moe_route_scores_kernel(MoeParams P) {
  __shared__ float sc[ROUTE_MAX], ch[ROUTE_MAX];
  const int b = blockIdx.x, NR = P.X + P.identity;
  const float* row = P.proj + (long long)b * P.ld;
  if (threadIdx.x == 0) {
    float mx = -INFINITY;
    for (int e = 0; e < NR; ++e) mx = fmaxf(mx, row[P.off_router + e]);
    float sum = 0.f;
    for (int e = 0; e < NR; ++e) {
      sc[e] = expf(row[P.off_router + e] - mx);
      sum += sc[e];
    }
    for (int e = 0; e < NR; ++e) {
      sc[e] /= sum;
      ch[e] = sc[e] + P.router_b[e];
    }
    if (P.group_count > 1) {  // drop the groups outside the best group_keep
      const int per = NR / P.group_count;
      unsigned long long kept = 0ull;
      for (int q = 0; q < P.group_keep; ++q) {
        int best = -1;
        float bv = -INFINITY;
        for (int gi = 0; gi < P.group_count; ++gi) {
          if (kept >> gi & 1ull) continue;
          float gm = -INFINITY;
          for (int e = gi * per; e < (gi + 1) * per; ++e) gm = fmaxf(gm, ch[e]);
          if (best < 0 || gm > bv) {
            best = gi;
            bv = gm;
          }
        }
        kept |= 1ull << best;
      }
      for (int gi = 0; gi < P.group_count; ++gi)
        if (!(kept >> gi & 1ull))
          for (int e = gi * per; e < (gi + 1) * per; ++e) ch[e] = -INFINITY;
    }
    float idw = 0.f;
    for (int jj = 0; jj < P.top; ++jj) {
      int best = 0;
      float bv = -INFINITY;
      bool any = false;
      for (int e = 0; e < NR; ++e) {
        if (ch[e] == -INFINITY) continue;  // outside the kept groups, or taken
        if (!any || ch[e] > bv) {
          best = e;
          bv = ch[e];
          any = true;
        }
      }
      if (any) ch[best] = -INFINITY;
      const bool real = any && best < P.X;
      P.eids[(long long)b * P.ld_top + jj] = real ? best : 0;
      P.ew[(long long)b * P.ld_top + jj] = real ? sc[best] : 0.f;
      if (any && !real) idw += sc[best];
    }
    P.idw[b] = idw;
    if (P.Fs > 0) P.sgate[b] = 1.f;
  }
  T* hm = (T*)P.hmid + (long long)b * P.ld_hmid + P.top * P.F;
  for (int f = threadIdx.x; f < P.Fs; f += 256) st(hm + f, silu(row[P.off_sgate + f]) * row[P.off_sup + f]);
}
// ---- a few rows (decode steps): routing and the routed and shared activations in one launch, as the top-k router's
// moe_route_experts_kernel. Grid (ff units / 4, row x (top + 1)); every wave routes its row itself with one router
// output per lane (X + identity <= 64): softmax across the lanes, one wave maximum per group, `keep` rounds of "best
// group", `top` rounds of "best output" (ties: the lower lane). Block (0, row, 0) records ids, weights and idw.
template <typename T>
__global__ __launch_bounds__(256) void moe_route_scores_experts_kernel(MoeParams P, int vec) {
  const int lane = threadIdx.x & 63;
  const int f = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int b = blockIdx.y / (P.top + 1), jj = blockIdx.y % (P.top + 1);
  const float* row = P.proj + (long long)b * P.ld;
  T* hm = (T*)P.hmid + (long long)b * P.ld_hmid;
  if (jj == P.top) {  // shared expert
    if (f < P.Fs && lane == 0) st(hm + P.top * P.F + f, silu(row[P.off_sgate + f]) * row[P.off_sup + f]);
    return;
  }
  const int NR = P.X + P.identity;
  const bool has = lane < NR;
  const float z = has ? row[P.off_router + lane] : -INFINITY;
  const float zmax = wave_max(z);  // (every lane takes part in a wave reduction: never inside a lane condition)
  const float ex = has ? expf(z - zmax) : 0.f;
  const float sc = ex / wave_sum(ex);
  float ch = has ? sc + P.router_b[lane] : -INFINITY;
  if (P.group_count > 1) {
    const int per = NR / P.group_count, mine = has ? lane / per : -1;
    float gmax = -INFINITY;  // the largest choice score of this lane's group
    for (int gi = 0; gi < P.group_count; ++gi) {
      const float v = wave_max(mine == gi ? ch : -INFINITY);
      if (mine == gi) gmax = v;
    }
    bool kept = false;
    float gm = has ? gmax : -INFINITY;
    for (int q = 0; q < P.group_keep; ++q) {
      const float best = wave_max(gm);
      const int who = max(0, __ffsll((unsigned long long)__ballot(gm == best)) - 1);  // lowest lane of the best group
      const int gsel = who / per;
      if (mine == gsel) {
        kept = true;
        gm = -INFINITY;
      }
    }
    if (!kept) ch = -INFINITY;
  }
  int e = -1;
  float idw = 0.f;
  const bool rec = threadIdx.x < 64 && blockIdx.x == 0 && jj == 0;  // the wave that records the row's routing
  for (int q = 0; q < P.top; ++q) {
    const float mx = wave_max(ch);
    const bool any = mx != -INFINITY;
    const int who = max(0, __ffsll((unsigned long long)__ballot(ch == mx && has)) - 1);
    const float w = __shfl(sc, who, 64);
    const bool real = any && who < P.X;
    if (q == jj) e = real ? who : -1;
    if (any && !real) idw += w;
    if (rec && lane == 0) {
      P.eids[(long long)b * P.ld_top + q] = real ? who : 0;
      P.ew[(long long)b * P.ld_top + q] = real ? w : 0.f;
    }
    if (lane == who) ch = -INFINITY;
  }
  if (rec && lane == 0) {
    P.idw[b] = idw;
    if (P.Fs > 0) P.sgate[b] = 1.f;
  }
  if (f >= P.F) return;
  if (e < 0) {  // an identity output (or none): its place carries weight 0, and a finite activation
    if (lane == 0) st(hm + jj * P.F + f, 0.f);
    return;
  }
  const T* x = (const T*)P.h + (long long)b * P.E;
  const T* wg = (const T*)P.w_gu + ((long long)e * 2 * P.F + f) * P.E;
  const T* wu = wg + (long long)P.F * P.E;
  const float gate = wave_dot<T>(wg, x, P.E, lane, vec != 0);
  const float up = wave_dot<T>(wu, x, P.E, lane, vec != 0);
  if (lane == 0) st(hm + jj * P.F + f, silu(gate) * up);
}
bool moe_route_scores_fused_supported(const MoeParams& P) { return P.X + P.identity <= 64 && P.group_count <= 64; }
void moe_route_scores_experts(const MoeParams& P, hipStream_t s) {
  check(P.B > 0 && P.proj && P.eids && P.ew && P.idw && P.router_b && P.h && P.w_gu && P.hmid && moe_route_scores_fused_supported(P) &&
            P.top > 0 && P.top <= MOE_MAX_TOP && P.group_count >= 1 && (P.X + P.identity) % P.group_count == 0 &&
            P.group_keep >= 1 && P.group_keep <= P.group_count && (P.Fs == 0 || P.sgate),
        "fused score router: operands or sizes (up to 64 router outputs)");
  const dim3 grid((std::max(P.F, P.Fs) + 3) / 4, P.B * (P.top + 1));
  if (P.f32)
    hipLaunchKernelGGL(moe_route_scores_experts_kernel<float>, grid, dim3(256), 0, s, P,
                       (int)(vec_ok<float>(P.h, P.E, P.E) && vec_ok<float>(P.w_gu, P.E, P.E)));
  else
    hipLaunchKernelGGL(moe_route_scores_experts_kernel<bf16>, grid, dim3(256), 0, s, P,
                       (int)(vec_ok<bf16>(P.h, P.E, P.E) && vec_ok<bf16>(P.w_gu, P.E, P.E)));
  launched("moe_route_scores_experts");
}
void moe_route_scores(const MoeParams& P, hipStream_t s) {
  check(P.B > 0 && P.proj && P.eids && P.ew && P.idw && P.router_b && P.X + P.identity <= ROUTE_MAX && P.top > 0 &&
            P.top <= MOE_MAX_TOP && P.group_count >= 1 && P.group_count <= 64 && (P.X + P.identity) % P.group_count == 0 &&
            P.group_keep >= 1 && P.group_keep <= P.group_count && (P.Fs == 0 || (P.sgate && P.hmid)),
        "score router: operands or sizes (up to 256 outputs in up to 64 groups)");
  if (P.f32)
    hipLaunchKernelGGL(moe_route_scores_kernel<float>, dim3(P.B), dim3(256), 0, s, P);
  else
    hipLaunchKernelGGL(moe_route_scores_kernel<bf16>, dim3(P.B), dim3(256), 0, s, P);
  launched("moe_route_scores");
}

}  // namespace stack
}  // namespace omx
