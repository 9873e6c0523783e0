// gfx950 kernels of layer-list models (interface and operand layouts: stack_ops.h). Every kernel is
// instantiated for bfloat16 and float32 matrices; norms, scores, softmax weights, router logits, the
// retention state and the residual stream are float32 in both. Wave = 64 lanes.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>
#include <stdexcept>
#include <string>

#include "stack_device.h"
#include "stack_ops.h"

namespace omx {
namespace stack {

// ------------------------------------------------------------------------------------------------ epilogue
struct Epi {
  int mode;
  float* C;
  int ldc;
  float mult;
  const float* add;
  float cap;
};
__device__ __forceinline__ void epi_store(const Epi& e, int m, int n, float acc) {
  float* c = e.C + (long long)m * e.ldc + n;
  if (e.mode == EPI_RESID) {
    const float extra = e.add ? e.add[(long long)m * e.ldc + n] : 0.f;
    *c = *c + e.mult * (acc + extra);
  } else if (e.mode == EPI_SOFTCAP && e.cap != 0.f) {
    *c = e.cap * tanhf(acc / e.cap);
  } else if (e.mode == EPI_SCALE) {
    *c = e.mult * acc;
  } else {
    *c = acc;
  }
}

// ------------------------------------------------------------------------------------------------ GEMV (M <= 8)
// one wave per weight row; the row is read once and meets every activation row
template <typename T>
__global__ __launch_bounds__(256) void gemv_rows_kernel(const T* __restrict__ A, int lda, const T* __restrict__ W, int M,
                                                        int N, int K, Epi e, int vec) {
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= N) return;
  const T* w = W + (long long)n * K;
  for (int m = 0; m < M; ++m) {
    const float acc = wave_dot<T>(w, A + (long long)m * lda, K, lane, vec != 0);
    if (lane == 0) epi_store(e, m, n, acc);
  }
}

// ---- decode steps: layer norm (nb null: RMS norm) + input projection (+ the attention layer's query temperature and K/V store)
// Every block normalises the step's few rows again (they are E floats each) into LDS, rounded to the matrix
// dtype as the unfused path stores them, then its four waves take one weight row each. Block 0 also writes the
// normed rows out for the routed experts. QkvEpi: outputs in the q range are multiplied by the row's query
// temperature, outputs in the k and v ranges are also stored at the row's cache slot.
struct QkvEpi {
  int on;
  int off_q, n_q, off_k, n_k, off_v, n_v;
  int G, D, Dv, bs;
  float coef;
  int every;
  const int* pos;
  const int* slot;
  void* kc;
  void* vc;
};
constexpr int LN_LDS_BYTES = 32768;
constexpr int LN_RW = 4;  // weight rows per wave
constexpr int LN_XR = 16;  // row elements per thread: E <= 4096
constexpr int LN_PF = 4;  // 512-element steps of them requested before the norm (bfloat16)
template <typename T>
__global__ __launch_bounds__(256) void gemv_ln_kernel(const float* __restrict__ x, int E, const float* __restrict__ nw,
                                                      const float* __restrict__ nb, float eps, const T* __restrict__ W,
                                                      int M, int N, float* __restrict__ C, int ldc, T* __restrict__ hout,
                                                      QkvEpi q, int vec) {
  __shared__ __attribute__((aligned(16))) unsigned char hs_raw[LN_LDS_BYTES];
  __shared__ float red[4];
  T* hs = (T*)hs_raw;
  const int tid = threadIdx.x, lane = tid & 63;
  const int n0 = (blockIdx.x * 4 + (tid >> 6)) * LN_RW;
  // bfloat16: the first LN_PF steps of this wave's weight rows are requested before the norm, so the norm's round
  // trips and barriers pass while the weights are on their way (E <= 2048: all of them)
  constexpr bool PREF = sizeof(T) == 2;
  u32x4 pre[LN_PF][LN_RW];
  if (PREF && vec) {
#pragma unroll
    for (int it = 0; it < LN_PF; ++it)
#pragma unroll
      for (int u = 0; u < LN_RW; ++u) {
        const int k = min(lane * 8 + it * 512, E - 8);
        pre[it][u] = *(const u32x4*)(W + (long long)min(n0 + u, N - 1) * E + k);
      }
  }
  for (int m = 0; m < M; ++m) {  // the row is read once (E <= 256 LN_XR) and normalised from registers
    const float* row = x + (long long)m * E;
    float xr[LN_XR], gw[LN_XR], gb[LN_XR];
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < LN_XR; ++j) {
      const int i = tid + 256 * j;
      xr[j] = i < E ? row[i] : 0.f;
      gw[j] = i < E ? nw[i] : 0.f;
      gb[j] = (nb && i < E) ? nb[i] : 0.f;
      sum += xr[j];
    }
    const float mean = nb ? block_sum256(sum, red) / (float)E : 0.f;  // no bias vector: an RMS norm, nothing is centred
    float sq = 0.f;
#pragma unroll
    for (int j = 0; j < LN_XR; ++j) {
      const float d = tid + 256 * j < E ? xr[j] - mean : 0.f;
      sq += d * d;
    }
    const float rstd = 1.f / sqrtf(block_sum256(sq, red) / (float)E + eps);
#pragma unroll
    for (int j = 0; j < LN_XR; ++j) {
      const int i = tid + 256 * j;
      if (i < E) {
        st(hs + (long long)m * E + i, (xr[j] - mean) * rstd * gw[j] + gb[j]);
        if (blockIdx.x == 0) hout[(long long)m * E + i] = hs[(long long)m * E + i];
      }
    }
  }
  __syncthreads();
  // LN_RW weight rows per wave, streamed together (independent loads in flight), against every activation row
  if (n0 >= N) return;
  for (int m = 0; m < M; ++m) {
    float accs[LN_RW];
#pragma unroll
    for (int u = 0; u < LN_RW; ++u) accs[u] = 0.f;
    const T* xr = hs + (long long)m * E;
    if (vec) {
      constexpr int PER = 16 / (int)sizeof(T);
      int k = lane * PER;
      if constexpr (PREF) {  // the steps fetched ahead
#pragma unroll
        for (int it = 0; it < LN_PF; ++it) {
          if (k < E) {
            float xv[8];
            load8<T>(xr + k, xv);
#pragma unroll
            for (int u = 0; u < LN_RW; ++u)
#pragma unroll
              for (int i = 0; i < 4; ++i)
                accs[u] += __uint_as_float(pre[it][u][i] << 16) * xv[2 * i] +
                           __uint_as_float(pre[it][u][i] & 0xffff0000u) * xv[2 * i + 1];
          }
          k += 64 * PER;
        }
      }
      for (; k < E; k += 64 * PER) {
        float xv[8], wv[LN_RW][8];
#pragma unroll
        for (int u = 0; u < LN_RW; ++u) {
          const T* w = W + (long long)min(n0 + u, N - 1) * E + k;
          if constexpr (PER == 8) {
            load8<T>(w, wv[u]);
          } else {
            const f32x4 t4 = *(const f32x4*)w;
            wv[u][0] = t4[0], wv[u][1] = t4[1], wv[u][2] = t4[2], wv[u][3] = t4[3];
          }
        }
        if constexpr (PER == 8) {
          load8<T>(xr + k, xv);
        } else {
          const f32x4 t4 = *(const f32x4*)(xr + k);
          xv[0] = t4[0], xv[1] = t4[1], xv[2] = t4[2], xv[3] = t4[3];
        }
#pragma unroll
        for (int u = 0; u < LN_RW; ++u)
#pragma unroll
          for (int i = 0; i < PER; ++i) accs[u] += wv[u][i] * xv[i];
      }
    } else {
      for (int k = lane; k < E; k += 64) {
        const float xv = ld(xr + k);
#pragma unroll
        for (int u = 0; u < LN_RW; ++u) accs[u] += ld(W + (long long)min(n0 + u, N - 1) * E + k) * xv;
      }
    }
#pragma unroll
    for (int u = 0; u < LN_RW; ++u) accs[u] = wave_sum(accs[u]);
#pragma unroll
    for (int u = 0; u < LN_RW; ++u) {
    const int n = n0 + u;
    float acc = accs[u];
    if (lane == 0 && n < N) {
      if (q.on) {
        if (n >= q.off_q && n < q.off_q + q.n_q) {
          if (q.coef != 0.f) acc *= 1.f + q.coef * logf(floorf((float)(q.pos[m] + 1) / (float)q.every) + 1.f);
        } else if (n >= q.off_k && n < q.off_k + q.n_k) {
          const int i = n - q.off_k, slot = q.slot[m];
          const long long blk = slot / q.bs, off = slot % q.bs;
          st((T*)q.kc + ((blk * q.G + i / q.D) * q.bs + off) * q.D + i % q.D, acc);
        } else if (n >= q.off_v && n < q.off_v + q.n_v) {
          const int i = n - q.off_v, slot = q.slot[m];
          const long long blk = slot / q.bs, off = slot % q.bs;
          st((T*)q.vc + ((blk * q.G + i / q.Dv) * q.bs + off) * q.Dv + i % q.Dv, acc);
        }
      }
      C[(long long)m * ldc + n] = acc;
    }
    }
  }
}
bool gemv_ln_supported(int M, int E, int f32) {
  return M > 0 && M <= 8 && E <= 256 * LN_XR && (long long)M * E * (f32 ? 4 : 2) <= LN_LDS_BYTES;
}
void gemv_ln(const float* x, int E, const float* nw, const float* nb, float eps, const void* W, int M, int N, float* C,
             int ldc, void* hout, const AttnParams* A, const StepRows* R, int f32, hipStream_t s) {
  check(gemv_ln_supported(M, E, f32) && x && nw && W && C && hout && N > 0 && ldc >= N, "gemv_ln: bad operands");
  QkvEpi q{};
  if (A) {
    check(R && R->pos && R->slot && A->kc && A->vc, "gemv_ln: attention epilogue without rows or pools");
    q = QkvEpi{1, A->off_q, A->H * A->D, A->off_k, A->G * A->D, A->off_v, A->G * A->Dv, A->G, A->D, A->Dv, R->bs,
               A->qtemp_coef, A->qtemp_every, R->pos, R->slot, A->kc, A->vc};
  }
  dim3 grid((N + 4 * LN_RW - 1) / (4 * LN_RW));
  if (f32)
    hipLaunchKernelGGL(gemv_ln_kernel<float>, grid, dim3(256), 0, s, x, E, nw, nb, eps, (const float*)W, M, N, C, ldc,
                       (float*)hout, q, (int)(E % 4 == 0 && ((uintptr_t)W & 15) == 0));
  else
    hipLaunchKernelGGL(gemv_ln_kernel<bf16>, grid, dim3(256), 0, s, x, E, nw, nb, eps, (const bf16*)W, M, N, C, ldc,
                       (bf16*)hout, q, (int)(E % 8 == 0 && ((uintptr_t)W & 15) == 0));
  launched("gemv_ln");
}

// ------------------------------------------------------------------------------------------------ FMA tile GEMM
// 64 x 64 output tile per block, K in steps of 16 through LDS, 4 x 4 outputs per thread; true float32
template <typename T>
__global__ __launch_bounds__(256) void gemm_fma_kernel(const T* __restrict__ A, int lda, const T* __restrict__ W, int M,
                                                       int N, int K, Epi e) {
  __shared__ float As[16][68];
  __shared__ float Ws[16][68];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int tx = tid & 15, ty = tid >> 4;
  float acc[4][4] = {};
  const int lr = tid >> 2, lk = (tid & 3) * 4;  // this thread stages row lr, k lk .. lk + 3 of both tiles
  for (int k0 = 0; k0 < K; k0 += 16) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + lk + j;
      As[lk + j][lr] = (m0 + lr < M && k < K) ? ld(A + (long long)(m0 + lr) * lda + k) : 0.f;
      Ws[lk + j][lr] = (n0 + lr < N && k < K) ? ld(W + (long long)(n0 + lr) * K + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
      if (m < M && n < N) epi_store(e, m, n, acc[i][j]);
    }
}

// ------------------------------------------------------------------------------------------------ MFMA tile GEMM
// bfloat16: (32 TM) x (32 TN) output tile per block of 4 waves (2 x 2), each wave TM x TN fragments of
// v_mfma_f32_32x32x16_bf16; K in steps of 32 through LDS (rows padded to 40 elements so the 16-byte
// fragment reads of 32 consecutive rows spread over the banks), the next step's global loads in flight
// while the current one is multiplied. K % 8 == 0 and 16-byte aligned rows (host-checked).
constexpr int MF_BK = 32, MF_LD = 40;
// Grouped form (routed experts): blockIdx.y walks a device-side table of row tiles {expert, first row, rows} over
// rows sorted by expert; the tile's weight matrix is W + expert * w_stride, row m of the tile reads activation
// row gather[m] / gdiv (or m itself) and writes output row m.
struct Group {
  const int* tiles;   // null: a plain product
  const int* ntiles;
  const int* gather;
  int gdiv;
  long long w_stride;
};
template <int TM, int TN>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(const bf16* __restrict__ A, int lda, const bf16* __restrict__ W,
                                                        int M, int N, int K, Epi e, Group G) {
  constexpr int BM = 64 * TM, BN = 64 * TN;
  __shared__ __attribute__((aligned(16))) uint16_t As[2][BM * MF_LD];
  __shared__ __attribute__((aligned(16))) uint16_t Ws[2][BN * MF_LD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * BN;
  if (G.tiles) {
    if ((int)blockIdx.y >= *G.ntiles) return;
    const int* t = G.tiles + 3 * blockIdx.y;
    W += (long long)t[0] * G.w_stride;
    m0 = t[1];
    M = t[1] + t[2];
  }
  const int fr = lane & 31, fq = lane >> 5;
  // staging: 4 threads per row (8 elements each), 64 rows per pass
  const int sr = tid >> 2, sk = (tid & 3) * 8;
  long long arow[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + sr + 64 * i;
    arow[i] = (G.gather && m < M) ? G.gather[m] / G.gdiv : m;
  }
  u32x4 ra[TM], rw[TN];
  auto fetch = [&](int k0) {
    const int k = k0 + sk;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = m0 + sr + 64 * i;
      ra[i] = (m < M && k < K) ? *(const u32x4*)(A + arow[i] * lda + k) : u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + sr + 64 * j;
      rw[j] = (n < N && k < K) ? *(const u32x4*)(W + (long long)n * K + k) : u32x4{0, 0, 0, 0};
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < TM; ++i) *(u32x4*)(&As[buf][(sr + 64 * i) * MF_LD + sk]) = ra[i];
#pragma unroll
    for (int j = 0; j < TN; ++j) *(u32x4*)(&Ws[buf][(sr + 64 * j) * MF_LD + sk]) = rw[j];
  };
  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  fetch(0);
  stage(0);
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += MF_BK) {
    const bool more = k0 + MF_BK < K;
    if (more) fetch(k0 + MF_BK);
#pragma unroll
    for (int kk = 0; kk < MF_BK / 16; ++kk) {
      bf16x8 a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        a[i] = *(const bf16x8*)(&As[buf][(wm * 32 * TM + 32 * i + fr) * MF_LD + kk * 16 + fq * 8]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        b[j] = *(const bf16x8*)(&Ws[buf][(wn * 32 * TN + 32 * j + fr) * MF_LD + kk * 16 + fq * 8]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
    if (more) stage(buf ^ 1);  // the other buffer's readers finished before the previous barrier
    __syncthreads();
    buf ^= 1;
  }
  // C fragment: column (weight row) = lane & 31, row (activation row) = (r & 3) + 8 (r >> 2) + 4 (lane >> 5)
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + wn * 32 * TN + 32 * j + fr;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 32 * TM + 32 * i + (r & 3) + 8 * (r >> 2) + 4 * fq;
        if (m < M && n < N) epi_store(e, m, n, acc[i][j][r]);
      }
    }
}

static int g_mfma = 1;
void set_gemm_mfma(int on) { g_mfma = on; }

int gemm_path(int M, int N, int K, int f32) {
  if (M <= 8) return 0;
  if (!f32 && g_mfma && K % 8 == 0) return 1;
  return 2;
}

void gemm(const GemmParams& P, hipStream_t s) {
  check(P.M > 0 && P.N > 0 && P.K > 0 && P.lda >= P.K && P.ldc >= P.N && P.A && P.W && P.C, "gemm: bad operands");
  Epi e{P.epi, P.C, P.ldc, P.mult, P.add, P.cap};
  int path = gemm_path(P.M, P.N, P.K, P.f32);
  if (path == 1 && !(vec_ok<bf16>(P.A, P.lda, P.K) && vec_ok<bf16>(P.W, P.K, P.K))) path = 2;
  if (path == 0) {
    dim3 grid((P.N + 3) / 4);
    if (P.f32) {
      const int v = vec_ok<float>(P.A, P.lda, P.K) && vec_ok<float>(P.W, P.K, P.K);
      hipLaunchKernelGGL(gemv_rows_kernel<float>, grid, dim3(256), 0, s, (const float*)P.A, P.lda, (const float*)P.W, P.M,
                         P.N, P.K, e, v);
    } else {
      const int v = vec_ok<bf16>(P.A, P.lda, P.K) && vec_ok<bf16>(P.W, P.K, P.K);
      hipLaunchKernelGGL(gemv_rows_kernel<bf16>, grid, dim3(256), 0, s, (const bf16*)P.A, P.lda, (const bf16*)P.W, P.M,
                         P.N, P.K, e, v);
    }
  } else if (path == 1) {
    // 128 x 128 tiles once they still fill the chip, else 64 x 64
    const long long big = (long long)((P.M + 127) / 128) * ((P.N + 127) / 128);
    if (big >= 256) {
      dim3 grid((P.N + 127) / 128, (P.M + 127) / 128);
      hipLaunchKernelGGL((gemm_mfma_kernel<2, 2>), grid, dim3(256), 0, s, (const bf16*)P.A, P.lda, (const bf16*)P.W, P.M,
                         P.N, P.K, e, Group{});
    } else {
      dim3 grid((P.N + 63) / 64, (P.M + 63) / 64);
      hipLaunchKernelGGL((gemm_mfma_kernel<1, 1>), grid, dim3(256), 0, s, (const bf16*)P.A, P.lda, (const bf16*)P.W, P.M,
                         P.N, P.K, e, Group{});
    }
  } else {
    dim3 grid((P.N + 63) / 64, (P.M + 63) / 64);
    if (P.f32)
      hipLaunchKernelGGL(gemm_fma_kernel<float>, grid, dim3(256), 0, s, (const float*)P.A, P.lda, (const float*)P.W, P.M,
                         P.N, P.K, e);
    else
      hipLaunchKernelGGL(gemm_fma_kernel<bf16>, grid, dim3(256), 0, s, (const bf16*)P.A, P.lda, (const bf16*)P.W, P.M, P.N,
                         P.K, e);
  }
  launched("gemm");
}

// ------------------------------------------------------------------------------------------------ embed / norm
template <typename T>
__global__ __launch_bounds__(256) void embed_kernel(const T* __restrict__ table, const int* __restrict__ tokens, int E,
                                                    int V, float* __restrict__ resid, float* __restrict__ x0,
                                                    float scale) {
  const int b = blockIdx.x;
  int t = tokens[b];
  t = t < 0 ? 0 : (t >= V ? V - 1 : t);
  for (int i = threadIdx.x; i < E; i += 256) {
    const float v = ld(table + (long long)t * E + i) * scale;
    resid[(long long)b * E + i] = v;
    x0[(long long)b * E + i] = v;
  }
}
void embed(const void* table, const int* tokens, int B, int E, int V, float* resid, float* x0, float scale, int f32,
           hipStream_t s) {
  check(B > 0 && table && tokens && resid && x0, "embed: bad operands");
  if (f32)
    hipLaunchKernelGGL(embed_kernel<float>, dim3(B), dim3(256), 0, s, (const float*)table, tokens, E, V, resid, x0, scale);
  else
    hipLaunchKernelGGL(embed_kernel<bf16>, dim3(B), dim3(256), 0, s, (const bf16*)table, tokens, E, V, resid, x0, scale);
  launched("embed");
}

// (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b, one block per row
template <typename T>
__global__ __launch_bounds__(256) void layer_norm_kernel(const float* __restrict__ x, const int* __restrict__ idx, int E,
                                                         const float* __restrict__ w, const float* __restrict__ b,
                                                         float eps, T* __restrict__ out) {
  __shared__ float red[4];
  const int r = blockIdx.x;
  const float* row = x + (long long)(idx ? idx[r] : r) * E;
  float sum = 0.f;
  for (int i = threadIdx.x; i < E; i += 256) sum += row[i];
  const float mean = block_sum256(sum, red) / (float)E;
  float sq = 0.f;
  for (int i = threadIdx.x; i < E; i += 256) {
    const float d = row[i] - mean;
    sq += d * d;
  }
  const float rstd = 1.f / sqrtf(block_sum256(sq, red) / (float)E + eps);
  for (int i = threadIdx.x; i < E; i += 256) st(out + (long long)r * E + i, (row[i] - mean) * rstd * w[i] + b[i]);
}
void layer_norm_cast(const float* x, const int* idx, int rows, int E, const float* w, const float* b, float eps, void* out,
                     int f32, hipStream_t s) {
  check(rows > 0 && x && w && b && out, "layer_norm: bad operands");
  if (f32)
    hipLaunchKernelGGL(layer_norm_kernel<float>, dim3(rows), dim3(256), 0, s, x, idx, E, w, b, eps, (float*)out);
  else
    hipLaunchKernelGGL(layer_norm_kernel<bf16>, dim3(rows), dim3(256), 0, s, x, idx, E, w, b, eps, (bf16*)out);
  launched("layer_norm");
}

template <typename T>
__global__ __launch_bounds__(256) void concat_kernel(const float* __restrict__ x, const float* __restrict__ x0, int E,
                                                     T* __restrict__ out) {
  const int r = blockIdx.x;
  for (int i = threadIdx.x; i < E; i += 256) {
    st(out + (long long)r * 2 * E + i, x[(long long)r * E + i]);
    st(out + (long long)r * 2 * E + E + i, x0[(long long)r * E + i]);
  }
}
void concat_cast(const float* x, const float* x0, int rows, int E, void* out, int f32, hipStream_t s) {
  check(rows > 0 && x && x0 && out, "concat: bad operands");
  if (f32)
    hipLaunchKernelGGL(concat_kernel<float>, dim3(rows), dim3(256), 0, s, x, x0, E, (float*)out);
  else
    hipLaunchKernelGGL(concat_kernel<bf16>, dim3(rows), dim3(256), 0, s, x, x0, E, (bf16*)out);
  launched("concat");
}

// ------------------------------------------------------------------------------------------------ attention
template <typename T>
__global__ __launch_bounds__(256) void attn_prepare_kernel(AttnParams P, StepRows R) {
  const int b = blockIdx.x;
  float* row = P.proj + (long long)b * P.ld;
  if (P.qtemp_coef != 0.f) {
    const float p1 = (float)(R.pos[b] + 1);
    const float temp = 1.f + P.qtemp_coef * logf(floorf(p1 / (float)P.qtemp_every) + 1.f);
    for (int i = threadIdx.x; i < P.H * P.D; i += 256) row[P.off_q + i] *= temp;
  }
  const int slot = R.slot[b];
  const long long blk = slot / R.bs, off = slot % R.bs;
  T* kc = (T*)P.kc;
  T* vc = (T*)P.vc;
  for (int i = threadIdx.x; i < P.G * P.D; i += 256) {
    const int g = i / P.D, d = i % P.D;
    st(kc + ((blk * P.G + g) * R.bs + off) * P.D + d, row[P.off_k + i]);
  }
  for (int i = threadIdx.x; i < P.G * P.Dv; i += 256) {
    const int g = i / P.Dv, d = i % P.Dv;
    st(vc + ((blk * P.G + g) * R.bs + off) * P.Dv + d, row[P.off_v + i]);
  }
}
void attn_prepare(const AttnParams& P, const StepRows& R, hipStream_t s) {
  check(R.B > 0 && P.proj && P.kc && P.vc, "attn_prepare: bad operands");
  if (P.f32)
    hipLaunchKernelGGL(attn_prepare_kernel<float>, dim3(R.B), dim3(256), 0, s, P, R);
  else
    hipLaunchKernelGGL(attn_prepare_kernel<bf16>, dim3(R.B), dim3(256), 0, s, P, R);
  launched("attn_prepare");
}

// One wave per (row, key/value head, batch of up to RQ query heads that share it). Keys go by in groups of 64:
// lane j reads the K row of key t0 + j once (16-byte loads) and scores it against every query head of the
// batch; each head keeps a running maximum and sum; every lane owns value dims lane, lane + 64, ... of every
// head's output, and a V row is read once for all of them.
constexpr int ATT_MAXD = 256;
constexpr int ATT_MAXD_DECODE = 1024;  // the block-per-(row, head) kernel keeps one query in LDS: wide shared key rows fit
template <typename T>
__device__ __forceinline__ void load8(const T* p, float* out);
template <>
__device__ __forceinline__ void load8<bf16>(const bf16* p, float* out) {
  const u32x4 a = *(const u32x4*)p;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    out[2 * i] = __uint_as_float(a[i] << 16);
    out[2 * i + 1] = __uint_as_float(a[i] & 0xffff0000u);
  }
}
template <>
__device__ __forceinline__ void load8<float>(const float* p, float* out) {
  const f32x4 a = *(const f32x4*)p, b = *(const f32x4*)(p + 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    out[i] = a[i];
    out[4 + i] = b[i];
  }
}
// DC = ceil(Dv / 64) value dims per lane. SPLIT: the block's four waves share ONE item and take the 64-key groups
// in turn (few rows: decode steps), merging their running maxima, sums and outputs through LDS at the end;
// otherwise every wave has its own item (prompt portions).
template <typename T, int RQ, int DC, bool SPLIT>
__global__ __launch_bounds__(256) void attention_kernel(AttnParams P, StepRows R, int nbatch, int vec) {
  __shared__ __attribute__((aligned(16))) float qs[SPLIT ? 1 : 4][RQ][ATT_MAXD];
  __shared__ float mg[SPLIT ? 4 : 1][RQ][2];
  __shared__ float ag[SPLIT ? 4 : 1][RQ][SPLIT ? DC * 64 : 1];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int qw = SPLIT ? 0 : wv;
  const int item = SPLIT ? blockIdx.x : blockIdx.x * 4 + wv;
  const bool live = item < R.B * P.G * nbatch;
  const int b = live ? item / (P.G * nbatch) : 0;
  const int g = live ? (item / nbatch) % P.G : 0;
  const int hb = live ? item % nbatch : 0;
  const int per = P.H / P.G;
  const int h0 = g * per + hb * RQ;            // first query head of this batch
  const int nr = min(RQ, per - hb * RQ);       // heads in it
  if (!SPLIT || wv == 0) {
#pragma unroll
    for (int r = 0; r < RQ; ++r)
      for (int d = lane; d < P.D; d += 64)
        qs[qw][r][d] = (live && r < nr) ? P.proj[(long long)b * P.ld + P.off_q + (h0 + r) * P.D + d] : 0.f;
  }
  __syncthreads();
  if (!live) return;  // SPLIT: uniform over the block
  const int n = R.q_len[b];
  const int* bt = R.block_table + (long long)R.q_seq[b] * R.max_blocks;
  const T* kc = (const T*)P.kc;
  const T* vc = (const T*)P.vc;
  const long long ldk = P.ldk ? P.ldk : P.D, ldv = P.ldv ? P.ldv : P.Dv;  // row strides of the pools
  float m[RQ], l[RQ], acc[RQ][DC];
#pragma unroll
  for (int r = 0; r < RQ; ++r) {
    m[r] = -INFINITY;
    l[r] = 0.f;
#pragma unroll
    for (int c = 0; c < DC; ++c) acc[r][c] = 0.f;
  }
  const int lo = P.window > 0 ? max(0, n - P.window) : 0;  // sliding window: the keys lo .. n - 1
  for (int t0 = lo + (SPLIT ? 64 * wv : 0); t0 < n; t0 += SPLIT ? 256 : 64) {
    const int t = t0 + lane;
    const bool valid = t < n;
    int rowidx = 0;
    float dot[RQ];
#pragma unroll
    for (int r = 0; r < RQ; ++r) dot[r] = 0.f;
    if (valid) rowidx = (bt[t / R.bs] * P.G + g) * R.bs + t % R.bs;
    // the first UB keys' value rows are requested ahead of the K rows: one round trip brings both
    constexpr int UB = 64 / DC;
    float v0[UB][DC];
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      const T* vr = vc + (long long)__builtin_amdgcn_readlane(rowidx, u) * ldv;  // a key past the end: row 0, weight 0
#pragma unroll
      for (int c = 0; c < DC; ++c) v0[u][c] = (lane + 64 * c < P.Dv) ? ld(vr + lane + 64 * c) : 0.f;
    }
    if (valid) {
      const T* kr = kc + (long long)rowidx * ldk;
      if (vec) {
        for (int d0 = 0; d0 < P.D; d0 += 64) {  // 64 dims of the row in flight at a time
          float k8[8][8];
#pragma unroll
          for (int u = 0; u < 8; ++u) load8<T>(kr + min(d0 + 8 * u, P.D - 8), k8[u]);
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const int d = d0 + 8 * u;
            if (d < P.D) {
#pragma unroll
              for (int r = 0; r < RQ; ++r) {
                const f32x4 qa = *(const f32x4*)&qs[qw][r][d], qb = *(const f32x4*)&qs[qw][r][d + 4];
                dot[r] += qa[0] * k8[u][0] + qa[1] * k8[u][1] + qa[2] * k8[u][2] + qa[3] * k8[u][3] + qb[0] * k8[u][4] +
                          qb[1] * k8[u][5] + qb[2] * k8[u][6] + qb[3] * k8[u][7];
              }
            }
          }
        }
      } else {
        for (int d = 0; d < P.D; ++d) {
          const float kv = ld(kr + d);
#pragma unroll
          for (int r = 0; r < RQ; ++r) dot[r] += qs[qw][r][d] * kv;
        }
      }
    }
    float p[RQ];
#pragma unroll
    for (int r = 0; r < RQ; ++r) {
      float sc = -INFINITY;
      if (valid) {
        sc = dot[r] * P.scale;
        if (P.softcap != 0.f) sc = P.softcap * tanhf(sc / P.softcap);
      }
      const float mn = fmaxf(m[r], wave_max(sc));
      const float corr = expf(m[r] - mn);  // first group: exp(-inf) = 0
      p[r] = valid ? expf(sc - mn) : 0.f;
      l[r] = l[r] * corr + wave_sum(p[r]);
#pragma unroll
      for (int c = 0; c < DC; ++c) acc[r][c] *= corr;
      m[r] = mn;
    }
    const int cnt = min(64, n - t0);
#pragma unroll
    for (int u = 0; u < UB; ++u)
#pragma unroll
      for (int r = 0; r < RQ; ++r) {
        const float pj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p[r]), u));  // 0 for keys past the end
#pragma unroll
        for (int c = 0; c < DC; ++c) acc[r][c] += pj * v0[u][c];
      }
    for (int j0 = UB; j0 < cnt; j0 += UB) {  // wide values: the rest of the group, UB rows in flight at a time
      float v[UB][DC];
#pragma unroll
      for (int u = 0; u < UB; ++u) {
        const T* vr = vc + (long long)__builtin_amdgcn_readlane(rowidx, j0 + u) * ldv;
#pragma unroll
        for (int c = 0; c < DC; ++c) v[u][c] = (lane + 64 * c < P.Dv) ? ld(vr + lane + 64 * c) : 0.f;
      }
#pragma unroll
      for (int u = 0; u < UB; ++u)
#pragma unroll
        for (int r = 0; r < RQ; ++r) {
          const float pj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p[r]), j0 + u));
#pragma unroll
          for (int c = 0; c < DC; ++c) acc[r][c] += pj * v[u][c];
        }
    }
  }
  if (SPLIT) {
#pragma unroll
    for (int r = 0; r < RQ; ++r) {
      if (lane == 0) {
        mg[wv][r][0] = m[r];
        mg[wv][r][1] = l[r];
      }
#pragma unroll
      for (int c = 0; c < DC; ++c) ag[wv][r][lane + 64 * c] = acc[r][c];
    }
    __syncthreads();
    if (wv != 0) return;
#pragma unroll
    for (int r = 0; r < RQ; ++r) {
      float M = -INFINITY;
      for (int w = 0; w < 4; ++w) M = fmaxf(M, mg[w][r][0]);
      float L = 0.f;
#pragma unroll
      for (int c = 0; c < DC; ++c) acc[r][c] = 0.f;
      for (int w = 0; w < 4; ++w) {
        const float f = expf(mg[w][r][0] - M);  // a wave without keys: exp(-inf) = 0
        L += mg[w][r][1] * f;
#pragma unroll
        for (int c = 0; c < DC; ++c) acc[r][c] += ag[w][r][lane + 64 * c] * f;
      }
      l[r] = L;
      m[r] = M;
    }
  }
#pragma unroll
  for (int r = 0; r < RQ; ++r) {
    if (r < nr) {
      T* out = (T*)P.out + (long long)b * P.ld_out + (h0 + r) * P.Dv;
      if (P.sink) l[r] += expf(P.sink[h0 + r] - m[r]);  // the sink: a term of the denominator without key or value
      const float inv = 1.f / l[r];
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const int d = lane + 64 * c;
        if (d < P.Dv) st(out + d, acc[r][c] * inv);
      }
    }
  }
}
// ---- decode steps: one block per (row, query head); its four waves take the 64-key groups in turn and merge
// through LDS. Within a group lane j scores key j (its own K row against the query in LDS); for the values the
// lanes regroup as (key quarter kq, dim group dq): lane (kq, dq) walks 16 keys for DPL consecutive value dims
// (weights and row indices come from LDS), so a group costs 16 short iterations instead of 64, and the four
// quarters meet in two lane exchanges. The serial instruction count per wave is what bounds a decode step.
template <typename T, int DPL>
__global__ __launch_bounds__(256) void attention_decode_kernel(AttnParams P, StepRows R, int vec, int vvec, int nsplit) {
  __shared__ __attribute__((aligned(16))) float qs[ATT_MAXD_DECODE];
  __shared__ float ps[4][64];
  __shared__ int rs[4][64];
  __shared__ float mg[4][2];
  __shared__ float ag[4][16 * DPL];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  // output "heads": with vheads = G every (query head, value head) pair, else one per query head
  const int vh = P.vheads > 1 ? P.vheads : 1, NH = P.H * vh;
  const int b = blockIdx.x / NH, oh = blockIdx.x % NH, h = oh / vh;
  const int g = h / (P.H / P.G);
  const int gv = vh > 1 ? oh % vh : g;           // the value head this output meets
  const int KG = P.kshared ? 1 : P.G, kg = P.kshared ? 0 : g;  // a shared key row: the K pool has one head
  const int koff = P.maps > 1 ? (h % P.maps) * P.D : 0;      // several maps per head sit side by side in a K row
  const int split = blockIdx.y;  // long contexts: blockIdx.y-th of nsplit blocks, 64-key groups dealt round robin
  for (int d = threadIdx.x; d < P.D; d += 256) qs[d] = P.proj[(long long)b * P.ld + P.off_q + h * P.D + d];
  const int n = R.q_len[b];
  const int* bt = R.block_table + (long long)R.q_seq[b] * R.max_blocks;
  const T* kc = (const T*)P.kc;
  const T* vc = (const T*)P.vc;
  const long long ldk = P.ldk ? P.ldk : P.D, ldv = P.ldv ? P.ldv : P.Dv;
  const int kq = lane >> 4, dq = lane & 15;
  float m = -INFINITY, l = 0.f, acc[DPL];
#pragma unroll
  for (int c = 0; c < DPL; ++c) acc[c] = 0.f;
  __syncthreads();
  const int lo = P.window > 0 ? max(0, n - P.window) : 0;  // sliding window: the keys lo .. n - 1
  for (int t0 = lo + 64 * (split * 4 + wv); t0 < n; t0 += 256 * nsplit) {
    const int t = t0 + lane;
    const bool valid = t < n;
    int rowidx = 0;
    float dot = 0.f;
    if (valid) {
      const int blk = bt[t / R.bs];
      rowidx = (blk * P.G + gv) * R.bs + t % R.bs;  // the value's row; the key's may sit in a pool of another shape
      const T* kr = kc + (long long)((blk * KG + kg) * R.bs + t % R.bs) * ldk + koff;
      if (vec) {
        for (int d0 = 0; d0 < P.D; d0 += 64) {
          float k8[8][8];
#pragma unroll
          for (int u = 0; u < 8; ++u) load8<T>(kr + min(d0 + 8 * u, P.D - 8), k8[u]);
#pragma unroll
          for (int u = 0; u < 8; ++u) {
            const int d = d0 + 8 * u;
            if (d < P.D) {
              const f32x4 qa = *(const f32x4*)&qs[d], qb = *(const f32x4*)&qs[d + 4];
              dot += qa[0] * k8[u][0] + qa[1] * k8[u][1] + qa[2] * k8[u][2] + qa[3] * k8[u][3] + qb[0] * k8[u][4] +
                     qb[1] * k8[u][5] + qb[2] * k8[u][6] + qb[3] * k8[u][7];
            }
          }
        }
      } else {
        for (int d = 0; d < P.D; ++d) dot += qs[d] * ld(kr + d);
      }
    }
    float sc = -INFINITY;
    if (valid) {
      sc = dot * P.scale;
      if (P.softcap != 0.f) sc = P.softcap * tanhf(sc / P.softcap);
    }
    const float mn = fmaxf(m, wave_max(sc));
    const float corr = expf(m - mn);
    const float p = valid ? expf(sc - mn) : 0.f;
    l = l * corr + wave_sum(p);
    m = mn;
    ps[wv][lane] = p;
    rs[wv][lane] = valid ? rowidx : 0;  // a key past the end: row 0 with weight 0
#pragma unroll
    for (int c = 0; c < DPL; ++c) acc[c] *= corr;
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): this wave's LDS writes have landed
    float v[16][DPL];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const T* vr = vc + (long long)rs[wv][kq * 16 + i] * ldv + dq * DPL;
      if (vvec) {
        if (dq * DPL < P.Dv) {
          if constexpr (DPL == 4 && sizeof(T) == 2) {
            const unsigned long long w = *(const unsigned long long*)vr;
            v[i][0] = __uint_as_float((unsigned)(w << 16));
            v[i][1] = __uint_as_float((unsigned)w & 0xffff0000u);
            v[i][2] = __uint_as_float((unsigned)(w >> 16) & 0xffff0000u);
            v[i][3] = __uint_as_float((unsigned)(w >> 32) & 0xffff0000u);
          } else {
#pragma unroll
            for (int c8 = 0; c8 < DPL; c8 += 8) load8<T>(vr + c8, &v[i][c8]);
          }
        } else {
#pragma unroll
          for (int c = 0; c < DPL; ++c) v[i][c] = 0.f;
        }
      } else {
#pragma unroll
        for (int c = 0; c < DPL; ++c) v[i][c] = (dq * DPL + c < P.Dv) ? ld(vr + c) : 0.f;
      }
    }
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float pj = ps[wv][kq * 16 + i];
#pragma unroll
      for (int c = 0; c < DPL; ++c) acc[c] += pj * v[i][c];
    }
    __builtin_amdgcn_wave_barrier();
  }
  // the four key quarters of the wave, then the four waves of the block
#pragma unroll
  for (int c = 0; c < DPL; ++c) {
    acc[c] += xor_shfl<16>(acc[c]);
    acc[c] += xor_shfl<32>(acc[c]);
  }
  if (lane == 0) {
    mg[wv][0] = m;
    mg[wv][1] = l;
  }
  if (kq == 0) {
#pragma unroll
    for (int c = 0; c < DPL; ++c) ag[wv][dq * DPL + c] = acc[c];
  }
  __syncthreads();
  if (wv != 0 || kq != 0) return;
  float M = -INFINITY;
  for (int w = 0; w < 4; ++w) M = fmaxf(M, mg[w][0]);
  float L = 0.f;
#pragma unroll
  for (int c = 0; c < DPL; ++c) acc[c] = 0.f;
  for (int w = 0; w < 4; ++w) {
    // a wave without keys has maximum -inf and weighs nothing; a block without keys (a short row beside a long
    // one, split the same number of ways) has M = -inf too, and -inf - -inf must not become a NaN
    const float f = mg[w][0] == -INFINITY ? 0.f : expf(mg[w][0] - M);
    L += mg[w][1] * f;
#pragma unroll
    for (int c = 0; c < DPL; ++c) acc[c] += ag[w][dq * DPL + c] * f;
  }
  if (nsplit > 1) {  // partial {maximum, sum, un-normalised output}; attention_merge_kernel finishes the row
    float* w = P.split_ws + ((long long)blockIdx.x * nsplit + split) * (P.Dv + 2);
    if (lane == 0) {
      w[0] = M;
      w[1] = L;
    }
#pragma unroll
    for (int c = 0; c < DPL; ++c)
      if (dq * DPL + c < P.Dv) w[2 + dq * DPL + c] = acc[c];
    return;
  }
  if (P.sink) L += expf(P.sink[h] - M);
  const float inv = 1.f / L;
  if (P.out32) {
    float* out = P.out32 + (long long)b * P.ld_out32 + oh * P.Dv;
#pragma unroll
    for (int c = 0; c < DPL; ++c)
      if (dq * DPL + c < P.Dv) out[dq * DPL + c] = acc[c] * inv;
    return;
  }
  T* out = (T*)P.out + (long long)b * P.ld_out + oh * P.Dv;
#pragma unroll
  for (int c = 0; c < DPL; ++c)
    if (dq * DPL + c < P.Dv) st(out + dq * DPL + c, acc[c] * inv);
}
// one wave per (row, head): the nsplit partials of a long context into the output
template <typename T>
__global__ __launch_bounds__(256) void attention_merge_kernel(AttnParams P, int items, int nsplit) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= items) return;
  const float* w = P.split_ws + (long long)item * nsplit * (P.Dv + 2);
  float M = -INFINITY;
  for (int sidx = 0; sidx < nsplit; ++sidx) M = fmaxf(M, w[(long long)sidx * (P.Dv + 2)]);
  float L = 0.f;
  for (int sidx = 0; sidx < nsplit; ++sidx) {
    const float ms = w[(long long)sidx * (P.Dv + 2)];
    if (ms != -INFINITY) L += w[(long long)sidx * (P.Dv + 2) + 1] * expf(ms - M);  // a split without keys weighs nothing
  }
  const int vh = P.vheads > 1 ? P.vheads : 1, NH = P.H * vh;  // items are (row, output head)
  if (P.sink) L += expf(P.sink[(item % NH) / vh] - M);
  T* out = (T*)P.out + (long long)(item / NH) * P.ld_out + (item % NH) * P.Dv;
  float* out32 = P.out32 ? P.out32 + (long long)(item / NH) * P.ld_out32 + (item % NH) * P.Dv : nullptr;
  for (int d = lane; d < P.Dv; d += 64) {
    float o = 0.f;
    for (int sidx = 0; sidx < nsplit; ++sidx) {
      const float ms = w[(long long)sidx * (P.Dv + 2)];
      if (ms != -INFINITY) o += w[(long long)sidx * (P.Dv + 2) + 2 + d] * expf(ms - M);
    }
    if (out32)
      out32[d] = o / L;
    else
      st(out + d, o / L);
  }
}
template <typename T>
static void launch_attention_decode(const AttnParams& P, const StepRows& R, hipStream_t s) {
  const int ldk = P.ldk ? P.ldk : P.D, ldv = P.ldv ? P.ldv : P.Dv;
  const int vec = P.D % 8 == 0 && ldk % 8 == 0 && ((uintptr_t)P.kc & 15) == 0;  // (a map's offset is a multiple of D)
  const int NH = P.H * (P.vheads > 1 ? P.vheads : 1);
  const int ns = (P.nsplit > 1 && P.split_ws && (long long)R.B * NH * P.nsplit * (P.Dv + 2) <= P.split_ws_floats) ? P.nsplit : 1;
  dim3 grid(R.B * NH, ns);
  const int per = 16 / (int)sizeof(T);  // elements of a 16-byte load
  if (P.Dv <= 64) {
    const int vvec = P.Dv % 4 == 0 && ldv % 4 == 0 && (sizeof(T) == 2 ? 1 : 0) && ((uintptr_t)P.vc & 15) == 0;  // 8-byte pieces (bf16)
    hipLaunchKernelGGL((attention_decode_kernel<T, 4>), grid, dim3(256), 0, s, P, R, vec, sizeof(T) == 2 ? vvec : 0, ns);
  } else if (P.Dv <= 128) {
    const int vvec = P.Dv % 8 == 0 && ldv % 8 == 0 && ((uintptr_t)P.vc & 15) == 0 && per <= 8;
    hipLaunchKernelGGL((attention_decode_kernel<T, 8>), grid, dim3(256), 0, s, P, R, vec, vvec, ns);
  } else {
    const int vvec = P.Dv % 16 == 0 && ldv % 8 == 0 && ((uintptr_t)P.vc & 15) == 0 && per <= 8;
    hipLaunchKernelGGL((attention_decode_kernel<T, 16>), grid, dim3(256), 0, s, P, R, vec, vvec, ns);
  }
  if (ns > 1)
    hipLaunchKernelGGL(attention_merge_kernel<T>, dim3((R.B * NH + 3) / 4), dim3(256), 0, s, P, R.B * NH, ns);
}

template <typename T, int RQ, int DC>
static void launch_attention_rd(const AttnParams& P, const StepRows& R, int nbatch, int vec, hipStream_t s) {
  const int items = R.B * P.G * nbatch;
  if (items < 512)
    hipLaunchKernelGGL((attention_kernel<T, RQ, DC, true>), dim3(items), dim3(256), 0, s, P, R, nbatch, vec);
  else
    hipLaunchKernelGGL((attention_kernel<T, RQ, DC, false>), dim3((items + 3) / 4), dim3(256), 0, s, P, R, nbatch, vec);
}
template <typename T, int RQ>
static void launch_attention_r(const AttnParams& P, const StepRows& R, int nbatch, int vec, hipStream_t s) {
  if (P.Dv <= 64)
    launch_attention_rd<T, RQ, 1>(P, R, nbatch, vec, s);
  else if (P.Dv <= 128)
    launch_attention_rd<T, RQ, 2>(P, R, nbatch, vec, s);
  else
    launch_attention_rd<T, RQ, 4>(P, R, nbatch, vec, s);
}
template <typename T>
static void launch_attention(const AttnParams& P, const StepRows& R, hipStream_t s) {
  const int per = P.H / P.G;
  const int rq = per >= 4 ? 4 : per >= 2 ? 2 : 1;
  const int nbatch = (per + rq - 1) / rq;
  const int vec = P.D % 8 == 0 && (P.ldk ? P.ldk : P.D) % 8 == 0 && ((uintptr_t)P.kc & 15) == 0;
  if (rq == 4)
    launch_attention_r<T, 4>(P, R, nbatch, vec, s);
  else if (rq == 2)
    launch_attention_r<T, 2>(P, R, nbatch, vec, s);
  else
    launch_attention_r<T, 1>(P, R, nbatch, vec, s);
}
// ---- prompt portions on the matrix cores (bfloat16 K/V pools). One wave per (tile of up to 32 query rows of one
// sequence, query head); the host lists the tiles {first row, rows}. Keys go by 32 at a time:
//   S^T[key][q] = K Q^T      v_mfma_f32_32x32x16_bf16, A = K rows read straight from the pool (16-byte pieces),
//                            B = the tile's queries, kept in registers as bf16 high + low parts (two products,
//                            so the float32 queries keep ~16 bits of mantissa);
//   scale, cap, mask, running maximum and sum per query: lane (q, half) holds 16 keys of ITS query, so the
//                            softmax statistics are per-lane values plus one exchange between the two halves;
//   O^T[dv][q] += V^T P^T    A = V^T gathered from the wave's LDS copy of the 32 V rows, B = the weights, again
//                            as high + low bf16 parts; O^T keeps each lane's query in the lane, so the running
//                            rescale is a per-lane multiply.
// The K operand rows are loaded in the order key(m) = m with bits 2 and 3 swapped: the accumulator registers
// 0..7 / 8..15 of lane (q, half) then hold keys 8 half + 0..7 of the first / second 16-key group, which is the
// operand layout of the second product, so the weights never move between lanes.
constexpr int FL_LDV = 4;  // LDS row padding (elements): the two lane halves land in different banks
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned pack_bf(float a, float b) {  // round to nearest even (v_cvt_pk_bf16_f32)
  const bf16x2 v = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(unsigned, v);
}
// float32 exp and tanh on the transcendental unit (v_exp_f32, 1 ulp): the error stays below 1e-6 of the cap
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896341f); }
__device__ __forceinline__ float fast_tanh(float x) {
  const float e = __builtin_amdgcn_exp2f(fminf(x, 15.f) * 2.88539008177792681f);  // e^(2x)
  return 1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f);
}
template <int KD, int NV>
__global__ __launch_bounds__(64) void flash_prefill_kernel(AttnParams P, StepRows R, const int* __restrict__ tiles) {
  constexpr int D = 16 * KD, DV = 32 * NV, LDV = DV + FL_LDV;
  __shared__ __attribute__((aligned(16))) uint16_t Vl[32 * LDV];
  const int lane = threadIdx.x, q = lane & 31, hf = lane >> 5;
  const int row0 = tiles[2 * blockIdx.x], nrows = tiles[2 * blockIdx.x + 1];
  const int vh = P.vheads > 1 ? P.vheads : 1;  // output heads: (query head, value head) pairs with vheads = G
  const int oh = blockIdx.y, h = oh / vh, g = h / (P.H / P.G), gv = vh > 1 ? oh % vh : g;
  const int KG = P.kshared ? 1 : P.G, kg = P.kshared ? 0 : g;  // a shared key row: the K pool has one head
  const int koff = P.maps > 1 ? (h % P.maps) * D : 0;        // several maps per head sit side by side in a K row
  const int* bt = R.block_table + (long long)R.q_seq[row0] * R.max_blocks;
  const int qrow = row0 + min(q, nrows - 1);
  const int qlen = q < nrows ? R.q_len[qrow] : 0;
  const int kfirst = P.window > 0 ? qlen - P.window : 0;     // sliding window: this lane's query sees keys kfirst .. qlen - 1
  const int kmax = R.q_len[row0 + nrows - 1];
  const int kmin = P.window > 0 ? max(0, R.q_len[row0] - P.window) & ~31 : 0;  // the first key any row of the tile sees
  // queries: B operand, lane (q, hf) holds dims 16 kk + 8 hf + 0..7
  bf16x8 qhi[KD], qlo[KD];
  {
    const float* qp = P.proj + (long long)qrow * P.ld + P.off_q + h * D + 8 * hf;
#pragma unroll
    for (int kk = 0; kk < KD; ++kk) {
      const f32x4 a = *(const f32x4*)(qp + 16 * kk), b = *(const f32x4*)(qp + 16 * kk + 4);
      const float x[8] = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
      u32x4 hi, lo;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        hi[i] = pack_bf(x[2 * i], x[2 * i + 1]);
        lo[i] = pack_bf(x[2 * i] - __uint_as_float(hi[i] << 16), x[2 * i + 1] - __uint_as_float(hi[i] & 0xffff0000u));
      }
      qhi[kk] = __builtin_bit_cast(bf16x8, hi);
      qlo[kk] = __builtin_bit_cast(bf16x8, lo);
    }
  }
  const int m = lane & 31;
  const int kperm = (m & 0x13) | ((m & 4) << 1) | ((m & 8) >> 1);  // bits 2 and 3 swapped
  f32x16 o[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[j][r] = 0.f;
  float mi = -1e30f, li = 0.f;
  const float inv_cap = P.softcap != 0.f ? 1.f / P.softcap : 0.f;
  const uint16_t* kc = (const uint16_t*)P.kc;
  const uint16_t* vc = (const uint16_t*)P.vc;
  const long long ldk = P.ldk ? P.ldk : D, ldv = P.ldv ? P.ldv : DV;  // row strides of the pools
  // The K fragments and V rows of the NEXT key group are requested before the current group is multiplied, so a
  // group's global round trip passes behind the previous group's products and softmax.
  constexpr int CH = DV / 8;            // 16-byte pieces per V row
  constexpr int VPL = 32 * CH / 64;     // V pieces per lane per group
  u32x4 kf_n[KD], vs_n[VPL];
  auto fetch = [&](int t0) {
    {
      const int key = min(t0 + kperm, kmax - 1);
      const long long rowidx = (long long)(bt[key / R.bs] * KG + kg) * R.bs + key % R.bs;
      const uint16_t* kr = kc + rowidx * ldk + koff + 8 * hf;
#pragma unroll
      for (int kk = 0; kk < KD; ++kk) kf_n[kk] = *(const u32x4*)(kr + 16 * kk);
    }
#pragma unroll
    for (int i = 0; i < VPL; ++i) {  // keys past the end: the last key's row, their weights are zero
      const int c = lane + 64 * i;
      const int key = min(t0 + c / CH, kmax - 1), seg = c % CH;
      const long long rowidx = (long long)(bt[key / R.bs] * P.G + gv) * R.bs + key % R.bs;
      vs_n[i] = *(const u32x4*)(vc + rowidx * ldv + 8 * seg);
    }
  };
  fetch(kmin);
  for (int t0 = kmin; t0 < kmax; t0 += 32) {
    u32x4 kf_c[KD], vs_c[VPL];
#pragma unroll
    for (int kk = 0; kk < KD; ++kk) kf_c[kk] = kf_n[kk];
#pragma unroll
    for (int i = 0; i < VPL; ++i) vs_c[i] = vs_n[i];
    if (t0 + 32 < kmax) fetch(t0 + 32);
    // V rows of this key group into LDS
    __syncthreads();
#pragma unroll
    for (int i = 0; i < VPL; ++i) {
      const int c = lane + 64 * i;
      unsigned* dst = (unsigned*)&Vl[(c / CH) * LDV + 8 * (c % CH)];
      *(unsigned long long*)dst = (unsigned long long)vs_c[i][0] | ((unsigned long long)vs_c[i][1] << 32);
      *(unsigned long long*)(dst + 2) = (unsigned long long)vs_c[i][2] | ((unsigned long long)vs_c[i][3] << 32);
    }
    // S^T = K Q^T
    f32x16 sacc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
#pragma unroll
    for (int kk = 0; kk < KD; ++kk) {
      const bf16x8 kf = __builtin_bit_cast(bf16x8, kf_c[kk]);
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qhi[kk], sacc, 0, 0, 0);
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qlo[kk], sacc, 0, 0, 0);
    }
    // register r of lane (q, hf) is key t0 + 16 (r >> 3) + 8 hf + (r & 7)
    float pr[16];
    float mx = -1e30f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float sc = sacc[r] * P.scale;
      if (P.softcap != 0.f) sc = P.softcap * fast_tanh(sc * inv_cap);
      const int key = t0 + 16 * (r >> 3) + 8 * hf + (r & 7);
      const bool vis = key < qlen && key >= kfirst;
      pr[r] = vis ? sc : -1e30f;
      mx = fmaxf(mx, pr[r]);
    }
    mx = fmaxf(mx, xor_shfl<32>(mx));
    const float mn = fmaxf(mi, mx);
    const float corr = fast_exp(fmaxf(mi - mn, -100.f));
    float sum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      pr[r] = pr[r] > -1e29f ? fast_exp(pr[r] - mn) : 0.f;
      sum += pr[r];
    }
    sum += xor_shfl<32>(sum);
    li = li * corr + sum;
    mi = mn;
#pragma unroll
    for (int j = 0; j < NV; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[j][r] *= corr;
    bf16x8 phi[2], plo[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      u32x4 hi, lo;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float a = pr[8 * ks + 2 * i], b = pr[8 * ks + 2 * i + 1];
        hi[i] = pack_bf(a, b);
        lo[i] = pack_bf(a - __uint_as_float(hi[i] << 16), b - __uint_as_float(hi[i] & 0xffff0000u));
      }
      phi[ks] = __builtin_bit_cast(bf16x8, hi);
      plo[ks] = __builtin_bit_cast(bf16x8, lo);
    }
    __syncthreads();  // the V rows are in LDS
    // O^T += V^T P^T: A operand lane (dv = 32 j + m, hf) holds V[16 ks + 8 hf + i][dv], i = 0..7
#pragma unroll
    for (int j = 0; j < NV; ++j)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const uint16_t* vp = &Vl[(16 * ks + 8 * hf) * LDV + 32 * j + m];
        u32x4 vv;
#pragma unroll
        for (int i = 0; i < 4; ++i) vv[i] = (unsigned)vp[(2 * i) * LDV] | ((unsigned)vp[(2 * i + 1) * LDV] << 16);
        const bf16x8 vf = __builtin_bit_cast(bf16x8, vv);
        o[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, phi[ks], o[j], 0, 0, 0);
        o[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, plo[ks], o[j], 0, 0, 0);
      }
  }
  if (q < nrows) {  // register r of tile j: value dim 32 j + (r & 3) + 8 (r >> 2) + 4 hf of this lane's query
    if (P.sink) li += expf(P.sink[h] - mi);  // the sink: a term of the denominator without key or value
    const float inv = 1.f / li;
    if (P.out32) {
      float* out = P.out32 + (long long)qrow * P.ld_out32 + oh * DV;
#pragma unroll
      for (int j = 0; j < NV; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) out[32 * j + (r & 3) + 8 * (r >> 2) + 4 * hf] = o[j][r] * inv;
    } else {
      bf16* out = (bf16*)P.out + (long long)qrow * P.ld_out + oh * DV;
#pragma unroll
      for (int j = 0; j < NV; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) st(out + 32 * j + (r & 3) + 8 * (r >> 2) + 4 * hf, o[j][r] * inv);
    }
  }
}
// (key size / 16, value size / 32) the kernel is built for: equal key and value sizes 64 / 96 / 128, and the rows of
// latent attention (key = latent + shared rotated part, value = the latent)
#define FLASH_SHAPES(X) \
  X(4, 2) X(6, 3) X(8, 4) X(7, 3) X(8, 3) X(9, 4) X(10, 4) X(12, 5) X(14, 6) X(16, 6) X(16, 7) \
  X(2, 2) X(4, 4) X(12, 2) X(16, 2) X(16, 4)
bool flash_prefill_supported(const AttnParams& P) {
  bool shape = false;
#define FLASH_HAS(KD, NV) shape |= P.D == 16 * KD && P.Dv == 32 * NV;
  FLASH_SHAPES(FLASH_HAS)
#undef FLASH_HAS
  const int ldk = P.ldk ? P.ldk : P.D, ldv = P.ldv ? P.ldv : P.Dv;
  return !P.f32 && shape && ldk % 8 == 0 && ldv % 8 == 0 && (P.maps <= 1 || P.H % P.maps == 0) && P.ld % 4 == 0 &&
         P.off_q % 4 == 0 && (P.H * P.D) % 4 == 0 &&
         ((uintptr_t)P.proj & 15) == 0 && ((uintptr_t)P.kc & 15) == 0 && ((uintptr_t)P.vc & 15) == 0;
}
void flash_prefill(const AttnParams& P, const StepRows& R, const int* tiles, int ntiles, hipStream_t s) {
  check(flash_prefill_supported(P) && tiles && ntiles > 0 && P.G > 0 && P.H % P.G == 0 && (P.out || P.out32) &&
            (P.vheads <= 1 || P.vheads == P.G),
        "flash prefill: operands");
  dim3 grid(ntiles, P.H * (P.vheads > 1 ? P.vheads : 1));
#define FLASH_LAUNCH(KD, NV)                  \
  if (P.D == 16 * KD && P.Dv == 32 * NV)      \
    hipLaunchKernelGGL((flash_prefill_kernel<KD, NV>), grid, dim3(64), 0, s, P, R, tiles);
  FLASH_SHAPES(FLASH_LAUNCH)
#undef FLASH_LAUNCH
  launched("flash_prefill");
}
void attention(const AttnParams& P, const StepRows& R, hipStream_t s) {
  // a block per (row, head) serves decode steps (and short portions), float32 outputs, (query head, value head) pairs,
  // several maps per head and a shared key row (whose width may pass 256)
  const bool per_head = R.B * P.H <= 1024 || P.out32 || P.vheads > 1 || P.maps > 1 || P.kshared || P.D > ATT_MAXD;
  check(R.B > 0 && P.D > 0 && P.D <= (per_head ? ATT_MAXD_DECODE : ATT_MAXD) && P.Dv > 0 && P.Dv <= ATT_MAXD && P.G > 0 &&
            P.H % P.G == 0 && (P.out || P.out32) && (P.vheads <= 1 || P.vheads == P.G) && P.window >= 0 &&
            (P.maps <= 1 || P.H % (P.G * P.maps) == 0),
        "attention: head sizes up to 256 (a shared key row up to 1024), heads a multiple of key/value heads");
  if (per_head) {
    if (P.f32)
      launch_attention_decode<float>(P, R, s);
    else
      launch_attention_decode<bf16>(P, R, s);
  } else if (P.f32) {
    launch_attention<float>(P, R, s);
  } else {
    launch_attention<bf16>(P, R, s);
  }
  launched("attention");
}

// ------------------------------------------------------------------------------------------------ retention
// One block per (sequence segment of the step, head): the block of the segment's first row walks its rows in
// order. Thread (g, j) = (tid / Dv, tid % Dv) holds state elements S[i][j] for i = g, g + NG, ... in registers
// (NG = 256 / Dv thread groups), so the update S <- decay S + k v^T needs no communication and o = S^T q is a
// sum of NG partials per column. Rotation of q and k, k's 1/sqrt(D), the per-head unit RMS of o and the
// silu(g) gate are applied here; the state is read from and written back to its slot once per step.
template <typename T, int MAXI>
__global__ __launch_bounds__(256) void retention_kernel(RetParams P, StepRows R) {
  __shared__ float qs[256], ks[256], vs[256], po[256], red[4];
  const int r0 = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int seq = R.q_seq[r0];
  if (r0 > 0 && R.q_seq[r0 - 1] == seq) return;  // not the first row of its segment (uniform per block)
  const int D = P.D, Dv = P.Dv;
  const int NG = 256 / Dv;
  const int g = tid / Dv, j = tid % Dv;
  const bool act = g < NG;
  float S[MAXI];
  float* st_base = P.state + (((long long)seq * P.H + h) * D) * Dv;
#pragma unroll
  for (int ii = 0; ii < MAXI; ++ii) {
    const int i = g + ii * NG;
    S[ii] = (act && i < D) ? st_base[(long long)i * Dv + j] : 0.f;
  }
  const float dec = P.decay[h];
  const float kscale = 1.f / sqrtf((float)D);
  const int half = P.rot_dims / 2;
  for (int r = r0; r < R.B && R.q_seq[r] == seq; ++r) {
    const float* row = P.proj + (long long)r * P.ld;
    if (tid < D) {
      const float* q = row + P.off_q + h * D;
      const float* k = row + P.off_k + h * D;
      float qv = q[tid], kv = k[tid];
      if (tid < P.rot_dims) {
        const int i = tid < half ? tid : tid - half;
        const float ang = (float)R.pos[r] * P.inv_freq[i];
        const float c = cosf(ang), sn = sinf(ang);
        if (tid < half) {  // (u, v) -> (u cos - v sin, v cos + u sin), u = x[i], v = x[i + half]
          qv = q[tid] * c - q[tid + half] * sn;
          kv = k[tid] * c - k[tid + half] * sn;
        } else {
          qv = q[tid] * c + q[i] * sn;
          kv = k[tid] * c + k[i] * sn;
        }
      }
      qs[tid] = qv;
      ks[tid] = kv * kscale;
    }
    if (tid < Dv) vs[tid] = row[P.off_v + h * Dv + tid];
    __syncthreads();
    float part = 0.f;
    if (act) {
      const float vj = vs[j];
#pragma unroll
      for (int ii = 0; ii < MAXI; ++ii) {
        const int i = g + ii * NG;
        if (i < D) {
          S[ii] = dec * S[ii] + ks[i] * vj;
          part += S[ii] * qs[i];
        }
      }
    }
    po[tid] = part;
    __syncthreads();
    float o = 0.f;
    if (tid < Dv)
      for (int gg = 0; gg < NG; ++gg) o += po[gg * Dv + tid];
    const float ms = block_sum256(tid < Dv ? o * o : 0.f, red) / (float)Dv;
    if (tid < Dv) {
      const float gate = row[P.off_g + h * Dv + tid];
      st((T*)P.out + (long long)r * P.ld_out + h * Dv + tid, o / sqrtf(ms + P.eps) * silu(gate));
    }
    __syncthreads();
  }
#pragma unroll
  for (int ii = 0; ii < MAXI; ++ii) {
    const int i = g + ii * NG;
    if (act && i < D) st_base[(long long)i * Dv + j] = S[ii];
  }
}
// Prompt portions: the same recurrence in chunks of RC tokens. With g the head's decay, a chunk of n tokens that
// starts from state S computes, for its tokens t, s = 0 .. n - 1,
//   A[t][s] = (q_t . k_s) g^(t - s) for s <= t,   o_t = g^(t + 1) S^T q_t + sum_s A[t][s] v_s,
//   U = sum_s g^(n - 1 - s) k_s v_s^T,             S <- g^n S + U,
// all in float32 on the vector ALUs, in three launches over a host-built chunk table {first row, rows, state
// slot, flags (1: first chunk of its sequence's rows, 2: last)}:
//   1. every chunk's U, chunks in parallel                      (retention_u_kernel)
//   2. the scan S <- g^n S + U over each sequence's chunks, one thread per state element, which leaves every
//      chunk's incoming state and the sequence's final state    (retention_scan_kernel)
//   3. every chunk's outputs from its incoming state, in parallel (retention_out_kernel)
// then retention_finish_kernel applies the per-head unit RMS and the gate.
// Blocks of 1. and 3. take (chunk, head, 64 value columns); thread (g4, j) = (tid / 64, tid % 64).
constexpr int RC = 32;
// rotated q and scaled rotated k of the chunk's rows into LDS (rows past n and dims past D zero)
template <int MAXD, bool WITH_Q>
__device__ __forceinline__ void stage_qk(const RetParams& P, const StepRows& R, int row0, int cn, int h,
                                         float (*Qs)[MAXD], float (*Ks)[MAXD + 4]) {
  const int D = P.D, half = P.rot_dims / 2, tid = threadIdx.x;
  const float kscale = 1.f / sqrtf((float)D);
  constexpr int IT = RC * MAXD / 256;
  float qa[IT], qb[IT], ka[IT], kb[IT], ang[IT];
#pragma unroll
  for (int it = 0; it < IT; ++it) {  // every load first: one round trip for the chunk
    const int idx = tid + 256 * it;
    const int c = idx / MAXD, d = idx % MAXD;
    qa[it] = qb[it] = ka[it] = kb[it] = ang[it] = 0.f;
    if (c < cn && d < D) {
      const int r = row0 + c;
      const float* q = P.proj + (long long)r * P.ld + P.off_q + h * D;
      const float* k = P.proj + (long long)r * P.ld + P.off_k + h * D;
      ka[it] = k[d];
      if (WITH_Q) qa[it] = q[d];
      if (d < P.rot_dims) {
        const int pd = d < half ? d + half : d - half;
        kb[it] = k[pd];
        if (WITH_Q) qb[it] = q[pd];
        ang[it] = (float)R.pos[r] * P.inv_freq[d < half ? d : d - half];
      }
    }
  }
#pragma unroll
  for (int it = 0; it < IT; ++it) {
    const int idx = tid + 256 * it;
    const int c = idx / MAXD, d = idx % MAXD;
    float qv = qa[it], kv = ka[it];
    if (c < cn && d < P.rot_dims) {  // (u, v) -> (u cos - v sin, v cos + u sin), u the lower dim of the pair
      const float cs = cosf(ang[it]), sn = sinf(ang[it]);
      const float sg = d < half ? -1.f : 1.f;
      qv = qa[it] * cs + sg * qb[it] * sn;
      kv = ka[it] * cs + sg * kb[it] * sn;
    }
    if (WITH_Q) Qs[c][d] = qv;
    Ks[c][d] = kv * kscale;
  }
}
__device__ __forceinline__ void stage_v(const RetParams& P, int row0, int cn, int h, int jb, float (*Vs)[64]) {
  for (int idx = threadIdx.x; idx < RC * 64; idx += 256) {
    const int c = idx >> 6, jj = idx & 63;
    const int cc = jb * 64 + jj;
    Vs[c][jj] = (c < cn && cc < P.Dv) ? P.proj[(long long)(row0 + c) * P.ld + P.off_v + h * P.Dv + cc] : 0.f;
  }
}
template <int MAXD>
__global__ __launch_bounds__(256) void retention_u_kernel(RetParams P, StepRows R, const int* __restrict__ chunks,
                                                          float* __restrict__ U, long long u_stride, int NJ) {
  __shared__ __attribute__((aligned(16))) float Ks[RC][MAXD + 4];
  __shared__ float Vs[RC][64];
  __shared__ float pw[RC + 1];
  const int c = blockIdx.x, h = blockIdx.y / NJ, jb = blockIdx.y % NJ, tid = threadIdx.x;
  const int row0 = chunks[4 * c], cn = chunks[4 * c + 1];
  const int j = tid & 63, g4 = tid >> 6, col = jb * 64 + j;
  if (tid <= RC) pw[tid] = powf(P.decay[h], (float)tid);
  stage_qk<MAXD, false>(P, R, row0, cn, h, nullptr, Ks);
  stage_v(P, row0, cn, h, jb, Vs);
  __syncthreads();
  float u[MAXD / 4];
#pragma unroll
  for (int ii = 0; ii < MAXD / 4; ++ii) u[ii] = 0.f;
  for (int sx = 0; sx < cn; ++sx) {
    const float vv = Vs[sx][j] * pw[cn - 1 - sx];
#pragma unroll
    for (int ii = 0; ii < MAXD / 4; ++ii) u[ii] += Ks[sx][g4 + 4 * ii] * vv;
  }
  if (col < P.Dv) {
    float* out = U + c * u_stride + (long long)h * P.D * P.Dv;
#pragma unroll
    for (int ii = 0; ii < MAXD / 4; ++ii) {
      const int i = g4 + 4 * ii;
      if (i < P.D) out[(long long)i * P.Dv + col] = u[ii];
    }
  }
}
__global__ __launch_bounds__(256) void retention_scan_kernel(RetParams P, const int* __restrict__ chunks, int nchunks,
                                                             const float* __restrict__ U, float* __restrict__ Sin,
                                                             long long u_stride) {
  const long long e = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long per_head = (long long)P.D * P.Dv;
  if (e >= P.H * per_head) return;
  const float dec = P.decay[e / per_head];
  const float dfull = powf(dec, (float)RC);
  float S = 0.f;
  for (int c = 0; c < nchunks; ++c) {
    const int cn = chunks[4 * c + 1], slot = chunks[4 * c + 2], flags = chunks[4 * c + 3];
    float* st_e = P.state + (long long)slot * P.H * per_head + e;
    if (flags & 1) S = *st_e;
    Sin[c * u_stride + e] = S;
    S = (cn == RC ? dfull : powf(dec, (float)cn)) * S + U[c * u_stride + e];
    if (flags & 2) *st_e = S;
  }
}
template <int MAXD>
__global__ __launch_bounds__(256) void retention_out_kernel(RetParams P, StepRows R, const int* __restrict__ chunks,
                                                            const float* __restrict__ Sin, long long u_stride,
                                                            float* __restrict__ obuf, int ld_o, int NJ) {
  __shared__ __attribute__((aligned(16))) float Qs[RC][MAXD];
  __shared__ __attribute__((aligned(16))) float Ks[RC][MAXD + 4];
  __shared__ float Vs[RC][64];
  __shared__ float As[RC][RC + 1];
  __shared__ float pw[RC + 1];
  const int c = blockIdx.x, h = blockIdx.y / NJ, jb = blockIdx.y % NJ, tid = threadIdx.x;
  const int row0 = chunks[4 * c], cn = chunks[4 * c + 1];
  const int D = P.D, Dv = P.Dv;
  const int j = tid & 63, g4 = tid >> 6, col = jb * 64 + j;
  const bool colok = col < Dv;
  if (tid <= RC) pw[tid] = powf(P.decay[h], (float)tid);
  float S[MAXD];
  const float* sin_base = Sin + c * u_stride + (long long)h * D * Dv;
#pragma unroll
  for (int i = 0; i < MAXD; ++i) S[i] = (colok && i < D) ? sin_base[(long long)i * Dv + col] : 0.f;
  stage_qk<MAXD, true>(P, R, row0, cn, h, Qs, Ks);
  stage_v(P, row0, cn, h, jb, Vs);
  __syncthreads();
#pragma unroll
  for (int kx = 0; kx < RC * RC / 256; ++kx) {
    const int t = (tid >> 5) + 8 * kx, sx = tid & 31;
    float dot = 0.f;
    if (sx <= t) {
#pragma unroll
      for (int i4 = 0; i4 < MAXD / 4; ++i4) {
        const f32x4 qa = *(const f32x4*)&Qs[t][4 * i4], kb = *(const f32x4*)&Ks[sx][4 * i4];
        dot += qa[0] * kb[0] + qa[1] * kb[1] + qa[2] * kb[2] + qa[3] * kb[3];
      }
      dot *= pw[t - sx];
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
    for (int sx = 0; sx < RC; ++sx) intra += As[t][sx] * Vs[sx][j];  // As is zero above the diagonal
    if (colok) obuf[(long long)(row0 + t) * ld_o + h * Dv + col] = pw[t + 1] * inter + intra;
  }
}
// out = o / sqrt(mean_j(o^2) + eps) * silu(gate), one wave per (row, head)
template <typename T>
__global__ __launch_bounds__(256) void retention_finish_kernel(RetParams P, int B, const float* __restrict__ obuf,
                                                               int ld_o) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= B * P.H) return;
  const int b = item / P.H, h = item % P.H;
  const float* o = obuf + (long long)b * ld_o + h * P.Dv;
  float sq = 0.f;
  for (int jx = lane; jx < P.Dv; jx += 64) sq += o[jx] * o[jx];
  const float rs = 1.f / sqrtf(wave_sum(sq) / (float)P.Dv + P.eps);
  const float* gate = P.proj + (long long)b * P.ld + P.off_g + h * P.Dv;
  T* out = (T*)P.out + (long long)b * P.ld_out + h * P.Dv;
  for (int jx = lane; jx < P.Dv; jx += 64) st(out + jx, o[jx] * rs * silu(gate[jx]));
}
bool retention_chunk_supported(int D, int Dv) { return D > 0 && D <= 128 && Dv > 0 && Dv <= 256; }
void retention_chunked(const RetParams& P, const StepRows& R, const RetChunkWs& W, hipStream_t s) {
  check(R.B > 0 && P.proj && P.state && P.decay && P.out && W.obuf && W.ld_o >= P.H * P.Dv &&
            retention_chunk_supported(P.D, P.Dv),
        "chunked retention: dim <= 128, vdim <= 256");
  check(P.rot_dims % 2 == 0 && P.rot_dims <= P.D && (P.rot_dims == 0 || P.inv_freq), "retention: bad rotary dims");
  check(W.chunks && W.nchunks > 0 && W.U && W.Sin && W.u_stride >= (long long)P.H * P.D * P.Dv && W.nchunks <= W.max_chunks,
        "chunked retention: chunk table or workspace");
  const int NJ = (P.Dv + 63) / 64;
  dim3 grid(W.nchunks, P.H * NJ);
  if (P.D <= 64)
    hipLaunchKernelGGL(retention_u_kernel<64>, grid, dim3(256), 0, s, P, R, W.chunks, W.U, W.u_stride, NJ);
  else
    hipLaunchKernelGGL(retention_u_kernel<128>, grid, dim3(256), 0, s, P, R, W.chunks, W.U, W.u_stride, NJ);
  launched("retention_u");
  const long long elems = (long long)P.H * P.D * P.Dv;
  hipLaunchKernelGGL(retention_scan_kernel, dim3((unsigned)((elems + 255) / 256)), dim3(256), 0, s, P, W.chunks, W.nchunks, W.U,
                     W.Sin, W.u_stride);
  launched("retention_scan");
  if (P.D <= 64)
    hipLaunchKernelGGL(retention_out_kernel<64>, grid, dim3(256), 0, s, P, R, W.chunks, W.Sin, W.u_stride, W.obuf, W.ld_o, NJ);
  else
    hipLaunchKernelGGL(retention_out_kernel<128>, grid, dim3(256), 0, s, P, R, W.chunks, W.Sin, W.u_stride, W.obuf, W.ld_o, NJ);
  launched("retention_out");
  dim3 g2((R.B * P.H + 3) / 4);
  if (P.f32)
    hipLaunchKernelGGL(retention_finish_kernel<float>, g2, dim3(256), 0, s, P, R.B, W.obuf, W.ld_o);
  else
    hipLaunchKernelGGL(retention_finish_kernel<bf16>, g2, dim3(256), 0, s, P, R.B, W.obuf, W.ld_o);
  launched("retention_finish");
}
int retention_chunk_rows() { return RC; }

// Any head size up to RG_MAX: the state stays in global memory, thread j walks column j of it (reads and writes
// of a row of S are contiguous across threads). Slow, and only taken when the register kernels do not fit.
constexpr int RG_MAX = 1024;
template <typename T>
__global__ __launch_bounds__(256) void retention_general_kernel(RetParams P, StepRows R) {
  __shared__ float qs[RG_MAX], ks[RG_MAX], os[RG_MAX], red[4];
  const int r0 = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int seq = R.q_seq[r0];
  if (r0 > 0 && R.q_seq[r0 - 1] == seq) return;
  const int D = P.D, Dv = P.Dv, half = P.rot_dims / 2;
  float* S = P.state + (((long long)seq * P.H + h) * D) * Dv;
  const float dec = P.decay[h], kscale = 1.f / sqrtf((float)D);
  for (int r = r0; r < R.B && R.q_seq[r] == seq; ++r) {
    const float* row = P.proj + (long long)r * P.ld;
    for (int d = tid; d < D; d += 256) {
      const float* q = row + P.off_q + h * D;
      const float* k = row + P.off_k + h * D;
      float qv = q[d], kv = k[d];
      if (d < P.rot_dims) {
        const int i = d < half ? d : d - half;
        const float ang = (float)R.pos[r] * P.inv_freq[i];
        const float c = cosf(ang), sn = sinf(ang);
        const float sg = d < half ? -1.f : 1.f;
        const int pd = d < half ? d + half : d - half;
        qv = q[d] * c + sg * q[pd] * sn;
        kv = k[d] * c + sg * k[pd] * sn;
      }
      qs[d] = qv;
      ks[d] = kv * kscale;
    }
    __syncthreads();
    float sq = 0.f;
    for (int j = tid; j < Dv; j += 256) {
      const float vj = row[P.off_v + h * Dv + j];
      float o = 0.f;
      for (int i = 0; i < D; ++i) {
        const float sv = dec * S[(long long)i * Dv + j] + ks[i] * vj;
        S[(long long)i * Dv + j] = sv;
        o += sv * qs[i];
      }
      os[j] = o;
      sq += o * o;
    }
    const float ms = block_sum256(sq, red) / (float)Dv;
    for (int j = tid; j < Dv; j += 256)
      st((T*)P.out + (long long)r * P.ld_out + h * Dv + j, os[j] / sqrtf(ms + P.eps) * silu(row[P.off_g + h * Dv + j]));
    __syncthreads();
  }
}
bool retention_general_supported(int D, int Dv) { return D > 0 && Dv > 0 && D <= RG_MAX && Dv <= RG_MAX; }

bool retention_supported(int D, int Dv) {
  if (D <= 0 || Dv <= 0 || D > 256 || Dv > 256) return false;
  const int ng = 256 / Dv;
  return (D + ng - 1) / ng <= 64;
}
template <typename T>
static void launch_retention(const RetParams& P, const StepRows& R, hipStream_t s) {
  const int ng = 256 / P.Dv, ni = (P.D + ng - 1) / ng;
  dim3 grid(R.B, P.H);
  if (ni <= 8)
    hipLaunchKernelGGL((retention_kernel<T, 8>), grid, dim3(256), 0, s, P, R);
  else if (ni <= 16)
    hipLaunchKernelGGL((retention_kernel<T, 16>), grid, dim3(256), 0, s, P, R);
  else if (ni <= 32)
    hipLaunchKernelGGL((retention_kernel<T, 32>), grid, dim3(256), 0, s, P, R);
  else
    hipLaunchKernelGGL((retention_kernel<T, 64>), grid, dim3(256), 0, s, P, R);
}
void retention(const RetParams& P, const StepRows& R, hipStream_t s) {
  check(R.B > 0 && P.proj && P.state && P.decay && P.out && (retention_supported(P.D, P.Dv) ||
        retention_general_supported(P.D, P.Dv)), "retention: head sizes up to 1024");
  check(P.rot_dims % 2 == 0 && P.rot_dims <= P.D && (P.rot_dims == 0 || P.inv_freq), "retention: bad rotary dims");
  if (!retention_supported(P.D, P.Dv)) {
    dim3 grid(R.B, P.H);
    if (P.f32)
      hipLaunchKernelGGL(retention_general_kernel<float>, grid, dim3(256), 0, s, P, R);
    else
      hipLaunchKernelGGL(retention_general_kernel<bf16>, grid, dim3(256), 0, s, P, R);
    launched("retention_general");
    return;
  }
  if (P.f32)
    launch_retention<float>(P, R, s);
  else
    launch_retention<bf16>(P, R, s);
  launched("retention");
}

// ------------------------------------------------------------------------------------------------ routed FFN
// per row: the `top` largest router logits (ties: the lower expert), softmax over them; the shared expert's
// scalar gate and its activation silu(gate) * up from the input projection's columns
template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(MoeParams P) {
  const int b = blockIdx.x;
  const float* row = P.proj + (long long)b * P.ld;
  if (threadIdx.x == 0) {
    int ids[MOE_MAX_TOP];
    float val[MOE_MAX_TOP];
    for (int jj = 0; jj < P.top; ++jj) {
      int best = -1;
      float bv = -INFINITY;
      for (int e = 0; e < P.X; ++e) {
        bool taken = false;
        for (int q = 0; q < jj; ++q) taken |= ids[q] == e;
        if (taken) continue;
        const float z = row[P.off_router + e] + P.router_b[e];
        if (best < 0 || z > bv) {
          best = e;
          bv = z;
        }
      }
      ids[jj] = best;
      val[jj] = bv;
    }
    const float mx = val[0];  // picked first: the largest
    float sum = 0.f;
    for (int jj = 0; jj < P.top; ++jj) {
      val[jj] = expf(val[jj] - mx);
      sum += val[jj];
    }
    for (int jj = 0; jj < P.top; ++jj) {
      P.eids[(long long)b * P.ld_top + jj] = ids[jj];
      P.ew[(long long)b * P.ld_top + jj] = val[jj] / sum;
    }
    if (P.Fs > 0) P.sgate[b] = sigmoidf(row[P.off_sg]);
  }
  T* hm = (T*)P.hmid + (long long)b * P.ld_hmid + P.top * P.F;
  for (int f = threadIdx.x; f < P.Fs; f += 256) st(hm + f, silu(row[P.off_sgate + f]) * row[P.off_sup + f]);
}
// one wave per (row, routed expert, ff unit): gate and up rows of that expert meet the row's activations
template <typename T>
__global__ __launch_bounds__(256) void moe_experts_kernel(MoeParams P, int vec) {
  const int lane = threadIdx.x & 63;
  const int f = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int b = blockIdx.y / P.top, jj = blockIdx.y % P.top;
  if (f >= P.F) return;
  const int e = P.eids[(long long)b * P.ld_top + jj];
  const T* x = (const T*)P.h + (long long)b * P.E;
  const T* wg = (const T*)P.w_gu + ((long long)e * 2 * P.F + f) * P.E;
  const T* wu = wg + (long long)P.F * P.E;
  const float gate = wave_dot<T>(wg, x, P.E, lane, vec != 0);
  const float up = wave_dot<T>(wu, x, P.E, lane, vec != 0);
  if (lane == 0) st((T*)P.hmid + (long long)b * P.ld_hmid + jj * P.F + f, silu(gate) * up);
}
// one wave per (row, output unit): the routed experts' down rows in routing order, then the shared expert's
template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(MoeParams P, int vec, int vec_s) {
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int b = blockIdx.y;
  if (n >= P.E) return;
  const T* hm = (const T*)P.hmid + (long long)b * P.ld_hmid;
  float y = 0.f;
  for (int jj = 0; jj < P.top; ++jj) {
    const int e = P.eids[(long long)b * P.ld_top + jj];
    const T* wd = (const T*)P.w_down + ((long long)e * P.E + n) * P.F;
    y += P.ew[(long long)b * P.ld_top + jj] * wave_dot<T>(wd, hm + jj * P.F, P.F, lane, vec != 0);
  }
  if (P.Fs > 0)
    y += P.sgate[b] * wave_dot<T>((const T*)P.sh_down + (long long)n * P.Fs, hm + P.top * P.F, P.Fs, lane, vec_s != 0);
  if (lane == 0) P.y[(long long)b * P.E + n] = P.y_add ? P.y[(long long)b * P.E + n] + y : y;
}
// ---- prompt portions: pairs (row, routed expert) sorted by expert, one matrix-core product per expert tile
// One block: counts per expert (LDS atomics hand every pair its rank inside its expert; the order inside an
// expert does not reach the result, every pair's output row is its own), offsets, the tile table, and the two
// maps sorted position -> pair and pair -> sorted position.
__global__ __launch_bounds__(256) void moe_sort_kernel(const int* __restrict__ eids, int ld_top, int B, int top, int X,
                                                       int tile_m, int* __restrict__ rank, int* __restrict__ srow,
                                                       int* __restrict__ inv, int* __restrict__ tiles,
                                                       int* __restrict__ ntiles) {
  __shared__ int cnt[256], off[256];
  const int tid = threadIdx.x, P = B * top;
  for (int e = tid; e < X; e += 256) cnt[e] = 0;
  __syncthreads();
  for (int p = tid; p < P; p += 256) rank[p] = atomicAdd(&cnt[eids[(long long)(p / top) * ld_top + p % top]], 1);
  __syncthreads();
  if (tid == 0) {
    int at = 0, nt = 0;
    for (int e = 0; e < X; ++e) {
      off[e] = at;
      for (int t0 = 0; t0 < cnt[e]; t0 += tile_m) {
        tiles[3 * nt] = e;
        tiles[3 * nt + 1] = at + t0;
        tiles[3 * nt + 2] = min(tile_m, cnt[e] - t0);
        ++nt;
      }
      at += cnt[e];
    }
    *ntiles = nt;
  }
  __syncthreads();
  for (int p = tid; p < P; p += 256) {
    const int pos = off[eids[(long long)(p / top) * ld_top + p % top]] + rank[p];
    srow[pos] = p;
    inv[p] = pos;
  }
}
// hs[pos][f] = silu(gu[pos][f]) * gu[pos][F + f], in the matrix dtype
__global__ __launch_bounds__(256) void moe_act_kernel(const float* __restrict__ gu, int P, int F, bf16* __restrict__ hs) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long long)P * F) return;
  const long long pos = i / F;
  const int f = (int)(i % F);
  st(hs + i, silu(gu[pos * 2 * F + f]) * gu[pos * 2 * F + F + f]);
}
// y[b][n] = (shared ? sgate[b] * y[b][n] : 0) + sum_j ew[b][j] * ds[inv[b * top + j]][n], routing order
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ y, const float* __restrict__ ds,
                                                          const int* __restrict__ inv, const float* __restrict__ ew,
                                                          int ld_top, const float* __restrict__ sgate, int B, int E, int top,
                                                          int shared, int y_add) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= (long long)B * E) return;
  const int b = (int)(i / E), n = (int)(i % E);
  float acc = shared ? sgate[b] * y[i] : y_add ? y[i] : 0.f;  // (y_add: y is the residual stream, no shared expert)
  float routed = 0.f;
  for (int j = 0; j < top; ++j) routed += ew[(long long)b * ld_top + j] * ds[(long long)inv[b * top + j] * E + n];
  y[i] = routed + acc;
}
bool moe_grouped_supported(const MoeParams& P) {
  return !P.f32 && P.X <= 256 && P.E % 8 == 0 && P.F % 8 == 0 && (P.Fs == 0 || (P.Fs % 8 == 0 && (P.top * P.F) % 8 == 0 &&
         P.ld_hmid % 8 == 0));
}
void moe_grouped(const MoeParams& P, const MoeGroupWs& W, hipStream_t s) {
  check(moe_grouped_supported(P) && W.rank && W.srow && W.inv && W.tiles && W.ntiles && W.gu && W.hs && W.ds && !(P.y_add && P.Fs > 0),
        "grouped routed feed-forward: workspace or sizes");
  const int pairs = P.B * P.top;
  const int tile_m = pairs / P.X >= 192 ? 128 : 64;
  const int max_tiles = (pairs + tile_m - 1) / tile_m + P.X;
  check(pairs <= W.max_pairs && max_tiles <= W.max_tiles, "grouped routed feed-forward: workspace too small");
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(256), 0, s, P.eids, P.ld_top, P.B, P.top, P.X, tile_m, W.rank, W.srow,
                     W.inv, W.tiles, W.ntiles);
  launched("moe_sort");
  // gate | up of every pair with its expert's matrix
  {
    Epi e{EPI_STORE, W.gu, 2 * P.F, 0.f, nullptr, 0.f};
    Group G{W.tiles, W.ntiles, W.srow, P.top, (long long)2 * P.F * P.E};
    if (tile_m == 128) {
      dim3 grid((2 * P.F + 127) / 128, max_tiles);
      hipLaunchKernelGGL((gemm_mfma_kernel<2, 2>), grid, dim3(256), 0, s, (const bf16*)P.h, P.E, (const bf16*)P.w_gu, pairs,
                         2 * P.F, P.E, e, G);
    } else {
      dim3 grid((2 * P.F + 63) / 64, max_tiles);
      hipLaunchKernelGGL((gemm_mfma_kernel<1, 1>), grid, dim3(256), 0, s, (const bf16*)P.h, P.E, (const bf16*)P.w_gu, pairs,
                         2 * P.F, P.E, e, G);
    }
    launched("moe_gemm gate/up");
  }
  {
    const long long n = (long long)pairs * P.F;
    hipLaunchKernelGGL(moe_act_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, W.gu, pairs, P.F, (bf16*)W.hs);
    launched("moe_act");
  }
  {
    Epi e{EPI_STORE, W.ds, P.E, 0.f, nullptr, 0.f};
    Group G{W.tiles, W.ntiles, nullptr, 1, (long long)P.E * P.F};
    if (tile_m == 128) {
      dim3 grid((P.E + 127) / 128, max_tiles);
      hipLaunchKernelGGL((gemm_mfma_kernel<2, 2>), grid, dim3(256), 0, s, (const bf16*)W.hs, P.F, (const bf16*)P.w_down, pairs,
                         P.E, P.F, e, G);
    } else {
      dim3 grid((P.E + 63) / 64, max_tiles);
      hipLaunchKernelGGL((gemm_mfma_kernel<1, 1>), grid, dim3(256), 0, s, (const bf16*)W.hs, P.F, (const bf16*)P.w_down, pairs,
                         P.E, P.F, e, G);
    }
    launched("moe_gemm down");
  }
  if (P.Fs > 0) {  // the shared expert's down projection over every row, into y
    GemmParams g{(const bf16*)P.hmid + P.top * P.F, P.ld_hmid, P.sh_down, P.B, P.E, P.Fs, P.y, P.E, EPI_STORE, 0.f, nullptr,
                 0.f, 0};
    gemm(g, s);
  }
  {
    const long long n = (long long)P.B * P.E;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, P.y, W.ds, W.inv, P.ew, P.ld_top,
                       P.sgate, P.B, P.E, P.top, (int)(P.Fs > 0), P.y_add);
    launched("moe_combine");
  }
}

// ---- a few rows (decode steps): two launches for the whole feed-forward and the layer's residual update
// Routing of one row by one thread (the caller's thread 0): ids and weights into LDS arrays
__device__ __forceinline__ void route_row(const MoeParams& P, const float* row, int* ids, float* val) {
  for (int jj = 0; jj < P.top; ++jj) {
    int best = -1;
    float bv = -INFINITY;
    for (int e = 0; e < P.X; ++e) {
      bool taken = false;
      for (int q = 0; q < jj; ++q) taken |= ids[q] == e;
      if (taken) continue;
      const float z = row[P.off_router + e] + P.router_b[e];
      if (best < 0 || z > bv) {
        best = e;
        bv = z;
      }
    }
    ids[jj] = best;
    val[jj] = bv;
  }
  const float mx = val[0];
  float sum = 0.f;
  for (int jj = 0; jj < P.top; ++jj) {
    val[jj] = expf(val[jj] - mx);
    sum += val[jj];
  }
  for (int jj = 0; jj < P.top; ++jj) val[jj] /= sum;
}
// grid (ceil(max(F, Fs) / 4), B * (top + 1)): blocks y = b * (top + 1) + jj route row b again (a few dozen
// operations) and take routed expert jj < top, or (jj == top) the shared expert's activation from the input
// projection; the first block of a row also leaves ids, weights and the shared gate for the second launch
template <typename T>
__global__ __launch_bounds__(256) void moe_route_experts_kernel(MoeParams P, int vec) {
  __shared__ int ids[MOE_MAX_TOP];
  __shared__ float val[MOE_MAX_TOP];
  const int lane = threadIdx.x & 63;
  const int f = blockIdx.x * 4 + (threadIdx.x >> 6);
  const int b = blockIdx.y / (P.top + 1), jj = blockIdx.y % (P.top + 1);
  const float* row = P.proj + (long long)b * P.ld;
  T* hm = (T*)P.hmid + (long long)b * P.ld_hmid;
  if (jj == P.top) {  // shared expert
    if (f < P.Fs && lane == 0) st(hm + P.top * P.F + f, silu(row[P.off_sgate + f]) * row[P.off_sup + f]);
    return;
  }
  int e;
  if (P.X <= 64) {
    // every wave routes the row itself, one expert per lane: `top` rounds of (maximum, lowest lane that holds it)
    float z = lane < P.X ? row[P.off_router + lane] + P.router_b[lane] : -INFINITY;
    float mx0 = 0.f, sum = 0.f, mine = 0.f;
    e = 0;
    for (int q = 0; q < P.top; ++q) {
      const float mx = wave_max(z);
      // non-finite logits (a fault upstream) compare unequal to everything: expert 0 then, never an index of -1
      const int who = max(0, __ffsll((unsigned long long)__ballot(z == mx)) - 1);
      if (q == 0) mx0 = mx;
      const float w = expf(mx - mx0);
      sum += w;
      if (q == jj) e = who;
      if (lane == q) mine = w;       // lane q keeps the q-th weight (top <= 16 < 64)
      if (threadIdx.x == 0 && blockIdx.x == 0 && jj == 0) P.eids[(long long)b * P.ld_top + q] = who;
      if (lane == who) z = -INFINITY;
    }
    if (threadIdx.x < P.top && blockIdx.x == 0 && jj == 0) P.ew[(long long)b * P.ld_top + threadIdx.x] = mine / sum;
    if (threadIdx.x == 0 && blockIdx.x == 0 && jj == 0 && P.Fs > 0) P.sgate[b] = sigmoidf(row[P.off_sg]);
  } else {
    if (threadIdx.x == 0) {
      route_row(P, row, ids, val);
      if (blockIdx.x == 0 && jj == 0) {
        for (int q = 0; q < P.top; ++q) {
          P.eids[(long long)b * P.ld_top + q] = ids[q];
          P.ew[(long long)b * P.ld_top + q] = val[q];
        }
        if (P.Fs > 0) P.sgate[b] = sigmoidf(row[P.off_sg]);
      }
    }
    __syncthreads();
    e = ids[jj];
  }
  if (f >= P.F) return;
  const T* x = (const T*)P.h + (long long)b * P.E;
  const T* wg = (const T*)P.w_gu + ((long long)e * 2 * P.F + f) * P.E;
  const T* wu = wg + (long long)P.F * P.E;
  const float gate = wave_dot<T>(wg, x, P.E, lane, vec != 0);
  const float up = wave_dot<T>(wu, x, P.E, lane, vec != 0);
  if (lane == 0) st(hm + jj * P.F + f, silu(gate) * up);
}
// x[b][n] += mult * (W_o[n] . a[b] + sum_j w_j W_down[e_j][n] . hmid_j + sgate * W_shared_down[n] . hmid_s):
// one wave per output unit, every row of the step
template <typename T>
__global__ __launch_bounds__(256) void moe_down_out_kernel(MoeParams P, const T* __restrict__ a, int lda,
                                                           const T* __restrict__ w_o, int Ko, float* __restrict__ x,
                                                           float mult, int vec, int vec_s, int vec_o) {
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= P.E) return;
  for (int b = 0; b < P.B; ++b) {
    float y = wave_dot<T>(w_o + (long long)n * Ko, a + (long long)b * lda, Ko, lane, vec_o != 0);
    const T* hm = (const T*)P.hmid + (long long)b * P.ld_hmid;
    for (int jj = 0; jj < P.top; ++jj) {
      const int e = P.eids[(long long)b * P.ld_top + jj];
      const T* wd = (const T*)P.w_down + ((long long)e * P.E + n) * P.F;
      y += P.ew[(long long)b * P.ld_top + jj] * wave_dot<T>(wd, hm + jj * P.F, P.F, lane, vec != 0);
    }
    if (P.Fs > 0)
      y += P.sgate[b] * wave_dot<T>((const T*)P.sh_down + (long long)n * P.Fs, hm + P.top * P.F, P.Fs, lane, vec_s != 0);
    if (lane == 0) x[(long long)b * P.E + n] += mult * y;
  }
}
static void check_moe(const MoeParams& P, bool bias = true);
template <typename T>
static void launch_moe_fused(const MoeParams& P, const void* a, int lda, const void* w_o, int Ko, float* x, float mult,
                             hipStream_t s) {
  const int per = 16 / (int)sizeof(T);
  const int v1 = vec_ok<T>(P.h, P.E, P.E) && vec_ok<T>(P.w_gu, P.E, P.E);
  dim3 g1((std::max(P.F, P.Fs) + 3) / 4, P.B * (P.top + 1));
  hipLaunchKernelGGL(moe_route_experts_kernel<T>, g1, dim3(256), 0, s, P, v1);
  const int v = vec_ok<T>(P.hmid, P.ld_hmid, P.F) && vec_ok<T>(P.w_down, P.F, P.F);
  const int vs = P.Fs > 0 && vec_ok<T>(P.hmid, P.ld_hmid, P.Fs) && vec_ok<T>(P.sh_down, P.Fs, P.Fs) && (P.top * P.F) % per == 0;
  const int vo = vec_ok<T>(a, lda, Ko) && vec_ok<T>(w_o, Ko, Ko);
  dim3 g2((P.E + 3) / 4);
  hipLaunchKernelGGL(moe_down_out_kernel<T>, g2, dim3(256), 0, s, P, (const T*)a, lda, (const T*)w_o, Ko, x, mult, v, vs, vo);
}
void moe_fused_small(const MoeParams& P, const void* a, int lda, const void* w_o, int Ko, float* x, float mult,
                     hipStream_t s) {
  check_moe(P);
  check(a && w_o && x && Ko > 0 && lda >= Ko, "fused feed-forward + output projection: bad operands");
  if (P.f32)
    launch_moe_fused<float>(P, a, lda, w_o, Ko, x, mult, s);
  else
    launch_moe_fused<bf16>(P, a, lda, w_o, Ko, x, mult, s);
  launched("moe_fused_small");
}

static void check_moe(const MoeParams& P, bool bias) {  // bias: the caller reads router_b
  check(P.B > 0 && P.X > 0 && P.top > 0 && P.top <= P.X + P.identity && P.top <= MOE_MAX_TOP && P.F > 0 && P.proj && P.h && P.w_gu &&
            P.w_down && P.eids && P.ew && P.hmid && P.y && (P.router_b || !bias) && P.ld_top >= P.top &&
            P.ld_hmid >= P.top * P.F + P.Fs && (P.Fs == 0 || (P.sh_down && P.sgate)),
        "routed feed-forward: bad operands (top <= 16)");
}
void moe_route(const MoeParams& P, hipStream_t s) {
  check_moe(P);
  if (P.f32)
    hipLaunchKernelGGL(moe_route_kernel<float>, dim3(P.B), dim3(256), 0, s, P);
  else
    hipLaunchKernelGGL(moe_route_kernel<bf16>, dim3(P.B), dim3(256), 0, s, P);
  launched("moe_route");
}
void moe_experts(const MoeParams& P, hipStream_t s) {
  check_moe(P, false);
  dim3 grid((P.F + 3) / 4, P.B * P.top);
  if (P.f32)
    hipLaunchKernelGGL(moe_experts_kernel<float>, grid, dim3(256), 0, s, P,
                       (int)(vec_ok<float>(P.h, P.E, P.E) && vec_ok<float>(P.w_gu, P.E, P.E)));
  else
    hipLaunchKernelGGL(moe_experts_kernel<bf16>, grid, dim3(256), 0, s, P,
                       (int)(vec_ok<bf16>(P.h, P.E, P.E) && vec_ok<bf16>(P.w_gu, P.E, P.E)));
  launched("moe_experts");
}
template <typename T>
static void launch_moe_down(const MoeParams& P, hipStream_t s) {
  // hmid rows: expert j's slice starts at j * F, the shared slice at top * F
  const int v = vec_ok<T>(P.hmid, P.ld_hmid, P.F) && vec_ok<T>(P.w_down, P.F, P.F) && P.F % (16 / (int)sizeof(T)) == 0;
  const int vs = P.Fs > 0 && v && vec_ok<T>(P.sh_down, P.Fs, P.Fs) && (P.top * P.F) % (16 / (int)sizeof(T)) == 0;
  dim3 grid((P.E + 3) / 4, P.B);
  hipLaunchKernelGGL(moe_down_kernel<T>, grid, dim3(256), 0, s, P, v, vs);
}
void moe_down(const MoeParams& P, hipStream_t s) {
  check_moe(P, false);
  if (P.f32)
    launch_moe_down<float>(P, s);
  else
    launch_moe_down<bf16>(P, s);
  launched("moe_down");
}

}  // namespace stack
}  // namespace omx
