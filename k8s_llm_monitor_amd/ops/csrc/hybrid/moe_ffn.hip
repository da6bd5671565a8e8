// Routed feed-forward of the layer-list decoders (any sizes, bf16 or fp32 activations).
//   moe_router    fp32 logits = Wr h + b (h widened from its storage dtype; b may be absent), the K
//                 largest chosen (lowest index wins a tie), weights = softmax over the chosen logits
//                 only, or (over_all) the chosen experts' probabilities in the softmax over all E
//                 logits, not renormalised; one more row of Wr, if present, gives
//                 gate = sigmoid(Wr[E] h) (the shared expert's)
//   router_grouped  sigmoid scores; the experts form equal groups of neighbours, a group scores the sum of its
//                 two largest, only the `keep` best groups' experts can be chosen; the K largest scores among
//                 them, weights = score / (sum of the chosen + 1e-20) * scale
//   grouped_gemm  Y[r] = W[e(r)] A[row(r)] over expert-sorted rows r (offsets / sorted_idx from the
//                 counting sort), the A rows gathered on load; ACT 1 (SwiGLU): W = [gate rows ; up
//                 rows] and Y = silu(gate) * up; ACT 2: Y = gelu(W A) (erf form); ACT 3: gated like 1 with the clamped unit
//                 g sigmoid(1.702 g) (u + 1), g = min(gate, limit), u = clamp(up, -limit, limit).  64 x 64 tiles, fp32
//                 accumulation.
//   moe_combine   out[t] = sum_k w[t][k] Y[inv[t*K + k]] + gate[t] * shared[t]   (fp32; no gate: 1)
#include "hy_common.h"

namespace k8sllm {

constexpr int kMaxE = 256;
constexpr int kMaxK = 16;

// NACC > 0: at most NACC weight rows - every thread reads its columns of h once and keeps all the
// rows' partial dot products in registers (h is the large operand; the fp32 weight rows stay in L1);
// NACC == 0: any number of rows, one wave per row in turn.
template <typename T, int NACC>
__global__ __launch_bounds__(256) void hy_router_kernel(int* __restrict__ ids, float* __restrict__ wts,
                                                        float* __restrict__ gate, const T* __restrict__ h, int d,
                                                        const float* __restrict__ wr, const float* __restrict__ bias,
                                                        int E, int K, int rows_w, int over_all) {
  __shared__ float lg[kMaxE + 1];
  __shared__ float part[4][NACC > 0 ? NACC : 1];
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* x = h + t * d;
  if (NACC > 0) {
    float acc[NACC > 0 ? NACC : 1];
#pragma unroll
    for (int e = 0; e < NACC; ++e) acc[e] = 0.f;
    if ((d & 7) == 0) {  // 8 columns per thread and trip: 16-byte loads of h, 32 bytes of each weight row
      for (int c = threadIdx.x * 8; c < d; c += 2048) {
        float xv[8];
        load8(x + c, xv);
#pragma unroll
        for (int e = 0; e < NACC; ++e)
          if (e < rows_w) {
            const float4 wa = *reinterpret_cast<const float4*>(wr + (long)e * d + c);
            const float4 wb = *reinterpret_cast<const float4*>(wr + (long)e * d + c + 4);
            acc[e] += xv[0] * wa.x + xv[1] * wa.y + xv[2] * wa.z + xv[3] * wa.w + xv[4] * wb.x + xv[5] * wb.y +
                      xv[6] * wb.z + xv[7] * wb.w;
          }
      }
    } else {
#pragma unroll 4
      for (int c = threadIdx.x; c < d; c += 256) {
        const float xv = ldf(x + c);
#pragma unroll
        for (int e = 0; e < NACC; ++e)
          if (e < rows_w) acc[e] += xv * wr[(long)e * d + c];
      }
    }
#pragma unroll
    for (int e = 0; e < NACC; ++e) {
      const float v = wave_sum(acc[e]);
      if (lane == 0) part[wave][e] = v;
    }
    __syncthreads();
    if (threadIdx.x < rows_w) {
      const int e = threadIdx.x;
      const float a = part[0][e] + part[1][e] + part[2][e] + part[3][e];
      lg[e] = (e < E && bias != nullptr) ? a + bias[e] : a;
    }
  } else {
    for (int e = wave; e < rows_w; e += 4) {
      const float* w = wr + (long)e * d;
      float a = 0.f;
      for (int c = lane; c < d; c += 64) a += ldf(x + c) * w[c];
      a = wave_sum(a);
      if (lane == 0) lg[e] = (e < E && bias != nullptr) ? a + bias[e] : a;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int sel[kMaxK];
    float val[kMaxK];
    float mx = -INFINITY;
    for (int k = 0; k < K; ++k) {
      int best = -1;
      float bv = -INFINITY;
      for (int e = 0; e < E; ++e) {
        bool taken = false;
        for (int j = 0; j < k; ++j) taken |= sel[j] == e;
        if (!taken && (best < 0 || lg[e] > bv)) {
          bv = lg[e];
          best = e;
        }
      }
      sel[k] = best;
      val[k] = bv;
      mx = fmaxf(mx, bv);
    }
    float z = 0.f;
    if (over_all) {  // the denominator runs over every expert (val[0] is the largest logit of all)
      for (int e = 0; e < E; ++e) z += expf(lg[e] - mx);
      for (int k = 0; k < K; ++k) val[k] = expf(val[k] - mx);
    } else {
      for (int k = 0; k < K; ++k) {
        val[k] = expf(val[k] - mx);
        z += val[k];
      }
    }
    for (int k = 0; k < K; ++k) {
      ids[t * K + k] = sel[k];
      wts[t * K + k] = val[k] / z;
    }
    if (gate != nullptr) gate[t] = 1.f / (1.f + expf(-lg[E]));
  }
}

// Sigmoid router with a choice restricted to the best groups.  One workgroup per token computes the logits
// (fp32 weights, h widened; NACC as in hy_router_kernel), thread 0 scores the groups and picks.
template <typename T, int NACC>
__global__ __launch_bounds__(256) void hy_router_grouped_kernel(int* __restrict__ ids, float* __restrict__ wts,
                                                                const T* __restrict__ h, int d,
                                                                const float* __restrict__ wr, int E, int K, int groups,
                                                                int keep, float scale) {
  __shared__ float sc[kMaxE];
  __shared__ float gsc[kMaxE];
  __shared__ float part[4][NACC > 0 ? NACC : 1];
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* x = h + t * d;
  if (NACC > 0) {  // at most NACC experts: h is read once, every expert's partial sum stays in a register
    float acc[NACC > 0 ? NACC : 1];
#pragma unroll
    for (int e = 0; e < NACC; ++e) acc[e] = 0.f;
    if ((d & 7) == 0) {
      for (int c = threadIdx.x * 8; c < d; c += 2048) {
        float xv[8];
        load8(x + c, xv);
#pragma unroll
        for (int e = 0; e < NACC; ++e)
          if (e < E) {
            const float4 wa = *reinterpret_cast<const float4*>(wr + (long)e * d + c);
            const float4 wb = *reinterpret_cast<const float4*>(wr + (long)e * d + c + 4);
            acc[e] += xv[0] * wa.x + xv[1] * wa.y + xv[2] * wa.z + xv[3] * wa.w + xv[4] * wb.x + xv[5] * wb.y +
                      xv[6] * wb.z + xv[7] * wb.w;
          }
      }
    } else {
#pragma unroll 4
      for (int c = threadIdx.x; c < d; c += 256) {
        const float xv = ldf(x + c);
#pragma unroll
        for (int e = 0; e < NACC; ++e)
          if (e < E) acc[e] += xv * wr[(long)e * d + c];
      }
    }
#pragma unroll
    for (int e = 0; e < NACC; ++e) {
      const float v = wave_sum(acc[e]);
      if (lane == 0) part[wave][e] = v;
    }
    __syncthreads();
    if (threadIdx.x < E) {
      const int e = threadIdx.x;
      sc[e] = 1.f / (1.f + expf(-(part[0][e] + part[1][e] + part[2][e] + part[3][e])));
    }
  } else {
    for (int e = wave; e < E; e += 4) {
      const float* w = wr + (long)e * d;
      float a = 0.f;
      for (int c = lane; c < d; c += 64) a += ldf(x + c) * w[c];
      a = wave_sum(a);
      if (lane == 0) sc[e] = 1.f / (1.f + expf(-a));
    }
  }
  __syncthreads();
  const int per = E / groups;
  if (threadIdx.x < groups) {  // a group's score: its two largest scores (one expert per group: its score)
    float m1 = -1.f, m2 = -1.f;
    for (int e = threadIdx.x * per; e < (threadIdx.x + 1) * per; ++e) {
      const float v = sc[e];
      if (v > m1) {
        m2 = m1;
        m1 = v;
      } else if (v > m2) {
        m2 = v;
      }
    }
    gsc[threadIdx.x] = per > 1 ? m1 + m2 : m1;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    if (keep < groups) {  // scores of experts outside the best groups drop below every sigmoid
      for (int k = 0; k < keep; ++k) {
        int best = -1;
        float bv = -INFINITY;
        for (int g = 0; g < groups; ++g)
          if (gsc[g] > bv) {
            bv = gsc[g];
            best = g;
          }
        gsc[best] = -INFINITY;  // marks a kept group
      }
    }
    int sel[kMaxK];
    float val[kMaxK];
    float z = 0.f;
    for (int k = 0; k < K; ++k) {
      int best = -1;
      float bv = -INFINITY;
      for (int e = 0; e < E; ++e) {
        if (keep < groups && gsc[e / per] != -INFINITY) continue;
        bool taken = false;
        for (int j = 0; j < k; ++j) taken |= sel[j] == e;
        if (!taken && (best < 0 || sc[e] > bv)) {
          bv = sc[e];
          best = e;
        }
      }
      sel[k] = best;
      val[k] = bv;
      z += bv;
    }
    for (int k = 0; k < K; ++k) {
      ids[t * K + k] = sel[k];
      wts[t * K + k] = val[k] / (z + 1e-20f) * scale;
    }
  }
}

constexpr int TM = 64, TN = 64, TK = 16;

__device__ __forceinline__ float gelu_erf_f(float z) { return 0.5f * z * (1.f + erff(z * 0.70710678118654752f)); }
__device__ __forceinline__ float clamped_unit_f(float g, float u, float limit) {
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g * sigmoid_f(1.702f * g) * (u + 1.f);
}

template <typename T, int ACT>
__global__ __launch_bounds__(256) void hy_grouped_gemm_kernel(T* __restrict__ Y, const T* __restrict__ A,
                                                              const T* __restrict__ W, const int* __restrict__ offsets,
                                                              const int* __restrict__ sorted_idx, int div, int E,
                                                              int N, int Kd, long w_es, int il, float limit) {
  constexpr bool SWIGLU = ACT == 1 || ACT == 3;  // gated: gate rows and up rows
  __shared__ float As[TK][TM + 4];
  __shared__ float Ws[TK][TN + 4];
  __shared__ float Us[SWIGLU ? TK : 1][TN + 4];
  // this workgroup's (expert, row tile): tiles are numbered expert by expert
  int e = 0, tile = blockIdx.x, r0 = 0, r1 = 0;
  for (; e < E; ++e) {
    r0 = offsets[e];
    r1 = offsets[e + 1];
    const int nt = (r1 - r0 + TM - 1) / TM;
    if (tile < nt) break;
    tile -= nt;
  }
  if (e >= E) return;
  r0 += tile * TM;
  const int n0 = blockIdx.y * TN;
  const T* We = W + (long)e * w_es;
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;  // 4 x 4 outputs per thread: rows ty*4.., cols tx*4..
  float acc[4][4], accu[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = accu[i][j] = 0.f;
  // loader: thread -> (row lr, k offsets lk, lk + 4, ...) of the 64 x 16 tiles
  const int lr = tid >> 2, lk = (tid & 3) * 4;
  const int arow = r0 + lr;
  long asrc = -1;
  if (arow < r1) asrc = sorted_idx != nullptr ? sorted_idx[arow] / div : arow;
  const int wrow = n0 + lr;
  // row of W holding output column wrow's gate (or only) weights, and its up weights
  const long grow = SWIGLU && il ? (long)(wrow >> 6) * 128 + (wrow & 63) : wrow;
  const long urow = il ? grow + 64 : (long)N + wrow;
  for (int k0 = 0; k0 < Kd; k0 += TK) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + lk + j;
      As[lk + j][lr] = (asrc >= 0 && k < Kd) ? ldf(A + asrc * Kd + k) : 0.f;
      Ws[lk + j][lr] = (wrow < N && k < Kd) ? ldf(We + grow * Kd + k) : 0.f;
      if (SWIGLU) Us[lk + j][lr] = (wrow < N && k < Kd) ? ldf(We + urow * Kd + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < TK; ++k) {
      float a[4], b[4], u[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[k][tx * 4 + j];
      if (SWIGLU) {
#pragma unroll
        for (int j = 0; j < 4; ++j) u[j] = Us[k][tx * 4 + j];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] += a[i] * b[j];
          if (SWIGLU) accu[i][j] += a[i] * u[j];
        }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + ty * 4 + i;
    if (r >= r1) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (SWIGLU) {
        // the separate-projection form rounds gate and up to the storage dtype before the product
        T gq, uq;
        stf(&gq, v);
        stf(&uq, accu[i][j]);
        v = ACT == 3 ? clamped_unit_f(ldf(&gq), ldf(&uq), limit) : silu_f(ldf(&gq)) * ldf(&uq);
      } else if (ACT == 2) {  // the projection is rounded to the storage dtype before the activation
        T gq;
        stf(&gq, v);
        v = gelu_erf_f(ldf(&gq));
      }
      stf(Y + (long)r * N + n, v);
    }
  }
}

// bf16 on the matrix cores (K a multiple of 32): one wave = 16 sorted rows x 16 NT output columns
// (NT = 4; NT = 1 with a deeper unroll when there are few rows, so that a decode step's weight
// stream is spread over four times as many waves),
// v_mfma_f32_16x16x32_bf16 with both operands loaded straight from global memory as 16-byte
// fragments (A = the gathered activation rows, B = weight rows, 8 consecutive k per lane).  Few
// rows per expert (decode) make this a weight-streaming kernel: many small workgroups, no LDS.
// ``il``: the gate / up rows are interleaved per 128 rows as [64 gate | 64 up] (the prefill tile
// GEMM's pairing), else [all gate rows ; all up rows].
template <int ACT, int NT>
__global__ __launch_bounds__(64) void hy_grouped_gemm_mfma_kernel(bf16_t* __restrict__ Y, const bf16_t* __restrict__ A,
                                                                  const bf16_t* __restrict__ W,
                                                                  const int* __restrict__ offsets,
                                                                  const int* __restrict__ sorted_idx, int div, int E,
                                                                  int N, int Kd, long w_es, int il, float limit) {
  constexpr bool SWIGLU = ACT == 1 || ACT == 3;  // gated: gate rows and up rows
  int e = 0, tile = blockIdx.x, r0 = 0, r1 = 0;
  for (; e < E; ++e) {
    r0 = offsets[e];
    r1 = offsets[e + 1];
    const int nt = (r1 - r0 + 15) >> 4;
    if (tile < nt) break;
    tile -= nt;
  }
  if (e >= E) return;
  r0 += tile * 16;
  const int lane = threadIdx.x, c16 = lane & 15, quad = lane >> 4;
  const int n0 = blockIdx.y * (16 * NT);
  const bf16_t* We = W + (long)e * w_es;
  const int arow = min(r0 + c16, r1 - 1);
  const long asrc = sorted_idx != nullptr ? sorted_idx[arow] / div : arow;
  const bf16_t* ap = A + asrc * Kd + 8 * quad;
  const bf16_t* wg[NT];
  const bf16_t* wu[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int n = min(n0 + 16 * t + c16, N - 1);
    const long g = SWIGLU && il ? (long)(n >> 6) * 128 + (n & 63) : n;
    wg[t] = We + g * Kd + 8 * quad;
    wu[t] = We + (SWIGLU ? (il ? g + 64 : (long)N + n) : 0) * Kd + 8 * quad;
  }
  f32x4 acc[NT], accu[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = accu[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll(NT == 1 ? 8 : 2)
  for (int k0 = 0; k0 < Kd; k0 += 32) {
    const bf16x8 a = *reinterpret_cast<const bf16x8*>(ap + k0);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, *reinterpret_cast<const bf16x8*>(wg[t] + k0), acc[t], 0, 0, 0);
      if (SWIGLU)
        accu[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, *reinterpret_cast<const bf16x8*>(wu[t] + k0), accu[t], 0, 0, 0);
    }
  }
#pragma unroll
  for (int t = 0; t < NT; ++t) {  // acc[t][i]: row r0 + 4 quad + i, column n0 + 16 t + c16
    const int n = n0 + 16 * t + c16;
    if (n >= N) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int r = r0 + 4 * quad + i;
      if (r >= r1) continue;
      float v = acc[t][i];
      if (ACT == 3) v = clamped_unit_f(bf2f(f2bf(v)), bf2f(f2bf(accu[t][i])), limit);
      else if (SWIGLU) v = silu_f(bf2f(f2bf(v))) * bf2f(f2bf(accu[t][i]));
      else if (ACT == 2) v = gelu_erf_f(bf2f(f2bf(v)));
      Y[(long)r * N + n] = f2bf(v);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void hy_combine_kernel(float* __restrict__ out, const T* __restrict__ ys,
                                                         const int* __restrict__ inv, const float* __restrict__ wts,
                                                         const T* __restrict__ shared, const float* __restrict__ gate,
                                                         int K, int d) {
  const long t = blockIdx.x;
  for (int c = threadIdx.x; c < d; c += 256) {
    float a = 0.f;
    for (int k = 0; k < K; ++k) a += wts[t * K + k] * ldf(ys + (long)inv[t * K + k] * d + c);
    if (shared != nullptr) a += (gate != nullptr ? gate[t] : 1.f) * ldf(shared + t * d + c);
    out[t * d + c] = a;
  }
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" {

int k8sllm_hy_router(int* ids, float* wts, float* gate, const void* h, long T, int d, const float* wr,
                     const float* bias, int E, int K, int rows_w, int over_all, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (E > kMaxE || K > kMaxK || K > E || K < 1 || rows_w < E || rows_w > E + 1) return -1;
#define K8SLLM_RT(T_, NACC)                                                                                       \
  hipLaunchKernelGGL((hy_router_kernel<T_, NACC>), dim3(T), dim3(256), 0, s, ids, wts, gate, (const T_*)h, d, wr, bias, \
                     E, K, rows_w, over_all)
  if (f32) {
    if (rows_w <= 9) K8SLLM_RT(float, 9); else if (rows_w <= 17) K8SLLM_RT(float, 17); else K8SLLM_RT(float, 0);
  } else {
    if (rows_w <= 9) K8SLLM_RT(bf16_t, 9); else if (rows_w <= 17) K8SLLM_RT(bf16_t, 17); else K8SLLM_RT(bf16_t, 0);
  }
#undef K8SLLM_RT
  return (int)hipGetLastError();
}

int k8sllm_hy_router_grouped(int* ids, float* wts, const void* h, long T, int d, const float* wr, int E, int K,
                             int groups, int keep, float scale, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (E > kMaxE || K > kMaxK || K < 1 || groups < 1 || E % groups || keep < 1 || keep > groups ||
      K > keep * (E / groups))
    return -1;
#define K8SLLM_RG(T_, NACC)                                                                                        \
  hipLaunchKernelGGL((hy_router_grouped_kernel<T_, NACC>), dim3(T), dim3(256), 0, s, ids, wts, (const T_*)h, d, wr, E, K, \
                     groups, keep, scale)
  if (f32) {
    if (E <= 8) K8SLLM_RG(float, 8); else if (E <= 16) K8SLLM_RG(float, 16); else K8SLLM_RG(float, 0);
  } else {
    if (E <= 8) K8SLLM_RG(bf16_t, 8); else if (E <= 16) K8SLLM_RG(bf16_t, 16); else K8SLLM_RG(bf16_t, 0);
  }
#undef K8SLLM_RG
  return (int)hipGetLastError();
}

// rows: the sorted rows in all (an upper bound of the row tiles is rows / 64 + E)
int k8sllm_hy_grouped_gemm(void* Y, const void* A, const void* W, const int* offsets, const int* sorted_idx, int div,
                           int E, long rows, int N, int Kd, long w_es, int act, int il, int f32, int mfma, float limit,
                           hipStream_t s) {
  if (rows <= 0) return 0;
  if (act < 0 || act > 3) return -1;
  const bool swiglu = act == 1;
  if (il && (!swiglu || N % 64)) return -1;
  if (!f32 && mfma && Kd % 32 == 0) {
    const bool few = rows <= 512;  // a decode-sized step: one n-tile per wave
    const dim3 g16((unsigned)(rows / 16 + E), (unsigned)(few ? (N + 15) / 16 : (N + 63) / 64));
#define K8SLLM_GM(SW, NT)                                                                                        \
  hipLaunchKernelGGL((hy_grouped_gemm_mfma_kernel<SW, NT>), g16, dim3(64), 0, s, (bf16_t*)Y, (const bf16_t*)A,      \
                     (const bf16_t*)W, offsets, sorted_idx, div, E, N, Kd, w_es, il, limit)
    if (swiglu) {
      if (few) K8SLLM_GM(1, 1); else K8SLLM_GM(1, 4);
    } else if (act == 3) {
      if (few) K8SLLM_GM(3, 1); else K8SLLM_GM(3, 4);
    } else if (act == 2) {
      if (few) K8SLLM_GM(2, 1); else K8SLLM_GM(2, 4);
    } else {
      if (few) K8SLLM_GM(0, 1); else K8SLLM_GM(0, 4);
    }
#undef K8SLLM_GM
    return (int)hipGetLastError();
  }
  const dim3 grid((unsigned)(rows / TM + E), (unsigned)((N + TN - 1) / TN));
#define K8SLLM_GG(T, SW)                                                                                            \
  hipLaunchKernelGGL((hy_grouped_gemm_kernel<T, SW>), grid, dim3(256), 0, s, (T*)Y, (const T*)A, (const T*)W, offsets, \
                     sorted_idx, div, E, N, Kd, w_es, il, limit)
  if (f32) {
    if (swiglu) K8SLLM_GG(float, 1); else if (act == 3) K8SLLM_GG(float, 3); else if (act == 2) K8SLLM_GG(float, 2);
    else K8SLLM_GG(float, 0);
  } else {
    if (swiglu) K8SLLM_GG(bf16_t, 1); else if (act == 3) K8SLLM_GG(bf16_t, 3); else if (act == 2) K8SLLM_GG(bf16_t, 2);
    else K8SLLM_GG(bf16_t, 0);
  }
#undef K8SLLM_GG
  return (int)hipGetLastError();
}

int k8sllm_hy_combine(float* out, const void* ys, const int* inv, const float* wts, const void* shared,
                      const float* gate, long T, int K, int d, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (f32)
    hipLaunchKernelGGL(hy_combine_kernel<float>, dim3(T), dim3(256), 0, s, out, (const float*)ys, inv, wts,
                       (const float*)shared, gate, K, d);
  else
    hipLaunchKernelGGL(hy_combine_kernel<bf16_t>, dim3(T), dim3(256), 0, s, out, (const bf16_t*)ys, inv, wts,
                       (const bf16_t*)shared, gate, K, d);
  return (int)hipGetLastError();
}
}
