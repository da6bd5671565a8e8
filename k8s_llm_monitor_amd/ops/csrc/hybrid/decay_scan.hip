// Linear attention with a decay per head and key channel, with or without the delta rule (any sizes up
// to 256 key channels; state, decays, unit norms and every product fp32).
//   decay_scan   per segment and head, token by token:
//                    S <- diag(g_t) S
//                    u  = beta_t (v_t - S^T k_t)      (delta rule)      |  u = v_t   (plain)
//                    S <- S + k_t u^T;   o_t = S^T q_t
//                with g_t = exp(-exp(a_log[h]) softplus(z_t + bias))  or  sigmoid(z_t + bias)^(1/tau), q and k
//                optionally made unit vectors (x / sqrt(sum x^2 + 1e-6)), q times q_scale, beta_t = sigmoid of
//                a projection column.  The state slot [H][dv][dk] (a value row's key channels contiguous) is
//                read at the segment's start (zero for a sequence that starts in this step), written at its end.
// A segment is one sequence's rows of this step: cu[s] .. cu[s+1], ctx[s] tokens already in its state,
// slot[s] its state slot (< 0: a padding row, output zero).
//
// Workgroup = 4 waves = (segment, head, PB value columns).  A value column p is owned by CH neighbouring
// lanes, each holding 8 key channels of S[p][.] in registers; 64 / CH columns per wave.  The read-out is
// taken from the decayed state BEFORE the write: with S' = diag(g) S,
//     o = S'^T q + u (k . q)
// so the two sums over key channels that a token needs (S'^T k and S'^T q) are independent and their
// lane reductions overlap; k . q does not depend on the state and is prepared with the tile.  The inputs
// of 16 tokens at a time are staged in LDS by the whole workgroup (q, k after the unit norm, the decays
// after their exponentials, v, beta, k . q), so the token loop reads only LDS.
//
// Prompts (long segments) run as two launches: decay_prep computes, for every token at once, what does not
// depend on the state - the decays after their exponentials, q and k after the unit norm and the query scale,
// k . q, beta - as fp32 rows in a workspace, and decay_scan_staged runs the recurrence reading those rows:
// a tile's inputs are fetched into registers while the previous tile's tokens are processed, so the
// sequential loop waits neither for global memory nor for exponentials (which the one-launch form
// evaluates once per block of value columns).  Decode steps (one token per segment) keep the one-launch form.
#include "hy_common.h"

namespace k8sllm {

template <int CH>
__device__ __forceinline__ float lanes_sum(float v) {
  if (CH >= 2) v += K8SLLM_DPP(v, 0xB1);
  if (CH >= 4) v += K8SLLM_DPP(v, 0x4E);
  if (CH >= 8) v += K8SLLM_DPP(v, 0x141);
  if (CH >= 16) v += K8SLLM_DPP(v, 0x140);
  if (CH >= 32) v = xor16_sum(v);
  return v;
}

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

template <typename T, int CH, bool DELTA>
__global__ __launch_bounds__(256) void decay_scan_kernel(float* __restrict__ o, const T* __restrict__ qkv, long stride,
                                                         int q_col, int k_col, int v_col, const T* __restrict__ z,
                                                         long z_stride, const float* __restrict__ z_bias,
                                                         const float* __restrict__ a_log, float inv_tau,
                                                         const T* __restrict__ beta, long b_stride,
                                                         float* __restrict__ state, const int* __restrict__ cu,
                                                         const int* __restrict__ ctx, const int* __restrict__ slot,
                                                         int H, int Gk, int dk, int dv, float q_scale, int unit) {
  constexpr int TB = 16, PW = 64 / CH, PB = 4 * PW;
  constexpr int ROW = 8 * CH + (CH / 8) * 4 + 4;  // channel n sits at n + 4 (n / 64): 64-float halves 4 banks apart
  __shared__ __attribute__((aligned(16))) float qs[TB][ROW];
  __shared__ __attribute__((aligned(16))) float ks[TB][ROW];
  __shared__ __attribute__((aligned(16))) float gs[TB][ROW];
  __shared__ float vs[TB][PB];
  __shared__ float bts[TB], kqs[TB];
  const int s = blockIdx.x, h = blockIdx.y;
  const int sl = slot[s];
  const int t0 = cu[s], t1 = cu[s + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int chunk = lane % CH, pl = wave * PW + lane / CH;
  const int p = blockIdx.z * PB + pl;
  const bool live = p < dv;
  const int inner = H * dv;
  if (sl < 0) {  // padding rows: defined output, no state
    if (live && chunk == 0)
      for (int t = t0; t < t1; ++t) o[(long)t * inner + (long)h * dv + p] = 0.f;
    return;
  }
  if (t1 <= t0) return;
  const int n0 = chunk * 8;
  const int g = h / (H / Gk);
  if (dk != 8 * CH)  // channels beyond dk stay zero (none where the lanes' 8-channel chunks cover dk exactly)
    for (int i = threadIdx.x; i < min(TB, t1 - t0) * ROW; i += 256) {
      (&qs[0][0])[i] = 0.f;
      (&ks[0][0])[i] = 0.f;
      (&gs[0][0])[i] = 0.f;
    }
  float S[8];
  float* sp = state + (((long)sl * H + h) * dv + p) * dk + n0;
  const bool carried = ctx[s] > 0;
  const bool vec = (dk & 7) == 0 && n0 + 8 <= dk;
  if (carried && live && vec) {
    const float4 a = *reinterpret_cast<const float4*>(sp), b = *reinterpret_cast<const float4*>(sp + 4);
    S[0] = a.x; S[1] = a.y; S[2] = a.z; S[3] = a.w;
    S[4] = b.x; S[5] = b.y; S[6] = b.z; S[7] = b.w;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) S[i] = (carried && live && n0 + i < dk) ? sp[i] : 0.f;
  }
  const float A = a_log != nullptr ? expf(a_log[h]) : 0.f;
  const int boff = n0 + (n0 >> 6) * 4;
  float* op = o + (long)t0 * inner + (long)h * dv + p;  // this lane's output column, advanced per tile
  for (int tb = t0; tb < t1; tb += TB) {
    const int nt = min(TB, t1 - tb);
    __syncthreads();  // the previous tile is consumed (and the zero fill is done)
#pragma unroll 4
    for (int i = threadIdx.x; i < nt * dk; i += 256) {  // unrolled: the independent loads go out together
      const int tt = i / dk, n = i - tt * dk;
      const T* row = qkv + (long)(tb + tt) * stride + (long)g * dk + n;
      const int off = n + (n >> 6) * 4;
      qs[tt][off] = ldf(row + q_col);
      ks[tt][off] = ldf(row + k_col);
      const float zz = ldf(z + (long)(tb + tt) * z_stride + (long)h * dk + n) + z_bias[h * dk + n];
      gs[tt][off] = a_log != nullptr ? expf(-A * softplus_f(zz)) : expf(-softplus_f(-zz) * inv_tau);
    }
    for (int i = threadIdx.x; i < nt * PB; i += 256) {
      const int tt = i / PB, pp = i % PB;
      const int pg = blockIdx.z * PB + pp;
      vs[tt][pp] = pg < dv ? ldf(qkv + (long)(tb + tt) * stride + v_col + (long)h * dv + pg) : 0.f;
    }
    if (DELTA && threadIdx.x < nt) bts[threadIdx.x] = sigmoid_f(ldf(beta + (long)(tb + threadIdx.x) * b_stride + h));
    __syncthreads();
    {  // 16 threads per token: unit norms, the query scale and k . q
      const int tt = threadIdx.x >> 4, j = threadIdx.x & 15;
      float sq = 0.f, sk = 0.f;
      if (unit) {
        for (int n = j; n < dk; n += 16) {
          const int off = n + (n >> 6) * 4;
          sq += qs[tt][off] * qs[tt][off];
          sk += ks[tt][off] * ks[tt][off];
        }
        sq = lanes_sum<16>(sq);
        sk = lanes_sum<16>(sk);
      }
      const float mq = unit ? q_scale / sqrtf(sq + 1e-6f) : q_scale;
      const float mk = unit ? 1.0f / sqrtf(sk + 1e-6f) : 1.f;
      float kq = 0.f;
      for (int n = j; n < dk; n += 16) {
        const int off = n + (n >> 6) * 4;
        const float qv = qs[tt][off] * mq, kv = ks[tt][off] * mk;
        qs[tt][off] = qv;
        ks[tt][off] = kv;
        kq += qv * kv;
      }
      kq = lanes_sum<16>(kq);
      if (j == 0) kqs[tt] = kq;
    }
    __syncthreads();
#pragma unroll 2
    for (int tt = 0; tt < nt; ++tt) {
      const float4 g0 = *reinterpret_cast<const float4*>(&gs[tt][boff]);
      const float4 g1 = *reinterpret_cast<const float4*>(&gs[tt][boff + 4]);
      const float4 k0 = *reinterpret_cast<const float4*>(&ks[tt][boff]);
      const float4 k1 = *reinterpret_cast<const float4*>(&ks[tt][boff + 4]);
      const float4 q0 = *reinterpret_cast<const float4*>(&qs[tt][boff]);
      const float4 q1 = *reinterpret_cast<const float4*>(&qs[tt][boff + 4]);
      const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
      const float kv[8] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};
      const float qv[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
      float pk = 0.f, pq = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        S[i] *= gv[i];
        if (DELTA) pk += S[i] * kv[i];
        pq += S[i] * qv[i];
      }
      if (DELTA) pk = lanes_sum<CH>(pk);
      pq = lanes_sum<CH>(pq);
      const float v = vs[tt][pl];
      const float u = DELTA ? bts[tt] * (v - pk) : v;
#pragma unroll
      for (int i = 0; i < 8; ++i) S[i] += kv[i] * u;
      if (live && chunk == 0) op[(long)tt * inner] = pq + u * kqs[tt];
    }
    op += (long)TB * inner;
  }
  if (live) {
    if (vec) {
      *reinterpret_cast<float4*>(sp) = make_float4(S[0], S[1], S[2], S[3]);
      *reinterpret_cast<float4*>(sp + 4) = make_float4(S[4], S[5], S[6], S[7]);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (n0 + i < dk) sp[i] = S[i];
    }
  }
}

// ---- the two-launch form for prompts
// workspace rows (fp32): qn, kn [T][Gk][dk], gd [T][H][dk], kq [T][Gk], bt [T][H]
template <typename T>
__global__ __launch_bounds__(256) void decay_prep_kernel(float* __restrict__ qn, float* __restrict__ kn,
                                                         float* __restrict__ gd, float* __restrict__ kq,
                                                         float* __restrict__ bt, const T* __restrict__ qkv, long stride,
                                                         int q_col, int k_col, const T* __restrict__ z, long z_stride,
                                                         const float* __restrict__ z_bias,
                                                         const float* __restrict__ a_log, float inv_tau,
                                                         const T* __restrict__ beta, long b_stride, int H, int Gk,
                                                         int dk, float q_scale, int unit) {
  // one workgroup per token: the decays of all heads, beta, then a wave per query / key head
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nd = H * dk;
  const T* zr = z + t * z_stride;
  float* gr = gd + t * nd;
  if (a_log != nullptr) {
    for (int e = threadIdx.x; e < nd; e += 256)
      gr[e] = expf(-expf(a_log[e / dk]) * softplus_f(ldf(zr + e) + z_bias[e]));
  } else {
    for (int e = threadIdx.x; e < nd; e += 256) gr[e] = expf(-softplus_f(-(ldf(zr + e) + z_bias[e])) * inv_tau);
  }
  if (beta != nullptr)
    for (int h = threadIdx.x; h < H; h += 256) bt[t * H + h] = sigmoid_f(ldf(beta + t * b_stride + h));
  for (int g = wave; g < Gk; g += 4) {
    const T* row = qkv + t * stride + (long)g * dk;
    float sq = 0.f, sk = 0.f;
    if (unit) {
      for (int n = lane; n < dk; n += 64) {
        const float q = ldf(row + q_col + n), k = ldf(row + k_col + n);
        sq += q * q;
        sk += k * k;
      }
      sq = wave_sum(sq);
      sk = wave_sum(sk);
    }
    const float mq = unit ? q_scale / sqrtf(sq + 1e-6f) : q_scale;
    const float mk = unit ? 1.0f / sqrtf(sk + 1e-6f) : 1.f;
    float dot = 0.f;
    for (int n = lane; n < dk; n += 64) {
      const float q = ldf(row + q_col + n) * mq, k = ldf(row + k_col + n) * mk;
      qn[(t * Gk + g) * dk + n] = q;
      kn[(t * Gk + g) * dk + n] = k;
      dot += q * k;
    }
    dot = wave_sum(dot);
    if (lane == 0) kq[t * Gk + g] = dot;
  }
}

template <typename T, int CH, bool DELTA>
__global__ __launch_bounds__(256) void decay_scan_staged_kernel(float* __restrict__ o, const T* __restrict__ qkv,
                                                                long stride, int v_col, const float* __restrict__ qn,
                                                                const float* __restrict__ kn,
                                                                const float* __restrict__ gd,
                                                                const float* __restrict__ kq,
                                                                const float* __restrict__ bt, float* __restrict__ state,
                                                                const int* __restrict__ cu, const int* __restrict__ ctx,
                                                                const int* __restrict__ slot, int H, int Gk, int dk,
                                                                int dv) {
  constexpr int TB = 16, PW = 64 / CH, PB = 4 * PW;
  constexpr int ROW = 8 * CH + (CH / 8) * 4 + 4;  // channel n sits at n + 4 (n / 64); a multiple of 4 floats
  constexpr int Q4 = 2 * CH;                      // 4-channel groups of a padded row
  constexpr int NB = (TB * Q4 + 255) / 256;       // ... per thread, of each of q, k, decays
  constexpr int NV = (TB * PB + 255) / 256;       // values per thread
  __shared__ __attribute__((aligned(16))) float qs[TB][ROW];
  __shared__ __attribute__((aligned(16))) float ks[TB][ROW];
  __shared__ __attribute__((aligned(16))) float gs[TB][ROW];
  __shared__ float vs[TB][PB];
  __shared__ float bts[TB], kqs[TB];
  const int s = blockIdx.x, h = blockIdx.y;
  const int sl = slot[s];
  const int t0 = cu[s], t1 = cu[s + 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int chunk = lane % CH, pl = wave * PW + lane / CH;
  const int p = blockIdx.z * PB + pl;
  const bool live = p < dv;
  const int inner = H * dv;
  if (sl < 0) {  // padding rows: defined output, no state
    if (live && chunk == 0)
      for (int t = t0; t < t1; ++t) o[(long)t * inner + (long)h * dv + p] = 0.f;
    return;
  }
  if (t1 <= t0) return;
  const int n0 = chunk * 8;
  const int g = h / (H / Gk);
  float S[8];
  float* sp = state + (((long)sl * H + h) * dv + p) * dk + n0;
  const bool carried = ctx[s] > 0;
  const bool vec = (dk & 7) == 0 && n0 + 8 <= dk;
  if (carried && live && vec) {
    const float4 a = *reinterpret_cast<const float4*>(sp), b = *reinterpret_cast<const float4*>(sp + 4);
    S[0] = a.x; S[1] = a.y; S[2] = a.z; S[3] = a.w;
    S[4] = b.x; S[5] = b.y; S[6] = b.z; S[7] = b.w;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) S[i] = (carried && live && n0 + i < dk) ? sp[i] : 0.f;
  }
  const int boff = n0 + (n0 >> 6) * 4;
  const bool vec4 = (dk & 3) == 0;
  // the next tile's inputs, in registers while this tile's tokens are processed
  float4 rq[NB], rk[NB], rg[NB];
  float rv[NV], rs = 0.f;
  auto fetch = [&](int tb) {
    const int nt = min(TB, t1 - tb);
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const int i = threadIdx.x + 256 * u;
      const int tt = i / Q4, n = (i % Q4) * 4;
      rq[u] = rk[u] = rg[u] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (tt < nt && n < dk) {
        const float* qp = qn + ((long)(tb + tt) * Gk + g) * dk + n;
        const float* kp = kn + ((long)(tb + tt) * Gk + g) * dk + n;
        const float* gp = gd + ((long)(tb + tt) * H + h) * dk + n;
        if (vec4) {
          rq[u] = *reinterpret_cast<const float4*>(qp);
          rk[u] = *reinterpret_cast<const float4*>(kp);
          rg[u] = *reinterpret_cast<const float4*>(gp);
        } else {
          rq[u].x = qp[0]; rk[u].x = kp[0]; rg[u].x = gp[0];
          if (n + 1 < dk) { rq[u].y = qp[1]; rk[u].y = kp[1]; rg[u].y = gp[1]; }
          if (n + 2 < dk) { rq[u].z = qp[2]; rk[u].z = kp[2]; rg[u].z = gp[2]; }
          if (n + 3 < dk) { rq[u].w = qp[3]; rk[u].w = kp[3]; rg[u].w = gp[3]; }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int i = threadIdx.x + 256 * u;
      const int tt = i / PB, pg = blockIdx.z * PB + i % PB;
      rv[u] = (tt < nt && pg < dv) ? ldf(qkv + (long)(tb + tt) * stride + v_col + (long)h * dv + pg) : 0.f;
    }
    if (threadIdx.x < nt) rs = kq[(long)(tb + threadIdx.x) * Gk + g];
    else if (DELTA && threadIdx.x >= TB && threadIdx.x - TB < nt) rs = bt[(long)(tb + threadIdx.x - TB) * H + h];
  };
  fetch(t0);
  float* op = o + (long)t0 * inner + (long)h * dv + p;  // this lane's output column, advanced per tile
  for (int tb = t0; tb < t1; tb += TB) {
    const int nt = min(TB, t1 - tb);
    __syncthreads();  // the previous tile is consumed
#pragma unroll
    for (int u = 0; u < NB; ++u) {
      const int i = threadIdx.x + 256 * u;
      const int tt = i / Q4, n = (i % Q4) * 4;
      if (tt < TB) {
        const int off = tt * ROW + n + (n >> 6) * 4;
        *reinterpret_cast<float4*>(&qs[0][0] + off) = rq[u];
        *reinterpret_cast<float4*>(&ks[0][0] + off) = rk[u];
        *reinterpret_cast<float4*>(&gs[0][0] + off) = rg[u];
      }
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int i = threadIdx.x + 256 * u;
      if (i < TB * PB) (&vs[0][0])[i] = rv[u];
    }
    if (threadIdx.x < TB) kqs[threadIdx.x] = rs;
    else if (DELTA && threadIdx.x < 2 * TB) bts[threadIdx.x - TB] = rs;
    __syncthreads();
    if (tb + TB < t1) fetch(tb + TB);
#pragma unroll 2
    for (int tt = 0; tt < nt; ++tt) {
      const float4 g0 = *reinterpret_cast<const float4*>(&gs[tt][boff]);
      const float4 g1 = *reinterpret_cast<const float4*>(&gs[tt][boff + 4]);
      const float4 k0 = *reinterpret_cast<const float4*>(&ks[tt][boff]);
      const float4 k1 = *reinterpret_cast<const float4*>(&ks[tt][boff + 4]);
      const float4 q0 = *reinterpret_cast<const float4*>(&qs[tt][boff]);
      const float4 q1 = *reinterpret_cast<const float4*>(&qs[tt][boff + 4]);
      const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
      const float kv[8] = {k0.x, k0.y, k0.z, k0.w, k1.x, k1.y, k1.z, k1.w};
      const float qv[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
      float pk = 0.f, pq = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        S[i] *= gv[i];
        if (DELTA) pk += S[i] * kv[i];
        pq += S[i] * qv[i];
      }
      if (DELTA) pk = lanes_sum<CH>(pk);
      pq = lanes_sum<CH>(pq);
      const float v = vs[tt][pl];
      const float u = DELTA ? bts[tt] * (v - pk) : v;
#pragma unroll
      for (int i = 0; i < 8; ++i) S[i] += kv[i] * u;
      if (live && chunk == 0) op[(long)tt * inner] = pq + u * kqs[tt];
    }
    op += (long)TB * inner;
  }
  if (live) {
    if (vec) {
      *reinterpret_cast<float4*>(sp) = make_float4(S[0], S[1], S[2], S[3]);
      *reinterpret_cast<float4*>(sp + 4) = make_float4(S[4], S[5], S[6], S[7]);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (n0 + i < dk) sp[i] = S[i];
    }
  }
}

}  // namespace k8sllm

using namespace k8sllm;

template <typename T, bool DELTA>
static int launch_decay_scan(float* o, const void* qkv, long stride, int q_col, int k_col, int v_col, const void* z,
                             long z_stride, const float* z_bias, const float* a_log, float inv_tau, const void* beta,
                             long b_stride, float* state, const int* cu, const int* ctx, const int* slot, int S, int H,
                             int Gk, int dk, int dv, float q_scale, int unit, hipStream_t s) {
#define K8SLLM_DS(CH)                                                                                                  \
  hipLaunchKernelGGL((decay_scan_kernel<T, CH, DELTA>),                                                                \
                     dim3((unsigned)S, (unsigned)H, (unsigned)((dv + 256 / CH - 1) / (256 / CH))), dim3(256), 0, s, o,  \
                     (const T*)qkv, stride, q_col, k_col, v_col, (const T*)z, z_stride, z_bias, a_log, inv_tau,         \
                     (const T*)beta, b_stride, state, cu, ctx, slot, H, Gk, dk, dv, q_scale, unit)
  if (dk <= 16) K8SLLM_DS(2);
  else if (dk <= 32) K8SLLM_DS(4);
  else if (dk <= 64) K8SLLM_DS(8);
  else if (dk <= 128) K8SLLM_DS(16);
  else if (dk <= 256) K8SLLM_DS(32);
  else return -1;
#undef K8SLLM_DS
  return (int)hipGetLastError();
}

template <typename T, bool DELTA>
static int launch_decay_staged(float* o, const void* qkv, long stride, int q_col, int k_col, int v_col, const void* z,
                               long z_stride, const float* z_bias, const float* a_log, float inv_tau, const void* beta,
                               long b_stride, float* state, const int* cu, const int* ctx, const int* slot, int S, int H,
                               int Gk, int dk, int dv, float q_scale, int unit, float* ws, long rows, hipStream_t s) {
  float* qn = ws;
  float* kn = qn + rows * Gk * dk;
  float* gd = kn + rows * Gk * dk;
  float* kq = gd + rows * H * dk;
  float* bt = kq + rows * Gk;
  hipLaunchKernelGGL(decay_prep_kernel<T>, dim3((unsigned)rows), dim3(256), 0, s, qn, kn, gd, kq, bt,
                     (const T*)qkv, stride, q_col, k_col, (const T*)z, z_stride, z_bias, a_log, inv_tau, (const T*)beta,
                     b_stride, H, Gk, dk, q_scale, unit);
#define K8SLLM_DS(CH)                                                                                                  \
  hipLaunchKernelGGL((decay_scan_staged_kernel<T, CH, DELTA>),                                                         \
                     dim3((unsigned)S, (unsigned)H, (unsigned)((dv + 256 / CH - 1) / (256 / CH))), dim3(256), 0, s, o,  \
                     (const T*)qkv, stride, v_col, qn, kn, gd, kq, bt, state, cu, ctx, slot, H, Gk, dk, dv)
  if (dk <= 16) K8SLLM_DS(2);
  else if (dk <= 32) K8SLLM_DS(4);
  else if (dk <= 64) K8SLLM_DS(8);
  else if (dk <= 128) K8SLLM_DS(16);
  else if (dk <= 256) K8SLLM_DS(32);
  else return -1;
#undef K8SLLM_DS
  return (int)hipGetLastError();
}

extern "C" {

// floats of workspace the two-launch form needs for T rows
long k8sllm_hy_decay_scan_ws(long T, int H, int Gk, int dk) { return T * ((long)2 * Gk * dk + (long)H * dk + Gk + H); }

// beta == nullptr: no delta rule.  a_log == nullptr: decays sigmoid(z + bias)^(inv_tau).  ws != nullptr: the
// two-launch form for prompts, with k8sllm_hy_decay_scan_ws(T, ...) floats of workspace (T = rows of the step)
int k8sllm_hy_decay_scan(float* o, const void* qkv, long stride, int q_col, int k_col, int v_col, const void* z,
                         long z_stride, const float* z_bias, const float* a_log, float inv_tau, const void* beta,
                         long b_stride, float* state, const int* cu, const int* ctx, const int* slot, int S, int H, int Gk,
                         int dk, int dv, float q_scale, int unit, int f32, float* ws, long T, hipStream_t s) {
  if (S <= 0) return 0;
  if (Gk < 1 || H % Gk || dk < 1 || dv < 1) return -1;
  if (ws != nullptr) {
#define K8SLLM_ARGS2                                                                                                 \
  o, qkv, stride, q_col, k_col, v_col, z, z_stride, z_bias, a_log, inv_tau, beta, b_stride, state, cu, ctx, slot, S, H, \
      Gk, dk, dv, q_scale, unit, ws, T, s
    if (beta != nullptr)
      return f32 ? launch_decay_staged<float, true>(K8SLLM_ARGS2) : launch_decay_staged<bf16_t, true>(K8SLLM_ARGS2);
    return f32 ? launch_decay_staged<float, false>(K8SLLM_ARGS2) : launch_decay_staged<bf16_t, false>(K8SLLM_ARGS2);
#undef K8SLLM_ARGS2
  }
#define K8SLLM_ARGS                                                                                                  \
  o, qkv, stride, q_col, k_col, v_col, z, z_stride, z_bias, a_log, inv_tau, beta, b_stride, state, cu, ctx, slot, S, H, \
      Gk, dk, dv, q_scale, unit, s
  if (beta != nullptr) return f32 ? launch_decay_scan<float, true>(K8SLLM_ARGS) : launch_decay_scan<bf16_t, true>(K8SLLM_ARGS);
  return f32 ? launch_decay_scan<float, false>(K8SLLM_ARGS) : launch_decay_scan<bf16_t, false>(K8SLLM_ARGS);
#undef K8SLLM_ARGS
}
}
