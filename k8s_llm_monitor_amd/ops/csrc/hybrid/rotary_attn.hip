// Rotary positions for grouped-query attention over the paged cache of window_attn.hip.
//   rotary_cache   in place on the fused rows [T][Hq*dk | G*dk | G*dv | ...]: the first 2 * nf entries of
//                  every query and key head turn by the angle position * freq[i] (nf frequencies, fp32;
//                  angle, sine and cosine fp32).  pairs == 0: entry i pairs with entry i + nf; pairs == 1:
//                  entry 2i pairs with entry 2i + 1.  Entries from 2 * nf on pass.  rot_off moves the turning
//                  block to entries rot_off .. rot_off + 2 nf of every head; rot_k == 0 leaves the keys as
//                  they are (already turned) and only copies them.  q_scale (optional, one
//                  number per query head) multiplies the whole query head in the same pass, before the one
//                  rounding to the activation dtype.  The keys (after the turn) and the values go to the
//                  pages at slots[t] (< 0: not written): keys [blocks][bs][G*dk], values dim-major
//                  [blocks][G][dv][bs].
//   rotary_norm_cache  the same turn with an RMS norm of every query and key head over its dk entries
//                  (fp32, eps inside the root): norm == 1 before the turn, times qw / kw [dk]; norm == 2 after
//                  the turn, no weight; norm == 0 none.  v_from_k: the row has no value columns and the value
//                  pages take the keys as projected (before norm and turn; dv == dk).  One wave per head, the
//                  head staged in LDS as fp32; the token's sines and cosines are evaluated once for all its
//                  heads; the result is rounded to the activation dtype once.
#include "hy_common.h"

namespace k8sllm {

constexpr int kMaxHeadDim = 1024;

template <typename T>
__global__ __launch_bounds__(256) void rotary_norm_cache_kernel(T* __restrict__ qkv, long stride, int Hq, int G, int dk,
                                                                int dv, const int* __restrict__ positions,
                                                                const float* __restrict__ freq, int nf, int pairs,
                                                                int norm, const float* __restrict__ qw,
                                                                const float* __restrict__ kw, float eps,
                                                                const float* __restrict__ q_scale,
                                                                T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                                const int* __restrict__ slots, int bs, int v_from_k) {
  extern __shared__ float heads[];  // [4 waves][dk], then the token's nf cosines and nf sines
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  T* row = qkv + t * stride;
  const int nq = Hq * dk, nk = G * dk, nv = G * dv;
  const float pos = (float)positions[t];
  const long slot = (slots != nullptr && k_cache != nullptr) ? slots[t] : -1;
  float* x = heads + wave * dk;
  float* cst = heads + 4 * dk;
  float* snt = cst + nf;
  for (int i = threadIdx.x; i < nf; i += 256) sincosf(pos * freq[i], snt + i, cst + i);  // once for all heads
  __syncthreads();
  // query heads, then key heads (contiguous in the row), a wave per head.  x is this wave's own LDS row: a
  // wave's LDS instructions execute in issue order, so a wave barrier (no reordering by the compiler) is all
  // that lanes reading what other lanes of the wave wrote need.
  for (int h = wave; h < Hq + G; h += 4) {
    T* hd = row + (long)h * dk;
    const bool is_k = h >= Hq;
    const int g = h - Hq;
    float ss = 0.f;
    for (int c = lane; c < dk; c += 64) {
      const float v = ldf(hd + c);
      x[c] = v;
      ss += v * v;
      if (is_k && v_from_k && slot >= 0) v_cache[((slot / bs) * nv + (long)g * dv + c) * bs + slot % bs] = hd[c];
    }
    if (norm == 1) {
      const float inv = 1.0f / sqrtf(wave_sum_dpp(ss) / (float)dk + eps);
      const float* w = is_k ? kw : qw;
      for (int c = lane; c < dk; c += 64) x[c] = x[c] * inv * w[c];
    }
    __builtin_amdgcn_wave_barrier();  // a lane turns pairs whose entries other lanes staged
    for (int i = lane; i < nf; i += 64) {
      const int a = pairs ? 2 * i : i, b = pairs ? 2 * i + 1 : i + nf;
      const float sn = snt[i], cs = cst[i];
      const float u = x[a], v = x[b];
      x[a] = u * cs - v * sn;
      x[b] = v * cs + u * sn;
    }
    __builtin_amdgcn_wave_barrier();
    float mul = 1.f;
    if (norm == 2) {
      float s2 = 0.f;
      for (int c = lane; c < dk; c += 64) s2 += x[c] * x[c];
      mul = 1.0f / sqrtf(wave_sum_dpp(s2) / (float)dk + eps);
    }
    if (!is_k && q_scale != nullptr) mul *= q_scale[h];
    T* kp = (is_k && slot >= 0) ? k_cache + slot * (long)nk + (long)g * dk : nullptr;
    for (int c = lane; c < dk; c += 64) {
      stf(hd + c, x[c] * mul);
      if (kp != nullptr) kp[c] = hd[c];
    }
    __builtin_amdgcn_wave_barrier();  // the next head reuses x
  }
  __syncthreads();  // the value copy below reads nothing the loop wrote, but keeps the workgroup together
  if (!v_from_k && slot >= 0)
    for (int c = threadIdx.x; c < nv; c += 256) v_cache[((slot / bs) * nv + c) * bs + slot % bs] = row[nq + nk + c];
}

template <typename T>
__global__ __launch_bounds__(256) void rotary_cache_kernel(T* __restrict__ qkv, long stride, int Hq, int G, int dk,
                                                           int dv, const int* __restrict__ positions,
                                                           const float* __restrict__ freq, int nf, int pairs,
                                                           int rot_off, int rot_k,
                                                           const float* __restrict__ q_scale,
                                                           T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                           const int* __restrict__ slots, int bs) {
  const long t = blockIdx.x;
  T* row = qkv + t * stride;
  const int nq = Hq * dk, nk = G * dk, nv = G * dv;
  const float pos = (float)positions[t];
  const long slot = (slots != nullptr && k_cache != nullptr) ? slots[t] : -1;
  T* kp = slot >= 0 ? k_cache + slot * (long)nk : nullptr;
  const int rest = dk - 2 * nf;  // entries of a head that do not turn: before rot_off and from rot_off + 2 nf on
  // the turning pairs of all query heads, then of all key heads: (head, i) owns entries (a, b)
  for (int e = threadIdx.x; e < (Hq + (rot_k ? G : 0)) * nf; e += 256) {
    const int h = e / nf, i = e - h * nf;
    const int a = rot_off + (pairs ? 2 * i : i), b = rot_off + (pairs ? 2 * i + 1 : i + nf);
    T* hd = row + (long)h * dk;  // query heads and key heads are contiguous in the row
    float sn, cs;
    sincosf(pos * freq[i], &sn, &cs);
    const float u = ldf(hd + a), v = ldf(hd + b);
    float x = u * cs - v * sn, y = v * cs + u * sn;
    if (h < Hq && q_scale != nullptr) {
      x *= q_scale[h];
      y *= q_scale[h];
    }
    stf(hd + a, x);
    stf(hd + b, y);
    if (h >= Hq && kp != nullptr) {
      kp[(h - Hq) * dk + a] = hd[a];
      kp[(h - Hq) * dk + b] = hd[b];
    }
  }
  if (rest > 0) {
    if (q_scale != nullptr)
      for (int e = threadIdx.x; e < Hq * rest; e += 256) {
        const int h = e / rest, r = e - h * rest, c = r < rot_off ? r : r + 2 * nf;
        T* p = row + (long)h * dk + c;
        stf(p, ldf(p) * q_scale[h]);
      }
    if (kp != nullptr && rot_k)
      for (int e = threadIdx.x; e < G * rest; e += 256) {
        const int g = e / rest, r = e - g * rest, c = r < rot_off ? r : r + 2 * nf;
        kp[g * dk + c] = row[nq + g * dk + c];
      }
  }
  if (kp != nullptr && !rot_k)
    for (int c = threadIdx.x; c < nk; c += 256) kp[c] = row[nq + c];
  if (slot >= 0)
    for (int c = threadIdx.x; c < nv; c += 256) v_cache[((slot / bs) * nv + c) * bs + slot % bs] = row[nq + nk + c];
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" {

int k8sllm_hy_rotary_cache(void* qkv, long stride, long T, int Hq, int G, int dk, int dv, const int* positions,
                           const float* freq, int nf, int pairs, int rot_off, int rot_k, const float* q_scale,
                           void* k_cache, void* v_cache, const int* slots, int bs, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (nf < 0 || rot_off < 0 || rot_off + 2 * nf > dk || Hq < 1 || G < 1) return -1;
  if (f32)
    hipLaunchKernelGGL(rotary_cache_kernel<float>, dim3(T), dim3(256), 0, s, (float*)qkv, stride, Hq, G, dk, dv,
                       positions, freq, nf, pairs, rot_off, rot_k, q_scale, (float*)k_cache, (float*)v_cache, slots, bs);
  else
    hipLaunchKernelGGL(rotary_cache_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (bf16_t*)qkv, stride, Hq, G, dk, dv,
                       positions, freq, nf, pairs, rot_off, rot_k, q_scale, (bf16_t*)k_cache, (bf16_t*)v_cache, slots, bs);
  return (int)hipGetLastError();
}

int k8sllm_hy_rotary_norm_cache(void* qkv, long stride, long T, int Hq, int G, int dk, int dv, const int* positions,
                                const float* freq, int nf, int pairs, int norm, const float* qw, const float* kw,
                                float eps, const float* q_scale, void* k_cache, void* v_cache, const int* slots, int bs,
                                int v_from_k, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (nf < 0 || 2 * nf > dk || Hq < 1 || G < 1 || dk > kMaxHeadDim || norm < 0 || norm > 2) return -1;
  if (norm == 1 && (qw == nullptr || kw == nullptr)) return -1;
  if (v_from_k && dv != dk) return -1;
  const size_t lds = (4 * (size_t)dk + 2 * (size_t)nf) * sizeof(float);
  if (f32)
    hipLaunchKernelGGL(rotary_norm_cache_kernel<float>, dim3(T), dim3(256), lds, s, (float*)qkv, stride, Hq, G, dk, dv,
                       positions, freq, nf, pairs, norm, qw, kw, eps, q_scale, (float*)k_cache, (float*)v_cache, slots, bs,
                       v_from_k);
  else
    hipLaunchKernelGGL(rotary_norm_cache_kernel<bf16_t>, dim3(T), dim3(256), lds, s, (bf16_t*)qkv, stride, Hq, G, dk, dv,
                       positions, freq, nf, pairs, norm, qw, kw, eps, q_scale, (bf16_t*)k_cache, (bf16_t*)v_cache, slots,
                       bs, v_from_k);
  return (int)hipGetLastError();
}
}
