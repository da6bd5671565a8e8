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
#include "hy_common.h"

namespace k8sllm {

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
}
