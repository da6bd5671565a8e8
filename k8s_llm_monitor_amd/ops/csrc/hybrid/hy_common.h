// Helpers shared by the layer-list decoders' kernels: activations are either bf16 (raw 16-bit
// patterns, common.h) or fp32, selected by a template parameter; all arithmetic is fp32.
#pragma once
#include "common.h"

namespace k8sllm {

template <typename T>
__device__ __forceinline__ float ldf(const T* p);
template <>
__device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf2f(*p); }

template <typename T>
__device__ __forceinline__ void stf(T* p, float v);
template <>
__device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = f2bf(v); }

// element i of a tensor whose dtype is only known at run time: 1 = bf16, 2 = fp32
__device__ __forceinline__ float ld_any(const void* p, int dt, long i) {
  return dt == 2 ? reinterpret_cast<const float*>(p)[i] : bf2f(reinterpret_cast<const bf16_t*>(p)[i]);
}

// 8 consecutive elements (16-byte aligned for bf16, 32-byte for fp32) as floats, and back
__device__ __forceinline__ void load8(const bf16_t* p, float* f) { unpack8(*reinterpret_cast<const uint4*>(p), f); }
__device__ __forceinline__ void load8(const float* p, float* f) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w;
  f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}
__device__ __forceinline__ void store8(bf16_t* p, const float* f) { *reinterpret_cast<uint4*>(p) = pack8(f); }
__device__ __forceinline__ void store8(float* p, const float* f) {
  *reinterpret_cast<float4*>(p) = make_float4(f[0], f[1], f[2], f[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(f[4], f[5], f[6], f[7]);
}
__device__ __forceinline__ void load8_any(const void* p, int dt, long i, float* f) {
  if (dt == 2) load8(reinterpret_cast<const float*>(p) + i, f);
  else load8(reinterpret_cast<const bf16_t*>(p) + i, f);
}

// Wave-wide butterflies without the LDS crossbar: quads and rows by DPP (quad_perm, the row's mirror
// controls pair equal partial results), rows 0/1 and 2/3 by v_permlane16_swap, the halves by
// v_permlane32_swap.  Every lane ends with the result.
#define K8SLLM_DPP(v, ctrl) __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), ctrl, 0xf, 0xf, true))
__device__ __forceinline__ float xor16_sum(float x) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float xor16_max(float x) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float xor32_sum_f(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float xor32_max_f(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float wave_sum_dpp(float v) {
  v += K8SLLM_DPP(v, 0xB1);
  v += K8SLLM_DPP(v, 0x4E);
  v += K8SLLM_DPP(v, 0x141);
  v += K8SLLM_DPP(v, 0x140);
  return xor32_sum_f(xor16_sum(v));
}
__device__ __forceinline__ float wave_max_dpp(float v) {
  v = fmaxf(v, K8SLLM_DPP(v, 0xB1));
  v = fmaxf(v, K8SLLM_DPP(v, 0x4E));
  v = fmaxf(v, K8SLLM_DPP(v, 0x141));
  v = fmaxf(v, K8SLLM_DPP(v, 0x140));
  return xor32_max_f(xor16_max(v));
}

__device__ __forceinline__ float silu_f(float z) { return z / (1.f + __expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }

// the segment that holds row r: largest s with cu[s] <= r (cu has S + 1 entries, cu[0] = 0)
__device__ __forceinline__ int find_segment(const int* __restrict__ cu, int S, int r) {
  int lo = 0, hi = S - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu[mid] <= r) lo = mid; else hi = mid - 1;
  }
  return lo;
}

}  // namespace k8sllm
