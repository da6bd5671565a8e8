// fp32 residual stream of the layer-list decoders.
//   embed_pos         x[t] = embed[id] + pos[position]            (fp32 rows)
//   add_norm          residual += a0 + a1 + a2 + vec;  out = residual / rms(residual) * (w | 1 + w)
//   gated_group_norm  out = group_rms_norm(y * silu(z)) * w       (y fp32, groups of equal size)
//   swiglu            out = silu(gu[:, :f]) * gu[:, f:]
//   norm_shift        h[t] = x[t] / rms(x[t]) * w;  out[t] = h[t] + (h[t-1] - h[t]) * mu, the row before
//                     a segment from the sequence's state slot; shift_state advances the slots
//   depth_mix         stack[n] += addend;  stack[n+1] = sum_j coef[j] * stack[j], j = 0 .. n
//   activation        erf GELU, tanh GELU, xIELU or SiLU, elementwise in fp32 (also over a column range)
//   gated_add_norm    residual += mult * y * sigmoid(gate + bias);  out = residual / rms(residual) * w
//   glu               out = act(gu[:, :f]) * gu[:, f:2f]           (rows may be wider than 2f)
//   norm_gate         out = y / rms(y) * w * sigmoid(z)            (y fp32)
//   sigmoid_gate      x *= sigmoid(z), in place
//   softcap           x = cap * tanh(x / cap), in place (fp32 logits)
//   sum_norm          residual += s0 a0 + s1 a1 + y / rms(y) * wy;  out = RMS or layer norm of it times w
//                     (or the new residual itself, rounded to the activation dtype)
//   gated_lookup      out = gelu_tanh(gate) * table[id][col : col + n]
#include "hy_common.h"

namespace k8sllm {

template <typename T>
__global__ __launch_bounds__(256) void embed_pos_kernel(float* __restrict__ out, const int* __restrict__ ids,
                                                        const int* __restrict__ positions, const T* __restrict__ emb,
                                                        const T* __restrict__ pos, const int* __restrict__ src,
                                                        const int* __restrict__ prev, int d, int vocab, int max_pos,
                                                        float scale) {
  const long t = blockIdx.x;
  int id = ids[t];
  if (src != nullptr && src[t] >= 0) id = prev[src[t]];
  id = min(max(id, 0), vocab - 1);
  const T* e = emb + (long)id * d;
  const T* p = nullptr;
  if (pos != nullptr) p = pos + (long)min(max(positions[t], 0), max_pos - 1) * d;
  for (int c = threadIdx.x; c < d; c += 256) out[t * d + c] = ldf(e + c) * scale + (p != nullptr ? ldf(p + c) : 0.f);
}

template <typename T>
__global__ __launch_bounds__(256) void add_norm_kernel(T* __restrict__ out, float* __restrict__ residual,
                                                       const void* a0, int t0, const void* a1, int t1, const void* a2,
                                                       int t2, const float* __restrict__ vec,
                                                       const float* __restrict__ w, int d, float eps, int one_plus) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  float* r = residual + row * d;
  float ss = 0.f;
  if ((d & 7) == 0) {  // 8 columns per thread and trip, 16 / 32-byte accesses
    for (int c = threadIdx.x * 8; c < d; c += 2048) {
      float x[8], a[8];
      load8(r + c, x);
      if (t0) {
        load8_any(a0, t0, row * d + c, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += a[i];
      }
      if (t1) {
        load8_any(a1, t1, row * d + c, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += a[i];
      }
      if (t2) {
        load8_any(a2, t2, row * d + c, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += a[i];
      }
      if (vec != nullptr) {
        load8(vec + c, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += a[i];
      }
      store8(r + c, x);
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
    }
    ss = block_sum<256>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    for (int c = threadIdx.x * 8; c < d; c += 2048) {  // each thread re-reads what it wrote
      float x[8], g[8];
      load8(r + c, x);
      load8(w + c, g);
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] *= inv * (one_plus ? 1.f + g[i] : g[i]);
      store8(out + row * d + c, x);
    }
    return;
  }
  for (int c = threadIdx.x; c < d; c += 256) {
    float x = r[c];
    if (t0) x += ld_any(a0, t0, row * d + c);
    if (t1) x += ld_any(a1, t1, row * d + c);
    if (t2) x += ld_any(a2, t2, row * d + c);
    if (vec != nullptr) x += vec[c];
    r[c] = x;
    ss += x * x;
  }
  ss = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += 256) {  // each thread re-reads what it wrote
    const float g = one_plus ? 1.f + w[c] : w[c];
    stf(out + row * d + c, r[c] * inv * g);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(T* __restrict__ out, const float* __restrict__ y,
                                                               const T* __restrict__ z, long z_stride,
                                                               const float* __restrict__ w, int n, int groups,
                                                               float eps, int after) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const int g = blockIdx.y, gs = n / groups;
  const float* yr = y + row * n + (long)g * gs;
  const T* zr = z + row * z_stride + (long)g * gs;
  float ss = 0.f;
  if (after) {  // the norm first, then a sigmoid gate
    for (int c = threadIdx.x; c < gs; c += 256) ss += yr[c] * yr[c];
    ss = block_sum<256>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
    for (int c = threadIdx.x; c < gs; c += 256)
      stf(out + row * n + (long)g * gs + c,
          yr[c] * inv * w[(long)g * gs + c] * (after == 2 ? silu_f(ldf(zr + c)) : sigmoid_f(ldf(zr + c))));
    return;
  }
  for (int c = threadIdx.x; c < gs; c += 256) {
    const float v = yr[c] * silu_f(ldf(zr + c));
    ss += v * v;
  }
  ss = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
  for (int c = threadIdx.x; c < gs; c += 256) {
    const float v = yr[c] * silu_f(ldf(zr + c));
    stf(out + row * n + (long)g * gs + c, v * inv * w[(long)g * gs + c]);
  }
}

// The norm-first forms (after 1 / 2) with small groups (a head's values): one wave per (row, group), the
// group's at most 64 NPL values in registers, so y is read once and no workgroup barrier is needed.
template <typename T, int NPL>
__global__ __launch_bounds__(256) void group_norm_gate_wave_kernel(T* __restrict__ out, const float* __restrict__ y,
                                                                   const T* __restrict__ z, long z_stride,
                                                                   const float* __restrict__ w, long rows, int n,
                                                                   int groups, float eps, int after) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long idx = (long)blockIdx.x * 4 + wave;
  if (idx >= rows * groups) return;
  const long row = idx / groups;
  const int g = (int)(idx - row * groups), gs = n / groups;
  const float* yr = y + row * n + (long)g * gs;
  const T* zr = z + row * z_stride + (long)g * gs;
  float v[NPL], gt[NPL];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const int c = lane + 64 * i;
    v[i] = c < gs ? yr[c] : 0.f;
    gt[i] = c < gs ? ldf(zr + c) : 0.f;
    ss += v[i] * v[i];
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
#pragma unroll
  for (int i = 0; i < NPL; ++i) {
    const int c = lane + 64 * i;
    if (c < gs)
      stf(out + row * n + (long)g * gs + c,
          v[i] * inv * w[(long)g * gs + c] * (after == 2 ? silu_f(gt[i]) : sigmoid_f(gt[i])));
  }
}

// residual += mult * y * sigmoid(gate + bias), then the RMSNorm of the new residual times w.  y: any
// float dtype, contiguous; gate: activation dtype, rows g_stride apart (a column range of a wider
// projection).  Sum, sigmoid and norm are fp32.
template <typename T>
__global__ __launch_bounds__(256) void gated_add_norm_kernel(T* __restrict__ out, float* __restrict__ residual,
                                                             const void* __restrict__ y, int yt,
                                                             const T* __restrict__ gate, long g_stride,
                                                             const float* __restrict__ bias, float mult,
                                                             const float* __restrict__ w, int d, float eps,
                                                             int one_plus, int vec) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  float* r = residual + row * d;
  const T* gr = gate + row * g_stride;
  float ss = 0.f;
  if (vec) {  // d, the gate's row stride and column offset are multiples of 8
    for (int c = threadIdx.x * 8; c < d; c += 2048) {
      float x[8], a[8], g[8], b[8];
      load8(r + c, x);
      load8_any(y, yt, row * d + c, a);
      load8(gr + c, g);
      load8(bias + c, b);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        x[i] += mult * a[i] * sigmoid_f(g[i] + b[i]);
        ss += x[i] * x[i];
      }
      store8(r + c, x);
    }
    ss = block_sum<256>(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)d + eps);
    for (int c = threadIdx.x * 8; c < d; c += 2048) {  // each thread re-reads what it wrote
      float x[8], g[8];
      load8(r + c, x);
      load8(w + c, g);
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] *= inv * (one_plus ? 1.f + g[i] : g[i]);
      store8(out + row * d + c, x);
    }
    return;
  }
  for (int c = threadIdx.x; c < d; c += 256) {
    const float x = r[c] + mult * ld_any(y, yt, row * d + c) * sigmoid_f(ldf(gr + c) + bias[c]);
    r[c] = x;
    ss += x * x;
  }
  ss = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += 256) stf(out + row * d + c, r[c] * inv * (one_plus ? 1.f + w[c] : w[c]));
}

template <typename T>
__global__ __launch_bounds__(256) void swiglu_kernel(T* __restrict__ out, const T* __restrict__ gu, long rows, int f) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * f) return;
  const long r = i / f;
  const int c = (int)(i - r * f);
  stf(out + i, silu_f(ldf(gu + r * 2 * f + c)) * ldf(gu + r * 2 * f + f + c));
}


// Token-shifted RMSNorm, one workgroup per row.  The row also norms its predecessor (the same fp32
// arithmetic in the same order as that row's own workgroup, so a prompt cut anywhere gives the same
// values); a segment's first row reads the sequence's slot instead (zeros for a fresh sequence).  A
// one-row segment writes its h to the slot right here (each thread overwrites only what it has read);
// longer segments leave that to shift_state_kernel, launched after every row has read the old slot.
template <typename T>
__global__ __launch_bounds__(256) void norm_shift_kernel(T* __restrict__ out, const float* __restrict__ x,
                                                         const float* __restrict__ w, const float* __restrict__ mu,
                                                         float* __restrict__ state, const int* __restrict__ cu,
                                                         const int* __restrict__ ctx, const int* __restrict__ slot,
                                                         int S, int d, float eps, int one_plus, int advance) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  const int s = find_segment(cu, S, (int)row);
  const bool first = row == cu[s], single = first && cu[s + 1] - cu[s] == 1;
  const int sl = slot[s];
  const float* xr = x + row * d;
  const float* xp = xr - d;
  float ss = 0.f, sp = 0.f;
  for (int c = threadIdx.x; c < d; c += 256) {
    const float v = xr[c];
    ss += v * v;
    if (!first) {
      const float u = xp[c];
      sp += u * u;
    }
  }
  ss = block_sum<256>(ss, red);
  if (!first) sp = block_sum<256>(sp, red);
  const float inv = 1.0f / sqrtf(ss / (float)d + eps), invp = 1.0f / sqrtf(sp / (float)d + eps);
  const bool from_state = first && sl >= 0 && ctx[s] > 0;
  float* st = sl >= 0 ? state + (long)sl * d : nullptr;
  for (int c = threadIdx.x; c < d; c += 256) {
    const float g = one_plus ? 1.f + w[c] : w[c];
    const float h = xr[c] * inv * g;
    float hp = 0.f;
    if (!first) hp = xp[c] * invp * g;
    else if (from_state) hp = st[c];
    stf(out + row * d + c, h + (hp - h) * mu[c]);
    if (advance && single && st != nullptr) st[c] = h;
  }
}

template <int DUMMY>
__global__ __launch_bounds__(256) void shift_state_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                          float* __restrict__ state, const int* __restrict__ cu,
                                                          const int* __restrict__ slot, int d, float eps,
                                                          int one_plus) {
  __shared__ float red[4];
  const int s = blockIdx.x;
  const int n = cu[s + 1] - cu[s], sl = slot[s];
  if (n < 2 || sl < 0) return;  // one-row segments were advanced by their own row
  const float* xr = x + (long)(cu[s + 1] - 1) * d;
  float ss = 0.f;
  for (int c = threadIdx.x; c < d; c += 256) ss += xr[c] * xr[c];
  ss = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)d + eps);
  for (int c = threadIdx.x; c < d; c += 256) state[(long)sl * d + c] = xr[c] * inv * (one_plus ? 1.f + w[c] : w[c]);
}

constexpr int kMaxDepth = 256;

// 4 consecutive elements per thread; entry n of the stack is completed with the addend on the way.
__global__ __launch_bounds__(256) void depth_mix_kernel(float* __restrict__ stack, long plane, int n,
                                                        const void* __restrict__ addend, int adt,
                                                        const float* __restrict__ coef) {
  __shared__ float cf[kMaxDepth];
  for (int j = threadIdx.x; j <= n; j += 256) cf[j] = coef[j];
  __syncthreads();
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= plane) return;
  float4 top = *reinterpret_cast<const float4*>(stack + (long)n * plane + i);
  if (adt) {
    top.x += ld_any(addend, adt, i);
    top.y += ld_any(addend, adt, i + 1);
    top.z += ld_any(addend, adt, i + 2);
    top.w += ld_any(addend, adt, i + 3);
    *reinterpret_cast<float4*>(stack + (long)n * plane + i) = top;
  }
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int j = 0; j < n; ++j) {
    const float4 v = *reinterpret_cast<const float4*>(stack + (long)j * plane + i);
    const float a = cf[j];
    acc.x += a * v.x; acc.y += a * v.y; acc.z += a * v.z; acc.w += a * v.w;
  }
  const float a = cf[n];
  acc.x += a * top.x; acc.y += a * top.y; acc.z += a * top.z; acc.w += a * top.w;
  *reinterpret_cast<float4*>(stack + (long)(n + 1) * plane + i) = acc;
}

// any T * d: one element per thread
__global__ __launch_bounds__(256) void depth_mix_scalar_kernel(float* __restrict__ stack, long plane, int n,
                                                               const void* __restrict__ addend, int adt,
                                                               const float* __restrict__ coef) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= plane) return;
  float top = stack[(long)n * plane + i];
  if (adt) {
    top += ld_any(addend, adt, i);
    stack[(long)n * plane + i] = top;
  }
  float acc = 0.f;
  for (int j = 0; j < n; ++j) acc += coef[j] * stack[(long)j * plane + i];
  stack[(long)(n + 1) * plane + i] = acc + coef[n] * top;
}

// KIND 0: erf GELU, 1: tanh GELU, 2: xIELU (a z^2 + z/2 above zero, b (exp(z) - 1 - z) + z/2 below), 3: SiLU,
// 4: ReLU
template <int KIND>
__device__ __forceinline__ float act_f(float z, float a, float b) {
  if (KIND == 4) return fmaxf(z, 0.f);
  if (KIND == 0) return 0.5f * z * (1.f + erff(z * 0.70710678118654752f));
  if (KIND == 1) return 0.5f * z * (1.f + tanhf(0.79788456080286536f * (z + 0.044715f * z * z * z)));
  if (KIND == 3) return z / (1.f + expf(-z));
  return z > 0.f ? a * z * z + 0.5f * z : b * (expm1f(z) - z) + 0.5f * z;
}

// out [rows, n] (contiguous) = act(x[:, 0:n]) where x's rows are x_stride apart; 8 columns per thread
// where n, the stride and the column offset are multiples of 8 (vec)
template <typename T, int KIND>
__global__ __launch_bounds__(256) void activation_cols_kernel(T* __restrict__ out, const T* __restrict__ x,
                                                              long x_stride, long rows, int n, int vec) {
  const int per = vec ? n / 8 : n;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * per) return;
  const long r = i / per;
  const int c = (int)(i - r * per);
  if (vec) {
    float v[8];
    load8(x + r * x_stride + 8 * c, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = act_f<KIND>(v[k], 0.f, 0.f);
    store8(out + r * n + 8 * c, v);
    return;
  }
  stf(out + r * n + c, act_f<KIND>(ldf(x + r * x_stride + c), 0.f, 0.f));
}

// KIND 5: the clamped unit g sigmoid(1.702 g) (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit);
// others: act(gate) * up
template <int KIND>
__device__ __forceinline__ float glu_unit(float g, float u, float limit) {
  if (KIND == 5) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g * sigmoid_f(1.702f * g) * (u + 1.f);
  }
  return act_f<KIND>(g, 0.f, 0.f) * u;
}

// out [rows, f] = act(gu[:, 0:f]) * gu[:, f:2f], gu's rows g_stride apart
template <typename T, int KIND>
__global__ __launch_bounds__(256) void glu_kernel(T* __restrict__ out, const T* __restrict__ gu, long g_stride,
                                                  long rows, int f, int vec, float limit) {
  const int per = vec ? f / 8 : f;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * per) return;
  const long r = i / per;
  const int c = (int)(i - r * per);
  const T* g = gu + r * g_stride;
  if (vec) {
    float a[8], u[8];
    load8(g + 8 * c, a);
    load8(g + f + 8 * c, u);
#pragma unroll
    for (int k = 0; k < 8; ++k) a[k] = glu_unit<KIND>(a[k], u[k], limit);
    store8(out + r * f + 8 * c, a);
    return;
  }
  stf(out + r * f + c, glu_unit<KIND>(ldf(g + c), ldf(g + f + c), limit));
}

// x [rows, n] (contiguous) *= sigmoid(z[:, 0:n]), z's rows z_stride apart
template <typename T>
__global__ __launch_bounds__(256) void sigmoid_gate_kernel(T* __restrict__ x, const T* __restrict__ z, long z_stride,
                                                           long rows, int n, int vec) {
  const int per = vec ? n / 8 : n;
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * per) return;
  const long r = i / per;
  const int c = (int)(i - r * per);
  if (vec) {
    float a[8], g[8];
    load8(x + r * n + 8 * c, a);
    load8(z + r * z_stride + 8 * c, g);
#pragma unroll
    for (int k = 0; k < 8; ++k) a[k] *= sigmoid_f(g[k]);
    store8(x + r * n + 8 * c, a);
    return;
  }
  stf(x + r * n + c, ldf(x + r * n + c) * sigmoid_f(ldf(z + r * z_stride + c)));
}

__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ x, long n, float cap) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

template <typename T, int KIND>
__global__ __launch_bounds__(256) void activation_kernel(T* __restrict__ out, const T* __restrict__ x, long n, float a,
                                                         float b) {
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i >= n) return;
  if (i + 8 <= n) {  // n a multiple of 8 whenever rows are: 16 / 32-byte accesses
    float v[8];
    load8(x + i, v);
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = act_f<KIND>(v[k], a, b);
    store8(out + i, v);
    return;
  }
  for (long k = i; k < n; ++k) stf(out + k, act_f<KIND>(ldf(x + k), a, b));
}

// residual += s0 a0 + s1 a1 + y / sqrt(mean(y^2) + eps) * wy, then out = the norm of the new residual times w:
// center 0 the RMS norm, 1 the layer norm (x - mean) / sqrt(mean((x - mean)^2) + eps), the variance taken
// from the deviations in a pass of its own (no cancellation).  w == nullptr: out = the new residual,
// rounded to T.  a0, a1, y: any float dtype (0 = absent), contiguous [rows, d].  One workgroup per row; a
// thread re-reads only what it wrote itself.
template <typename T>
__global__ __launch_bounds__(256) void sum_norm_kernel(T* __restrict__ out, float* __restrict__ residual, const void* a0,
                                                       int t0, float s0, const void* a1, int t1, float s1,
                                                       const void* y, int ty, const float* __restrict__ wy,
                                                       const float* __restrict__ w, int d, float eps, int center,
                                                       int one_plus) {
  __shared__ float red[4];
  const long row = blockIdx.x;
  float* r = residual + row * d;
  const bool v8 = (d & 7) == 0;
  const int step = v8 ? 8 : 1;
  float yinv = 0.f;
  if (ty) {
    float ss = 0.f;
    for (int c = threadIdx.x * step; c < d; c += 256 * step) {
      if (v8) {
        float a[8];
        load8_any(y, ty, row * d + c, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) ss += a[i] * a[i];
      } else {
        const float a = ld_any(y, ty, row * d + c);
        ss += a * a;
      }
    }
    ss = block_sum<256>(ss, red);
    yinv = 1.0f / sqrtf(ss / (float)d + eps);
    __syncthreads();  // red is reused below
  }
  float sum = 0.f, ssq = 0.f;
  for (int c = threadIdx.x * step; c < d; c += 256 * step) {
    if (v8) {
      float x[8], a[8], g[8];
      load8(r + c, x);
      if (t0) {
        load8_any(a0, t0, row * d + c, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += s0 * a[i];
      }
      if (t1) {
        load8_any(a1, t1, row * d + c, a);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += s1 * a[i];
      }
      if (ty) {
        load8_any(y, ty, row * d + c, a);
        load8(wy + c, g);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += a[i] * yinv * g[i];
      }
      store8(r + c, x);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        sum += x[i];
        ssq += x[i] * x[i];
      }
      if (w == nullptr) store8(out + row * d + c, x);
    } else {
      float x = r[c];
      if (t0) x += s0 * ld_any(a0, t0, row * d + c);
      if (t1) x += s1 * ld_any(a1, t1, row * d + c);
      if (ty) x += ld_any(y, ty, row * d + c) * yinv * wy[c];
      r[c] = x;
      sum += x;
      ssq += x * x;
      if (w == nullptr) stf(out + row * d + c, x);
    }
  }
  if (w == nullptr) return;
  float mean = 0.f;
  if (center) {
    mean = block_sum<256>(sum, red) / (float)d;
    __syncthreads();
    ssq = 0.f;
    for (int c = threadIdx.x * step; c < d; c += 256 * step) {
      if (v8) {
        float x[8];
        load8(r + c, x);
#pragma unroll
        for (int i = 0; i < 8; ++i) ssq += (x[i] - mean) * (x[i] - mean);
      } else {
        ssq += (r[c] - mean) * (r[c] - mean);
      }
    }
  }
  ssq = block_sum<256>(ssq, red);
  const float inv = 1.0f / sqrtf(ssq / (float)d + eps);
  for (int c = threadIdx.x * step; c < d; c += 256 * step) {
    if (v8) {
      float x[8], g[8];
      load8(r + c, x);
      load8(w + c, g);
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = (x[i] - mean) * inv * (one_plus ? 1.f + g[i] : g[i]);
      store8(out + row * d + c, x);
    } else {
      stf(out + row * d + c, (r[c] - mean) * inv * (one_plus ? 1.f + w[c] : w[c]));
    }
  }
}

// out[t][c] = gelu_tanh(gate[t][c]) * table[id(t)][col + c]; ids resolved as in embed_pos
template <typename T>
__global__ __launch_bounds__(256) void gated_lookup_kernel(T* __restrict__ out, const T* __restrict__ gate,
                                                           const T* __restrict__ table, long t_stride, int col,
                                                           const int* __restrict__ ids, const int* __restrict__ src,
                                                           const int* __restrict__ prev, long rows, int n, int vocab) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * n) return;
  const long t = i / n;
  const int c = (int)(i - t * n);
  int id = ids[t];
  if (src != nullptr && src[t] >= 0) id = prev[src[t]];
  id = min(max(id, 0), vocab - 1);
  stf(out + i, act_f<1>(ldf(gate + i), 0.f, 0.f) * ldf(table + (long)id * t_stride + col + c));
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" {

int k8sllm_hy_embed_pos(float* out, const int* ids, const int* positions, const void* emb, const void* pos,
                        const int* src, const int* prev, long T, int d, int vocab, int max_pos, float scale, int f32,
                        hipStream_t s) {
  if (T <= 0) return 0;
  if (f32)
    hipLaunchKernelGGL(embed_pos_kernel<float>, dim3(T), dim3(256), 0, s, out, ids, positions, (const float*)emb,
                       (const float*)pos, src, prev, d, vocab, max_pos, scale);
  else
    hipLaunchKernelGGL(embed_pos_kernel<bf16_t>, dim3(T), dim3(256), 0, s, out, ids, positions, (const bf16_t*)emb,
                       (const bf16_t*)pos, src, prev, d, vocab, max_pos, scale);
  return (int)hipGetLastError();
}

int k8sllm_hy_add_norm(void* out, float* residual, const void* a0, int t0, const void* a1, int t1, const void* a2,
                       int t2, const float* vec, const float* w, long rows, int d, float eps, int one_plus, int f32,
                       hipStream_t s) {
  if (rows <= 0) return 0;
  if (f32)
    hipLaunchKernelGGL(add_norm_kernel<float>, dim3(rows), dim3(256), 0, s, (float*)out, residual, a0, t0, a1, t1, a2,
                       t2, vec, w, d, eps, one_plus);
  else
    hipLaunchKernelGGL(add_norm_kernel<bf16_t>, dim3(rows), dim3(256), 0, s, (bf16_t*)out, residual, a0, t0, a1, t1,
                       a2, t2, vec, w, d, eps, one_plus);
  return (int)hipGetLastError();
}

// after 0: group_rms_norm(y * silu(z)) * w;  1: group_rms_norm(y) * w * sigmoid(z);  2: ... * silu(z)
int k8sllm_hy_gated_group_norm(void* out, const float* y, const void* z, long z_stride, const float* w, long rows,
                               int n, int groups, float eps, int after, int f32, hipStream_t s) {
  if (rows <= 0) return 0;
  if (groups < 1 || n % groups) return -1;
  const int gs = n / groups;
  if (after && groups > 1 && gs <= 256) {  // per-head norms: a wave per group
    const dim3 grid((unsigned)((rows * groups + 3) / 4));
#define K8SLLM_GW(T_, NPL)                                                                                         \
  hipLaunchKernelGGL((group_norm_gate_wave_kernel<T_, NPL>), grid, dim3(256), 0, s, (T_*)out, y, (const T_*)z, z_stride, \
                     w, rows, n, groups, eps, after)
    if (f32) {
      if (gs <= 64) K8SLLM_GW(float, 1); else if (gs <= 128) K8SLLM_GW(float, 2); else K8SLLM_GW(float, 4);
    } else {
      if (gs <= 64) K8SLLM_GW(bf16_t, 1); else if (gs <= 128) K8SLLM_GW(bf16_t, 2); else K8SLLM_GW(bf16_t, 4);
    }
#undef K8SLLM_GW
    return (int)hipGetLastError();
  }
  if (f32)
    hipLaunchKernelGGL(gated_group_norm_kernel<float>, dim3(rows, groups), dim3(256), 0, s, (float*)out, y,
                       (const float*)z, z_stride, w, n, groups, eps, after);
  else
    hipLaunchKernelGGL(gated_group_norm_kernel<bf16_t>, dim3(rows, groups), dim3(256), 0, s, (bf16_t*)out, y,
                       (const bf16_t*)z, z_stride, w, n, groups, eps, after);
  return (int)hipGetLastError();
}

// yt: 1 = bf16, 2 = fp32; vec: 8-wide accesses are aligned (checked by the caller)
int k8sllm_hy_gated_add_norm(void* out, float* residual, const void* y, int yt, const void* gate, long g_stride,
                             const float* bias, float mult, const float* w, long rows, int d, float eps, int one_plus,
                             int vec, int f32, hipStream_t s) {
  if (rows <= 0) return 0;
  if (f32)
    hipLaunchKernelGGL(gated_add_norm_kernel<float>, dim3(rows), dim3(256), 0, s, (float*)out, residual, y, yt,
                       (const float*)gate, g_stride, bias, mult, w, d, eps, one_plus, vec);
  else
    hipLaunchKernelGGL(gated_add_norm_kernel<bf16_t>, dim3(rows), dim3(256), 0, s, (bf16_t*)out, residual, y, yt,
                       (const bf16_t*)gate, g_stride, bias, mult, w, d, eps, one_plus, vec);
  return (int)hipGetLastError();
}

// kind: 1 tanh GELU, 3 SiLU, 4 ReLU, 5 the clamped unit (limit)
int k8sllm_hy_glu(void* out, const void* gu, long g_stride, long rows, int f, int kind, float limit, int vec, int f32,
                  hipStream_t s) {
  const long n = rows * (vec ? f / 8 : f);
  if (n <= 0) return 0;
  const dim3 g((unsigned)((n + 255) / 256));
#define K8SLLM_GLU(T, K) hipLaunchKernelGGL((glu_kernel<T, K>), g, dim3(256), 0, s, (T*)out, (const T*)gu, g_stride, rows, f, vec, limit)
  if (f32) {
    if (kind == 1) K8SLLM_GLU(float, 1); else if (kind == 3) K8SLLM_GLU(float, 3); else if (kind == 4) K8SLLM_GLU(float, 4);
    else if (kind == 5) K8SLLM_GLU(float, 5); else return -1;
  } else {
    if (kind == 1) K8SLLM_GLU(bf16_t, 1); else if (kind == 3) K8SLLM_GLU(bf16_t, 3); else if (kind == 4) K8SLLM_GLU(bf16_t, 4);
    else if (kind == 5) K8SLLM_GLU(bf16_t, 5); else return -1;
  }
#undef K8SLLM_GLU
  return (int)hipGetLastError();
}

int k8sllm_hy_activation_cols(void* out, const void* x, long x_stride, long rows, int n, int kind, int vec, int f32,
                              hipStream_t s) {
  const long tot = rows * (vec ? n / 8 : n);
  if (tot <= 0) return 0;
  const dim3 g((unsigned)((tot + 255) / 256));
#define K8SLLM_AC(T, K) hipLaunchKernelGGL((activation_cols_kernel<T, K>), g, dim3(256), 0, s, (T*)out, (const T*)x, x_stride, rows, n, vec)
  if (f32) {
    if (kind == 0) K8SLLM_AC(float, 0); else if (kind == 1) K8SLLM_AC(float, 1); else if (kind == 3) K8SLLM_AC(float, 3); else return -1;
  } else {
    if (kind == 0) K8SLLM_AC(bf16_t, 0); else if (kind == 1) K8SLLM_AC(bf16_t, 1); else if (kind == 3) K8SLLM_AC(bf16_t, 3); else return -1;
  }
#undef K8SLLM_AC
  return (int)hipGetLastError();
}

int k8sllm_hy_sigmoid_gate(void* x, const void* z, long z_stride, long rows, int n, int vec, int f32, hipStream_t s) {
  const long tot = rows * (vec ? n / 8 : n);
  if (tot <= 0) return 0;
  const dim3 g((unsigned)((tot + 255) / 256));
  if (f32)
    hipLaunchKernelGGL(sigmoid_gate_kernel<float>, g, dim3(256), 0, s, (float*)x, (const float*)z, z_stride, rows, n, vec);
  else
    hipLaunchKernelGGL(sigmoid_gate_kernel<bf16_t>, g, dim3(256), 0, s, (bf16_t*)x, (const bf16_t*)z, z_stride, rows, n, vec);
  return (int)hipGetLastError();
}

int k8sllm_hy_softcap(float* x, long n, float cap, hipStream_t s) {
  if (n <= 0) return 0;
  if (!(cap > 0.f)) return -1;
  hipLaunchKernelGGL(softcap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, x, n, cap);
  return (int)hipGetLastError();
}

int k8sllm_hy_swiglu(void* out, const void* gu, long rows, int f, int f32, hipStream_t s) {
  const long n = rows * f;
  if (n <= 0) return 0;
  const unsigned g = (unsigned)((n + 255) / 256);
  if (f32)
    hipLaunchKernelGGL(swiglu_kernel<float>, dim3(g), dim3(256), 0, s, (float*)out, (const float*)gu, rows, f);
  else
    hipLaunchKernelGGL(swiglu_kernel<bf16_t>, dim3(g), dim3(256), 0, s, (bf16_t*)out, (const bf16_t*)gu, rows, f);
  return (int)hipGetLastError();
}
int k8sllm_hy_norm_shift(void* out, const float* x, const float* w, const float* mu, float* state, const int* cu,
                         const int* ctx, const int* slot, int S, long rows, int d, float eps, int one_plus,
                         int advance, int multi, int f32, hipStream_t s) {
  if (rows <= 0 || S <= 0) return 0;
  if (f32)
    hipLaunchKernelGGL(norm_shift_kernel<float>, dim3(rows), dim3(256), 0, s, (float*)out, x, w, mu, state, cu, ctx,
                       slot, S, d, eps, one_plus, advance);
  else
    hipLaunchKernelGGL(norm_shift_kernel<bf16_t>, dim3(rows), dim3(256), 0, s, (bf16_t*)out, x, w, mu, state, cu, ctx,
                       slot, S, d, eps, one_plus, advance);
  if (advance && multi)
    hipLaunchKernelGGL(shift_state_kernel<0>, dim3(S), dim3(256), 0, s, x, w, state, cu, slot, d, eps, one_plus);
  return (int)hipGetLastError();
}

// plane = T * d
int k8sllm_hy_depth_mix(float* stack, long plane, int n, const void* addend, int adt, const float* coef,
                        hipStream_t s) {
  if (plane <= 0) return 0;
  if (n < 0 || n >= kMaxDepth) return -1;
  if (plane & 3) {
    hipLaunchKernelGGL(depth_mix_scalar_kernel, dim3((unsigned)((plane + 255) / 256)), dim3(256), 0, s, stack, plane, n,
                       addend, adt, coef);
    return (int)hipGetLastError();
  }
  hipLaunchKernelGGL(depth_mix_kernel, dim3((unsigned)((plane / 4 + 255) / 256)), dim3(256), 0, s, stack, plane, n,
                     addend, adt, coef);
  return (int)hipGetLastError();
}

int k8sllm_hy_activation(void* out, const void* x, long n, int kind, float a, float b, int f32, hipStream_t s) {
  if (n <= 0) return 0;
  const dim3 g((unsigned)((n + 2047) / 2048));
#define K8SLLM_ACT(T, K) hipLaunchKernelGGL((activation_kernel<T, K>), g, dim3(256), 0, s, (T*)out, (const T*)x, n, a, b)
  if (f32) {
    if (kind == 0) K8SLLM_ACT(float, 0); else if (kind == 1) K8SLLM_ACT(float, 1); else if (kind == 2) K8SLLM_ACT(float, 2); else if (kind == 3) K8SLLM_ACT(float, 3); else return -1;
  } else {
    if (kind == 0) K8SLLM_ACT(bf16_t, 0); else if (kind == 1) K8SLLM_ACT(bf16_t, 1); else if (kind == 2) K8SLLM_ACT(bf16_t, 2); else if (kind == 3) K8SLLM_ACT(bf16_t, 3); else return -1;
  }
#undef K8SLLM_ACT
  return (int)hipGetLastError();
}

// t0, t1, ty: 0 absent, 1 bf16, 2 fp32.  w == nullptr: no norm, out = the new residual
int k8sllm_hy_sum_norm(void* out, float* residual, const void* a0, int t0, float s0, const void* a1, int t1, float s1,
                       const void* y, int ty, const float* wy, const float* w, long rows, int d, float eps, int center,
                       int one_plus, int f32, hipStream_t s) {
  if (rows <= 0) return 0;
  if (f32)
    hipLaunchKernelGGL(sum_norm_kernel<float>, dim3(rows), dim3(256), 0, s, (float*)out, residual, a0, t0, s0, a1, t1, s1,
                       y, ty, wy, w, d, eps, center, one_plus);
  else
    hipLaunchKernelGGL(sum_norm_kernel<bf16_t>, dim3(rows), dim3(256), 0, s, (bf16_t*)out, residual, a0, t0, s0, a1, t1,
                       s1, y, ty, wy, w, d, eps, center, one_plus);
  return (int)hipGetLastError();
}

int k8sllm_hy_gated_lookup(void* out, const void* gate, const void* table, long t_stride, int col, const int* ids,
                           const int* src, const int* prev, long rows, int n, int vocab, int f32, hipStream_t s) {
  const long tot = rows * n;
  if (tot <= 0) return 0;
  const dim3 g((unsigned)((tot + 255) / 256));
  if (f32)
    hipLaunchKernelGGL(gated_lookup_kernel<float>, g, dim3(256), 0, s, (float*)out, (const float*)gate,
                       (const float*)table, t_stride, col, ids, src, prev, rows, n, vocab);
  else
    hipLaunchKernelGGL(gated_lookup_kernel<bf16_t>, g, dim3(256), 0, s, (bf16_t*)out, (const bf16_t*)gate,
                       (const bf16_t*)table, t_stride, col, ids, src, prev, rows, n, vocab);
  return (int)hipGetLastError();
}
}
