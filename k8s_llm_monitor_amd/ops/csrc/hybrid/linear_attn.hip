// Linear attention with a fixed decay per head on the matrix cores (bf16 activations, prompts).
//
//   S_t = lam S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t        (per head; S is [dk][dv], fp32)
//
// over chunks of 64 tokens: with i, j the places of a query and a key inside a chunk of n tokens,
//
//   o_i   = lam^(i+1) (q_i S_prev)  +  sum_{j <= i} lam^(i-j) (q_i . k_j) v_j
//   S_new = lam^n S_prev            +  sum_j lam^(n-1-j) k_j v_j^T
//
// so only the state crosses chunks.  q.k has bf16 inputs and runs on v_mfma_f32_16x16x32_bf16 (exact
// products, fp32 sums); everything that holds scores or state - (scores) V, q S_prev, (scaled k)^T V -
// runs on the fp32 matrix instruction v_mfma_f32_16x16x4_f32, so scores, decays and state stay 32-bit.
//
// A workgroup (4 waves) owns (segment, head, 16 NT value columns): value columns are independent, which
// gives the sequential chunk loop its parallel axis.  Wave w
// takes the chunk's queries 16w .. 16w+15 for the outputs and every fourth of the 2 KS NT state tiles
// (16 x 16) for the update; the state lives in those waves' accumulators and is republished in LDS once
// per chunk for the q S_prev products.  The fp32 k-steps
// take the tokens (or key dims) {4 q + i : q = 0..3}, which is how the score accumulators and the query
// fragments already sit in the lanes - no shuffles between the products.
#include "hy_common.h"

namespace k8sllm {

constexpr int kLaChunk = 64;
constexpr int kLaPV = 36;  // LDS row pitches (floats): 4 * pitch = 16 mod 32 banks, rows 16-byte aligned

template <int KS, int NT>  // key dim / 32, value columns / 16 per workgroup
__global__ __launch_bounds__(256) void linear_attn_chunk_kernel(float* __restrict__ y, const bf16_t* __restrict__ vkq,
                                                                const float* __restrict__ decay,
                                                                float* __restrict__ state, const int* __restrict__ cu,
                                                                const int* __restrict__ ctx,
                                                                const int* __restrict__ slot, int H, int dv) {
  constexpr int DK = 32 * KS, PK = DK + 4, PS = 34, NV = 16 * NT;
  constexpr int NTILES = 2 * KS * NT, TPW = (NTILES + 3) / 4;  // state tiles: all, per wave
  __shared__ __attribute__((aligned(16))) float Ks[kLaChunk * PK];   // k_j * lam^(n-1-j), [token][key dim]
  __shared__ __attribute__((aligned(16))) float Vs[kLaChunk * kLaPV];  // [token][value column]
  __shared__ float Ss[DK * PS];                                       // state before the chunk, [key dim][value column]
  __shared__ float lam[kLaChunk + 1];
  const int s = blockIdx.x, h = blockIdx.y, dvb = blockIdx.z * NV;
  const int sl = slot[s], t0 = cu[s], t1 = cu[s + 1];
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c16 = lane & 15, quad = lane >> 4;
  const long inner = (long)H * dv, C = inner + 2L * H * DK;
  if (sl < 0) {  // padding rows: defined output, no state
    for (int i = tid; i < (t1 - t0) * NV; i += 256) y[(long)(t0 + i / NV) * inner + (long)h * dv + dvb + (i % NV)] = 0.f;
    return;
  }
  if (t1 <= t0) return;
  const float lm = decay[h];
  if (tid <= kLaChunk) lam[tid] = tid == 0 ? 1.f : powf(lm, (float)tid);
  const bf16_t* vcol = vkq + (long)h * dv + dvb;
  const bf16_t* kcol = vkq + inner + (long)h * DK;
  const bf16_t* qcol = kcol + (long)H * DK;
  // this wave's state tiles: tile id = w + 4 j -> key-dim tile id / NT, value-column tile id % NT;
  // accumulator entry r of lane (c16, quad) is S[16 rt + 4 quad + r][16 ct + c16]
  f32x4 S[TPW];
  float* sp = state + ((long)sl * H + h) * DK * dv + dvb;
  const bool carried = ctx[s] > 0;
#pragma unroll
  for (int j = 0; j < TPW; ++j) {
    const int id = min(w + 4 * j, NTILES - 1), rt = id / NT, ct = id % NT;  // a wave's spare tile repeats the last one
#pragma unroll
    for (int r = 0; r < 4; ++r) S[j][r] = carried ? sp[(long)(16 * rt + 4 * quad + r) * dv + 16 * ct + c16] : 0.f;
  }
  // The next chunk's operands are fetched into registers while this chunk's products run (the chain of
  // chunks is sequential: without it every chunk starts with two exposed trips to memory): the raw key
  // and value rows this thread stages, this wave's query fragments and the key fragments of its tiles.
  uint4 rk[KS], rv;
  bf16x8 qn[KS], kn[4][KS];
  auto fetch = [&](int tb, int n) {
#pragma unroll
    for (int u = 0; u < KS; ++u) {
      const int idx = tid + 256 * u, row = idx / (DK / 8), c8 = idx - row * (DK / 8);
      rk[u] = *reinterpret_cast<const uint4*>(kcol + (long)(tb + min(row, n - 1)) * C + 8 * c8);
    }
    if (tid < kLaChunk * 2 * NT)
      rv = *reinterpret_cast<const uint4*>(vcol + (long)(tb + min(tid / (2 * NT), n - 1)) * C + 8 * (tid % (2 * NT)));
    if (16 * w < n) {
      const bf16_t* qrow = qcol + (long)(tb + min(16 * w + c16, n - 1)) * C + 8 * quad;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) qn[ks] = *reinterpret_cast<const bf16x8*>(qrow + 32 * ks);
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
        if (kt <= w) {
          const bf16_t* krow = kcol + (long)(tb + min(16 * kt + c16, n - 1)) * C + 8 * quad;
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) kn[kt][ks] = *reinterpret_cast<const bf16x8*>(krow + 32 * ks);
        }
    }
  };
  fetch(t0, min(kLaChunk, t1 - t0));
  for (int tb = t0; tb < t1; tb += kLaChunk) {
    const int n = min(kLaChunk, t1 - tb);
    __syncthreads();  // the previous chunk's products are done with Ks, Vs, Ss (and lam is written)
    // stage the chunk: keys scaled for the state update (fp32), values (fp32); rows from n on are zero
#pragma unroll
    for (int u = 0; u < KS; ++u) {
      const int idx = tid + 256 * u, row = idx / (DK / 8), c8 = idx - row * (DK / 8);
      float f[8];
      unpack8(rk[u], f);
      const float g = lam[max(n - 1 - row, 0)];
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = row < n ? f[e] * g : 0.f;
      store8(&Ks[row * PK + 8 * c8], f);
    }
    if (tid < kLaChunk * 2 * NT) {
      const int row = tid / (2 * NT), c8 = tid % (2 * NT);
      float f[8];
      unpack8(rv, f);
      if (row >= n) {
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = 0.f;
      }
      store8(&Vs[row * kLaPV + 8 * c8], f);
    }
#pragma unroll
    for (int j = 0; j < TPW; ++j) {
      const int id = w + 4 * j, rt = id / NT, ct = id % NT;
      if (id < NTILES) {
#pragma unroll
        for (int r = 0; r < 4; ++r) Ss[(16 * rt + 4 * quad + r) * PS + 16 * ct + c16] = S[j][r];
      }
    }
    // scores of this wave's 16 queries against the key tiles up to its own (bf16 fragments)
    const bool live = 16 * w < n;  // wave-uniform
    bf16x8 qf[KS];
    float a[4][4];
    if (live) {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) qf[ks] = qn[ks];
      const int qpos = 16 * w + c16;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        if (kt <= w) {
          f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kn[kt][ks], qf[ks], acc, 0, 0, 0);
#pragma unroll
          for (int i = 0; i < 4; ++i) {  // acc[i]: key 16 kt + 4 quad + i, query c16
            const int key = 16 * kt + 4 * quad + i;
            a[kt][i] = (key <= qpos && key < n) ? acc[i] * lam[max(qpos - key, 0)] : 0.f;
          }
        }
      }
    }
    __syncthreads();  // Ks, Vs, Ss staged
    if (tb + kLaChunk < t1) fetch(tb + kLaChunk, min(kLaChunk, t1 - tb - kLaChunk));  // in flight during the products
    if (live) {
      f32x4 o[NT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) o[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
      // q S_prev: k-step (ks, e) takes key dims 32 ks + 8 q + e, the query fragment's own entries
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float qa = (float)qf[ks][e];
          const float* srow = &Ss[(32 * ks + 8 * quad + e) * PS + c16];
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) o[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(qa, srow[16 * nt], o[nt], 0, 0, 0);
        }
      // o[nt][r]: query 16 w + 4 quad + r, value column 16 nt + c16
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float g = lam[min(16 * w + 4 * quad + r + 1, kLaChunk)];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) o[nt][r] *= g;
      }
      // (scores) V: k-step (kt, i) takes keys 16 kt + 4 q + i, the score accumulators' own entries
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        if (kt <= w) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float* vrow = &Vs[(16 * kt + 4 * quad + i) * kLaPV + c16];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) o[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[kt][i], vrow[16 * nt], o[nt], 0, 0, 0);
          }
        }
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = 16 * w + 4 * quad + r;
        if (row < n) {
          float* yr = y + (long)(tb + row) * inner + (long)h * dv + dvb + c16;
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) yr[16 * nt] = o[nt][r];
        }
      }
    }
    // the state update: S = lam^n S + (scaled k)^T V, token k-steps {16 kt + 4 q + i}
    const float gn = lam[n];
#pragma unroll
    for (int j = 0; j < TPW; ++j) {
      const int id = min(w + 4 * j, NTILES - 1), rt = id / NT, ct = id % NT;
#pragma unroll
      for (int r = 0; r < 4; ++r) S[j][r] *= gn;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        if (16 * kt < n) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int tok = 16 * kt + 4 * quad + i;
            S[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(Ks[tok * PK + 16 * rt + c16], Vs[tok * kLaPV + 16 * ct + c16], S[j], 0, 0, 0);
          }
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < TPW; ++j) {
    const int id = w + 4 * j, rt = id / NT, ct = id % NT;
    if (id < NTILES) {
#pragma unroll
      for (int r = 0; r < 4; ++r) sp[(long)(16 * rt + 4 * quad + r) * dv + 16 * ct + c16] = S[j][r];
    }
  }
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" {

// vkq [T][H*dv | H*dk | H*dk] bf16 (v, k, q head by head), state [slots][H][dk][dv] fp32, y [T][H*dv] fp32.
// Returns 1 (nothing launched) for sizes that are not this kernel's: dk a multiple of 32 up to 128, dv
// a multiple of 16.  nt: value-column tiles per workgroup, 1 or 2 (0: 1 - measured faster at every grid
// size: 225 against 256 us per 8192 tokens of 16 heads of 128 x 128, small grids and large).
int k8sllm_hy_linear_attn_chunk(float* y, const void* vkq, const float* decay, float* state, const int* cu,
                                const int* ctx, const int* slot, int S, int H, int dk, int dv, int nt, hipStream_t s) {
  if (S <= 0) return 0;
  if (dk % 32 || dk < 32 || dk > 128 || dv % 16 || dv < 16 || H < 1) return 1;
  if (nt != 0 && nt != 1 && nt != 2) return -1;
  if (nt == 2 && dv % 32) return 1;
  if (nt == 0) nt = 1;
  const dim3 grid((unsigned)S, (unsigned)H, (unsigned)(dv / (16 * nt)));
#define K8SLLM_LAC(KS)                                                                                               \
  if (nt == 2)                                                                                                       \
    hipLaunchKernelGGL((linear_attn_chunk_kernel<KS, 2>), grid, dim3(256), 0, s, y, (const bf16_t*)vkq, decay, state, \
                       cu, ctx, slot, H, dv);                                                                        \
  else                                                                                                               \
    hipLaunchKernelGGL((linear_attn_chunk_kernel<KS, 1>), grid, dim3(256), 0, s, y, (const bf16_t*)vkq, decay, state, \
                       cu, ctx, slot, H, dv)
  switch (dk / 32) {
    case 1: K8SLLM_LAC(1); break;
    case 2: K8SLLM_LAC(2); break;
    case 3: K8SLLM_LAC(3); break;
    default: K8SLLM_LAC(4); break;
  }
#undef K8SLLM_LAC
  return (int)hipGetLastError();
}
}
