// Latent (low-rank compressed) attention: what surrounds the attention kernels of window_attn.hip.
//   latent_prep     in place on the fused down-projections [T][q_rank | kv_rank | rot]: RMSNorm of the
//                   query latent; RMSNorm of the key/value latent and rotation of the shared key part,
//                   both written to the pages: key page row = [latent | rotated part | zeros up to the
//                   row pitch], value page = the latent once more, dim-major ([blocks][1][kv_rank][BS])
//   latent_queries  per head [q_lat (unrotated query times the key expansion) | rotated query part |
//                   zeros up to the same pitch]
//   latent_attention  the matrix-core attention over those pages (bf16), prompt chunks and decoding
// Rotation: entries i and i + nf of the first 2 * nf entries (nf frequencies, freq[i] given in fp32)
// turn by the angle position * freq[i] - or, pairs == 1, entries 2i and 2i + 1; angles, sine and cosine
// are fp32.
#include "hy_common.h"

namespace k8sllm {

template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(T* __restrict__ proj, long stride, int Q, int R, int dr,
                                                          const float* __restrict__ qw, const float* __restrict__ kw,
                                                          float eps, const int* __restrict__ positions,
                                                          const float* __restrict__ freq, int nf, int pairs,
                                                          T* __restrict__ k_cache, int kw_pitch,
                                                          T* __restrict__ v_cache,
                                                          const int* __restrict__ slots, int bs) {
  __shared__ float red[4];
  const long t = blockIdx.x;
  T* row = proj + t * stride;
  float sq = 0.f, sc = 0.f;
  for (int c = threadIdx.x; c < Q; c += 256) {
    const float v = ldf(row + c);
    sq += v * v;
  }
  sq = block_sum<256>(sq, red);
  const float iq = 1.0f / sqrtf(sq / (float)Q + eps);
  for (int c = threadIdx.x; c < Q; c += 256) stf(row + c, ldf(row + c) * iq * qw[c]);
  if (kw == nullptr) return;  // a layer that reads another layer's pages
  for (int c = threadIdx.x; c < R; c += 256) {
    const float v = ldf(row + Q + c);
    sc += v * v;
  }
  sc = block_sum<256>(sc, red);
  const float ic = 1.0f / sqrtf(sc / (float)R + eps);
  const long slot = (slots != nullptr && k_cache != nullptr) ? slots[t] : -1;
  T* kp = slot >= 0 ? k_cache + slot * (long)kw_pitch : nullptr;  // the pitch's tail stays zero
  for (int c = threadIdx.x; c < R; c += 256) {
    T* e = row + Q + c;
    stf(e, ldf(e) * ic * kw[c]);
    if (kp != nullptr) {
      kp[c] = *e;
      v_cache[((slot / bs) * R + c) * bs + slot % bs] = *e;
    }
  }
  T* kr = row + Q + R;
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < dr; i += 256) {
    if (i < nf) {  // this thread owns the pair (i, i + nf), or (2i, 2i + 1)
      const int a = pairs ? 2 * i : i, b = pairs ? 2 * i + 1 : i + nf;
      float sn, cs;
      sincosf(pos * freq[i], &sn, &cs);
      const float u = ldf(kr + a), v = ldf(kr + b);
      stf(kr + a, u * cs - v * sn);
      stf(kr + b, v * cs + u * sn);
      if (kp != nullptr) {
        kp[R + a] = kr[a];
        kp[R + b] = kr[b];
      }
    } else if (i >= 2 * nf && kp != nullptr) {
      kp[R + i] = kr[i];
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void latent_queries_kernel(T* __restrict__ out, const T* __restrict__ q, long q_stride,
                                                             const T* __restrict__ q_lat, long T_rows, int H, int dn,
                                                             int dr, int R, int w, const int* __restrict__ positions,
                                                             const float* __restrict__ freq, int nf, int pairs) {
  const long t = blockIdx.x;
  const float pos = (float)positions[t];
  T* o = out + t * (long)H * w;
  for (int c = threadIdx.x; c < H * w; c += 256) {  // w >= R + dr: the row's pitch, zeros behind the query
    const int h = c / w, j = c - h * w;
    if (j >= R + dr) {
      stf(o + c, 0.f);
      continue;
    }
    if (j < R) {
      o[c] = q_lat[((long)h * T_rows + t) * R + j];
      continue;
    }
    const int i = j - R;
    const T* qr = q + t * q_stride + (long)h * (dn + dr) + dn;
    if (i >= 2 * nf) {
      o[c] = qr[i];
      continue;
    }
    const int f = pairs ? i >> 1 : (i < nf ? i : i - nf);
    const bool lead = pairs ? !(i & 1) : i < nf;  // the pair's first entry
    float sn, cs;
    sincosf(pos * freq[f], &sn, &cs);
    const float u = ldf(qr + (pairs ? 2 * f : f)), v = ldf(qr + (pairs ? 2 * f + 1 : f + nf));
    stf(o + c, lead ? u * cs - v * sn : v * cs + u * sn);
  }
}


// bf16 latent attention on the matrix cores, prompt chunks and decoding alike.  All heads read the
// same key/value stream, so the 16 query columns of a tile are 16 HEADS of ONE token (the window
// mask is then the same for the whole tile), and a workgroup is (token, group of 16 heads):
//   S^T[key][head] = K Q^T     v_mfma_f32_16x16x32_bf16: A = key rows, 16-byte loads from the page
//                              ([latent | rotated part], padded with zeros to a multiple of 32),
//                              B = the token's query rows, in registers for the whole loop
//   O^T[d][head]  += V^T P^T   v_mfma_f32_16x16x16_bf16: B = the score accumulator itself, A = V^T,
//                              8-byte loads from the dim-major latent page
// The NW waves of a workgroup take the window's 16-key tiles in turn (decoding: the window is the
// only parallel axis of a row) and merge their (maximum, denominator, output) through LDS: the common
// maximum first, then the outputs summed wave after wave into one buffer.  Only wave 0 starts from
// the sink.  Scores, weights and sums are fp32, base-2 exponentials (the scale carries log2 e).
// QT consecutive tokens of a prompt chunk share a wave's key and value fragments (their windows
// differ by one key at each end).
// KS_MAX / DT_MAX bound the key width / 32 and the value width / 16 (register arrays); the real
// widths are run-time (wave-uniform guards).  cu == nullptr: one row per sequence at seq_lens - 1.
// how far (base-2 logits) a tile's maximum must exceed the running one before that is moved
constexpr float kLazy = 8.f;

// The page ids of a row's window, one per lane (64 tiles at a time): the id of a tile is then a
// v_readlane away instead of a dependent memory access in front of every tile's loads.
struct PageIds {
  const int* bt;
  int first, last, reg;
  __device__ __forceinline__ void init(const int* table, int first_tile, int last_tile) {
    bt = table;
    first = first_tile;
    last = last_tile;
    reg = bt[min(first + (int)(threadIdx.x & 63), last)];
  }
  __device__ __forceinline__ long at(int j0) {  // j0: wave-uniform key position of a tile
    int idx = __builtin_amdgcn_readfirstlane(j0 >> 4) - first;
    if (idx >= 64) {  // windows of more than 1024 keys: the next 64 ids
      first += idx & ~63;
      reg = bt[min(first + (int)(threadIdx.x & 63), last)];
      idx &= 63;
    }
    return (long)__builtin_amdgcn_readlane(reg, idx);
  }
};

template <int KS_MAX, int DT_MAX, int NW, int QT>
__global__ __launch_bounds__(64 * NW) void latent_attn_mfma_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q, long q_stride, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ cu, const int* __restrict__ ctx,
    const int* __restrict__ seq_lens, const int* __restrict__ block_tables, int bt_stride, int S, int H, int dkp,
    int dv, float scale, int window, const float* __restrict__ sinks) {
  static_assert(NW == 1 || QT == 1, "the window is split over waves only for single tokens");
  constexpr int OP = DT_MAX * 16 + 4;  // LDS row pitch of the merge buffer (floats)
  __shared__ __attribute__((aligned(16))) float o_s[NW > 1 ? 16 * OP : 4];
  __shared__ float m_s[NW > 1 ? NW : 1][16];
  __shared__ float l_s[NW > 1 ? NW : 1][16];
  const float sc2 = scale * 1.44269504088896341f;
  // Workgroups go to the 8 XCDs in turn (each with an L2 of its own): give every XCD one contiguous
  // eighth of the (token group, head group) list, so that the windows its waves read overlap in ITS L2
  const int nwg = gridDim.x * gridDim.y, lin = blockIdx.y * gridDim.x + blockIdx.x;
  const int xcd = lin & 7, glin = xcd * (nwg >> 3) + min(xcd, nwg & 7) + (lin >> 3);  // XCD x: workgroups x, x + 8, ..
  const int hg = glin % (int)gridDim.y, bx = glin / (int)gridDim.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c16 = lane & 15, quad = lane >> 4;
  // this workgroup's tokens: QT consecutive rows of one segment (token groups are numbered segment
  // by segment), or one sequence's newest token
  int s = 0, row0, p0, nt = 1;
  if (cu != nullptr) {
    if (QT == 1) {
      row0 = bx;
      s = find_segment(cu, S, row0);
      p0 = ctx[s] + row0 - cu[s];
    } else {
      int g = bx, n = 0;
      for (; s < S; ++s) {
        n = cu[s + 1] - cu[s];
        const int ng = (n + QT - 1) / QT;
        if (g < ng) break;
        g -= ng;
      }
      if (s >= S) return;
      row0 = cu[s] + g * QT;
      nt = min(QT, n - g * QT);
      p0 = ctx[s] + g * QT;
    }
  } else {
    s = row0 = bx;
    p0 = seq_lens[row0] - 1;
  }
  const int nh = min(16, H - hg * 16);
  bf16_t* obase = out + ((long)row0 * H + hg * 16) * dv;
  if (p0 < 0) {  // padding row of a decode bucket
    for (int c = threadIdx.x; c < nh * dv; c += 64 * NW) obase[c] = 0;
    return;
  }
  const int nks = dkp >> 5, ndt = dv >> 4;
  const int head = hg * 16 + min(c16, nh - 1);
  const int* bt = block_tables + (long)s * bt_stride;
  // token t of the group sits at position p0 + t and sees keys lo_t .. p0 + t
  const int lo = window > 0 ? max(0, p0 - window + 1) : 0, hi = p0 + nt;
  bf16x8 qf[QT][KS_MAX];
  f32x4 oacc[QT][DT_MAX];
  float m[QT], l[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const bf16_t* qrow = q + (long)(row0 + min(t, nt - 1)) * q_stride + (long)head * dkp + 8 * quad;
#pragma unroll
    for (int ks = 0; ks < KS_MAX; ++ks)
      if (ks < nks) qf[t][ks] = *reinterpret_cast<const bf16x8*>(qrow + 32 * ks);
#pragma unroll
    for (int dt = 0; dt < DT_MAX; ++dt) oacc[t][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m[t] = -INFINITY;
    l[t] = 0.f;
    if (wave == 0) {
      m[t] = sinks != nullptr ? sinks[head] * 1.44269504088896341f : 0.f;
      l[t] = 1.f;
    }
  }
  const bf16_t* kbase = k_cache + 8 * quad;
  const bf16_t* vbase = v_cache + (long)c16 * 16 + 4 * quad;
  const long vpage = (long)dv * 16;
  const int jfirst = (lo & ~15) + 16 * wave;
  PageIds pages;
  pages.init(bt, lo >> 4, (hi - 1) >> 4);
  bf16x8 kf_n[KS_MAX];
  s16x4 vf_n[DT_MAX];
  auto issue = [&](int j0) {
    const long pg = pages.at(j0);
    const bf16_t* krow = kbase + ((pg << 4) + (min(j0 + c16, hi - 1) & 15)) * dkp;
#pragma unroll
    for (int ks = 0; ks < KS_MAX; ++ks)
      if (ks < nks) kf_n[ks] = *reinterpret_cast<const bf16x8*>(krow + 32 * ks);
    const bf16_t* vpg = vbase + pg * vpage;
#pragma unroll
    for (int dt = 0; dt < DT_MAX; ++dt)
      if (dt < ndt) vf_n[dt] = *reinterpret_cast<const s16x4*>(vpg + dt * 256);
  };
  // no register double buffer: with fewer registers two waves fit a SIMD and hide each other's loads
  // better than one wave hides its own (measured both ways)
  for (int j0 = jfirst; j0 < hi; j0 += 16 * NW) {
    bf16x8 kf[KS_MAX];
    s16x4 vf[DT_MAX];
    issue(j0);
#pragma unroll
    for (int ks = 0; ks < KS_MAX; ++ks) kf[ks] = kf_n[ks];
#pragma unroll
    for (int dt = 0; dt < DT_MAX; ++dt) vf[dt] = vf_n[dt];
    s16x4 pb[QT];
    float alpha[QT];
    bool rescale[QT];
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      f32x4 sacc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS_MAX; ++ks)
        if (ks < nks) sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[ks], qf[t][ks], sacc, 0, 0, 0);
      const int pt = p0 + t, lot = window > 0 ? max(0, pt - window + 1) : 0;
      float sv[4], tmax = -INFINITY;
      if (t < nt && j0 >= lot && j0 + 15 <= pt) {  // wave-uniform: every key of the tile is live
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          sv[i] = sacc[i] * sc2;
          tmax = fmaxf(tmax, sv[i]);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {  // sacc[i]: key j0 + 4 quad + i, head c16
          const int j = j0 + 4 * quad + i;
          sv[i] = (t < nt && j >= lot && j <= pt) ? sacc[i] * sc2 : -INFINITY;
          tmax = fmaxf(tmax, sv[i]);
        }
      }
      tmax = xor32_max_f(xor16_max(tmax));
      // the running maximum only moves when it is beaten by more than kLazy (weights then stay below
      // 2^kLazy, harmless in fp32 sums): the rescale of the whole output accumulator becomes rare.
      // A wave's first tile always holds a live key (QT == 1) or m starts finite (the sink), so mn is finite
      const float mn = tmax > m[t] + kLazy ? tmax : m[t];
      alpha[t] = __builtin_amdgcn_exp2f(m[t] - mn);
      float ps = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pv = __builtin_amdgcn_exp2f(sv[i] - mn);
        ps += pv;
        pb[t][i] = (short)f2bf(pv);
      }
      ps = xor32_sum_f(xor16_sum(ps));
      l[t] = l[t] * alpha[t] + ps;
      m[t] = mn;
      rescale[t] = __any(alpha[t] != 1.f);
    }
    // the rescale of a token's whole accumulator is ONE block behind one wave-uniform branch (a branch
    // around each tile's four multiplies is flattened by the compiler into multiplies on every tile)
#pragma unroll
    for (int t = 0; t < QT; ++t)
      if (rescale[t]) {
#pragma unroll
        for (int dt = 0; dt < DT_MAX; ++dt)
#pragma unroll
          for (int i = 0; i < 4; ++i) oacc[t][dt][i] *= alpha[t];
      }
#pragma unroll
    for (int dt = 0; dt < DT_MAX; ++dt)
      if (dt < ndt) {
#pragma unroll
        for (int t = 0; t < QT; ++t)
          oacc[t][dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf[dt], pb[t], oacc[t][dt], 0, 0, 0);
      }
  }
  // oacc[t][dt][i] = O[token t][head c16][d = 16 dt + 4 quad + i]
  if (NW == 1) {
    if (c16 >= nh) return;
#pragma unroll
    for (int t = 0; t < QT; ++t) {
      if (t >= nt) break;
      const float inv = l[t] > 0.f ? 1.f / l[t] : 0.f;
      bf16_t* orow = obase + ((long)t * H + c16) * dv;
#pragma unroll
      for (int dt = 0; dt < DT_MAX; ++dt)
        if (dt < ndt) {
          uint2 w;
          w.x = pack2(oacc[t][dt][0] * inv, oacc[t][dt][1] * inv);
          w.y = pack2(oacc[t][dt][2] * inv, oacc[t][dt][3] * inv);
          *reinterpret_cast<uint2*>(orow + 16 * dt + 4 * quad) = w;
        }
    }
    return;
  }
  if (quad == 0) m_s[wave][c16] = m[0];
  __syncthreads();
  float M = -INFINITY;
#pragma unroll
  for (int w = 0; w < NW; ++w) M = fmaxf(M, m_s[w][c16]);  // wave 0's is finite (the sink)
  const float f = m[0] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m[0] - M);
  if (quad == 0) l_s[wave][c16] = l[0] * f;
  for (int w = 0; w < NW; ++w) {
    if (wave == w) {
#pragma unroll
      for (int dt = 0; dt < DT_MAX; ++dt)
        if (dt < ndt) {
          float4* dst = reinterpret_cast<float4*>(&o_s[c16 * OP + 16 * dt + 4 * quad]);
          float4 v = make_float4(oacc[0][dt][0] * f, oacc[0][dt][1] * f, oacc[0][dt][2] * f, oacc[0][dt][3] * f);
          if (w > 0) {
            const float4 o = *dst;
            v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
          }
          *dst = v;
        }
    }
    __syncthreads();
  }
  for (int c = threadIdx.x; c < nh * dv; c += 64 * NW) {
    const int hh = c / dv, dd = c - hh * dv;
    float L = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) L += l_s[w][hh];
    obase[c] = f2bf(L > 0.f ? o_s[hh * OP + dd] / L : 0.f);
  }
}

// Prompt chunks of large steps: the same tiles with the 16-key page staged ONCE per workgroup in LDS.
// A workgroup is 4 waves x QT consecutive tokens of one segment (x 16 heads); a key tile is one page,
// i.e. one contiguous block of the key pages and one of the value pages, so staging is two straight
// copies with 16-byte loads (the next three pages' loads are in flight while this one is computed,
// two LDS buffers, one barrier per tile).  LDS rows are padded (keys: + 8 elements, values: 16 tokens + 4) so
// that the fragment reads of a quarter wave fall on different banks.  Every wave starts from the sink.
template <int KS_MAX, int DT_MAX, int QT>
__global__ __launch_bounds__(256) void latent_attn_lds_kernel(
    bf16_t* __restrict__ out, const bf16_t* __restrict__ q, long q_stride, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int* __restrict__ cu, const int* __restrict__ ctx,
    const int* __restrict__ block_tables, int bt_stride, int S, int H, int dkp, int dv, float scale, int window,
    const float* __restrict__ sinks) {
  constexpr int TW = 4 * QT;           // tokens per workgroup
  constexpr int KP = KS_MAX * 32 + 8;  // LDS pitch of a key row (elements)
  constexpr int VP = 20;               // LDS pitch of a value dim's 16 tokens
  constexpr int KC = (KS_MAX * 32 * 2 + 255) / 256, VC = (DT_MAX * 16 * 2 + 255) / 256;  // 16-byte pieces per thread
  __shared__ __attribute__((aligned(16))) bf16_t k_s[2][16 * KP];
  __shared__ __attribute__((aligned(16))) bf16_t v_s[2][DT_MAX * 16 * VP];
  const float sc2 = scale * 1.44269504088896341f;
  const int nwg = gridDim.x * gridDim.y, lin = blockIdx.y * gridDim.x + blockIdx.x;
  const int xcd = lin & 7, glin = xcd * (nwg >> 3) + min(xcd, nwg & 7) + (lin >> 3);  // see latent_attn_mfma_kernel
  const int hg = glin % (int)gridDim.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c16 = lane & 15, quad = lane >> 4;
  int s = 0, g = glin / (int)gridDim.y, n = 0;
  for (; s < S; ++s) {  // token groups are numbered segment by segment
    n = cu[s + 1] - cu[s];
    const int ng = (n + TW - 1) / TW;
    if (g < ng) break;
    g -= ng;
  }
  if (s >= S) return;
  const int nt = min(TW, n - g * TW);             // live tokens of the group
  const int row0 = cu[s] + g * TW, p0 = ctx[s] + g * TW;
  const int nh = min(16, H - hg * 16);
  const int nks = dkp >> 5, ndt = dv >> 4;
  const int head = hg * 16 + min(c16, nh - 1);
  const int* bt = block_tables + (long)s * bt_stride;
  const int lo = window > 0 ? max(0, p0 - window + 1) : 0, hi = p0 + nt;
  const int tok0 = wave * QT;                     // this wave's first token in the group
  const bool wave_live = tok0 < nt;
  bf16x8 qf[QT][KS_MAX];
  f32x4 oacc[QT][DT_MAX];
  float m[QT], l[QT];
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    const bf16_t* qrow = q + (long)(row0 + min(tok0 + t, nt - 1)) * q_stride + (long)head * dkp + 8 * quad;
#pragma unroll
    for (int ks = 0; ks < KS_MAX; ++ks)
      if (ks < nks) qf[t][ks] = *reinterpret_cast<const bf16x8*>(qrow + 32 * ks);
#pragma unroll
    for (int dt = 0; dt < DT_MAX; ++dt) oacc[t][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m[t] = sinks != nullptr ? sinks[head] * 1.44269504088896341f : 0.f;
    l[t] = 1.f;
  }
  // staging: piece c of the page's keys is 8 elements of row c / (dkp / 8); piece c of its values is
  // tokens 8 (c & 1) .. of dim c / 2.  The LDS offsets of a thread's pieces never change.
  const int nkc = 2 * dkp, nvc = 2 * dv, kpr = dkp >> 3;
  int k_off[KC], v_off[VC];
#pragma unroll
  for (int i = 0; i < KC; ++i) {
    const int c = tid + 256 * i;
    k_off[i] = c < nkc ? (c / kpr) * KP + (c % kpr) * 8 : -1;
  }
#pragma unroll
  for (int i = 0; i < VC; ++i) {
    const int c = tid + 256 * i;
    v_off[i] = c < nvc ? (c >> 1) * VP + (c & 1) * 8 : -1;
  }
  PageIds pages;
  pages.init(bt, lo >> 4, (hi - 1) >> 4);
  // three register sets keep the pages of the next three tiles in flight (one tile of compute does not
  // cover a load's latency); a set is written to the idle LDS buffer one tile before its use and
  // refilled at once
  uint4 kr0[KC], vr0[VC], kr1[KC], vr1[VC], kr2[KC], vr2[VC];
  auto stage_load = [&](uint4 (&kreg)[KC], uint4 (&vreg)[VC], int j0) {
    if (j0 >= hi) return;
    const long pg = pages.at(j0);
    const uint4* ksrc = reinterpret_cast<const uint4*>(k_cache + pg * 16 * dkp);
    const uint4* vsrc = reinterpret_cast<const uint4*>(v_cache + pg * 16 * dv);
#pragma unroll
    for (int i = 0; i < KC; ++i)
      if (k_off[i] >= 0) kreg[i] = ksrc[tid + 256 * i];
#pragma unroll
    for (int i = 0; i < VC; ++i)
      if (v_off[i] >= 0) vreg[i] = vsrc[tid + 256 * i];
  };
  auto stage_store = [&](int b, const uint4 (&kreg)[KC], const uint4 (&vreg)[VC]) {
#pragma unroll
    for (int i = 0; i < KC; ++i)
      if (k_off[i] >= 0) *reinterpret_cast<uint4*>(&k_s[b][k_off[i]]) = kreg[i];
#pragma unroll
    for (int i = 0; i < VC; ++i)
      if (v_off[i] >= 0) {  // 8-byte aligned rows: two halves
        *reinterpret_cast<uint2*>(&v_s[b][v_off[i]]) = make_uint2(vreg[i].x, vreg[i].y);
        *reinterpret_cast<uint2*>(&v_s[b][v_off[i] + 4]) = make_uint2(vreg[i].z, vreg[i].w);
      }
  };
  const int jfirst = lo & ~15;
  stage_load(kr0, vr0, jfirst);
  stage_load(kr1, vr1, jfirst + 16);
  stage_load(kr2, vr2, jfirst + 32);
  stage_store(0, kr0, vr0);
  stage_load(kr0, vr0, jfirst + 48);
  __syncthreads();
  int buf = 0;
  // one tile: compute from LDS buffer ``buf``, then hand the next tile (held in nk / nv) to the other buffer
  auto tile = [&](int j0, uint4 (&nk)[KC], uint4 (&nv)[VC]) {
    if (wave_live) {
      const bf16_t* ks_ = &k_s[buf][c16 * KP + 8 * quad];
      const bf16_t* vs_ = &v_s[buf][c16 * VP + 4 * quad];
      f32x4 sacc[QT];
#pragma unroll
      for (int t = 0; t < QT; ++t) sacc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS_MAX; ++ks)
        if (ks < nks) {
          const bf16x8 kf = *reinterpret_cast<const bf16x8*>(ks_ + 32 * ks);
#pragma unroll
          for (int t = 0; t < QT; ++t) sacc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[t][ks], sacc[t], 0, 0, 0);
        }
      s16x4 pb[QT];
      float alpha[QT];
      bool rescale[QT];
#pragma unroll
      for (int t = 0; t < QT; ++t) {
        const int pt = p0 + tok0 + t, lot = window > 0 ? max(0, pt - window + 1) : 0;
        const bool tl = tok0 + t < nt;
        float sv[4], tmax = -INFINITY;
        if (tl && j0 >= lot && j0 + 15 <= pt) {  // wave-uniform: every key of the tile is live
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            sv[i] = sacc[t][i] * sc2;
            tmax = fmaxf(tmax, sv[i]);
          }
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) {  // sacc[t][i]: key j0 + 4 quad + i, head c16
            const int j = j0 + 4 * quad + i;
            sv[i] = (tl && j >= lot && j <= pt) ? sacc[t][i] * sc2 : -INFINITY;
            tmax = fmaxf(tmax, sv[i]);
          }
        }
        tmax = xor32_max_f(xor16_max(tmax));
        const float mn = tmax > m[t] + kLazy ? tmax : m[t];  // m is finite from the start (the sink)
        alpha[t] = __builtin_amdgcn_exp2f(m[t] - mn);
        float ps = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float pv = __builtin_amdgcn_exp2f(sv[i] - mn);
          ps += pv;
          pb[t][i] = (short)f2bf(pv);
        }
        ps = xor32_sum_f(xor16_sum(ps));
        l[t] = l[t] * alpha[t] + ps;
        m[t] = mn;
        rescale[t] = __any(alpha[t] != 1.f);
      }
#pragma unroll
      for (int t = 0; t < QT; ++t)
        if (rescale[t]) {  // one block for the whole accumulator (see latent_attn_mfma_kernel)
#pragma unroll
          for (int dt = 0; dt < DT_MAX; ++dt)
#pragma unroll
            for (int i = 0; i < 4; ++i) oacc[t][dt][i] *= alpha[t];
        }
#pragma unroll
      for (int dt = 0; dt < DT_MAX; ++dt)
        if (dt < ndt) {
          const s16x4 vf = *reinterpret_cast<const s16x4*>(vs_ + dt * 16 * VP);
#pragma unroll
          for (int t = 0; t < QT; ++t)
            oacc[t][dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf, pb[t], oacc[t][dt], 0, 0, 0);
        }
    }
    if (j0 + 16 < hi) {
      stage_store(buf ^ 1, nk, nv);
      stage_load(nk, nv, j0 + 64);
    }
    __syncthreads();
    buf ^= 1;
  };
  for (int j0 = jfirst;;) {
    tile(j0, kr1, vr1);
    if ((j0 += 16) >= hi) break;
    tile(j0, kr2, vr2);
    if ((j0 += 16) >= hi) break;
    tile(j0, kr0, vr0);
    if ((j0 += 16) >= hi) break;
  }
  if (!wave_live || c16 >= nh) return;
#pragma unroll
  for (int t = 0; t < QT; ++t) {
    if (tok0 + t >= nt) break;
    const float inv = l[t] > 0.f ? 1.f / l[t] : 0.f;
    bf16_t* orow = out + ((long)(row0 + tok0 + t) * H + hg * 16 + c16) * dv;
#pragma unroll
    for (int dt = 0; dt < DT_MAX; ++dt)
      if (dt < ndt) {
        uint2 w;
        w.x = pack2(oacc[t][dt][0] * inv, oacc[t][dt][1] * inv);
        w.y = pack2(oacc[t][dt][2] * inv, oacc[t][dt][3] * inv);
        *reinterpret_cast<uint2*>(orow + 16 * dt + 4 * quad) = w;
      }
  }
}

}  // namespace k8sllm

using namespace k8sllm;

extern "C" {

int k8sllm_hy_latent_prep(void* proj, long stride, long T, int Q, int R, int dr, const float* qw, const float* kw,
                          float eps, const int* positions, const float* freq, int nf, int pairs, void* k_cache,
                          int kw_pitch, void* v_cache, const int* slots, int bs, int f32, hipStream_t s) {
  if (T <= 0) return 0;
  if (2 * nf > dr || (k_cache != nullptr && kw_pitch < R + dr)) return -1;
  if (f32)
    hipLaunchKernelGGL(latent_prep_kernel<float>, dim3(T), dim3(256), 0, s, (float*)proj, stride, Q, R, dr, qw, kw, eps,
                       positions, freq, nf, pairs, (float*)k_cache, kw_pitch, (float*)v_cache, slots, bs);
  else
    hipLaunchKernelGGL(latent_prep_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (bf16_t*)proj, stride, Q, R, dr, qw, kw,
                       eps, positions, freq, nf, pairs, (bf16_t*)k_cache, kw_pitch, (bf16_t*)v_cache, slots, bs);
  return (int)hipGetLastError();
}

int k8sllm_hy_latent_queries(void* out, const void* q, long q_stride, const void* q_lat, long T, int H, int dn, int dr,
                             int R, int w, const int* positions, const float* freq, int nf, int pairs, int f32,
                             hipStream_t s) {
  if (T <= 0) return 0;
  if (2 * nf > dr || w < R + dr) return -1;
  if (f32)
    hipLaunchKernelGGL(latent_queries_kernel<float>, dim3(T), dim3(256), 0, s, (float*)out, (const float*)q, q_stride,
                       (const float*)q_lat, T, H, dn, dr, R, w, positions, freq, nf, pairs);
  else
    hipLaunchKernelGGL(latent_queries_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (bf16_t*)out, (const bf16_t*)q,
                       q_stride, (const bf16_t*)q_lat, T, H, dn, dr, R, w, positions, freq, nf, pairs);
  return (int)hipGetLastError();
}
// Matrix-core latent attention (bf16): rows = T tokens, each at the position its segment (cu / ctx,
// prompt chunks) or its sequence length (cu == nullptr, decoding) gives.  Returns 1 when the sizes
// are not the kernel's (the caller then takes the any-size kernels): key rows padded to a multiple
// of 32 (dkp), value width a multiple of 16, 16-token pages.
int k8sllm_hy_latent_attention(void* out, const void* q, long q_stride, const void* k_cache, const void* v_cache,
                               const int* cu, const int* ctx, const int* seq_lens, const int* block_tables,
                               int bt_stride, int S, long T, int H, int dkp, int dv, int bs, float scale, int window,
                               const float* sinks, int split, hipStream_t s) {
  if (T <= 0) return 0;
  if (bs != 16 || dkp % 32 || dv % 16 || dkp > 320 || dv > 256 || q_stride % 8) return 1;
  const unsigned hgs = (unsigned)((H + 15) / 16);
  // The launcher's choice (split 0): prompt chunks of a large step take the LDS-staged kernel with one
  // token per wave; small steps and decoding eight waves per token (a row's window is its only
  // parallel axis).  Forced (tests, measurements): 1 / 2 tokens per wave with fragments from global
  // memory, 4 / 8 waves per token, 32 / 33 the LDS-staged kernel with two / one token per wave.
  if (cu != nullptr && (split == 32 || split == 33 || (split == 0 && T * hgs >= 2048))) {
    const int qt = split == 32 ? 2 : 1;  // one token per wave measured faster (more waves per SIMD)
    const dim3 grid((unsigned)(T / (4 * qt) + S), hgs);
#define K8SLLM_LL(KS, DT, QT)                                                                                          \
  hipLaunchKernelGGL((latent_attn_lds_kernel<KS, DT, QT>), grid, dim3(256), 0, s, (bf16_t*)out, (const bf16_t*)q,        \
                     q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, cu, ctx, block_tables, bt_stride, S, H,  \
                     dkp, dv, scale, window, sinks)
    if (dkp <= 128 && dv <= 128) {
      if (qt == 1) K8SLLM_LL(4, 8, 1); else K8SLLM_LL(4, 8, 2);
    } else {
      if (qt == 1) K8SLLM_LL(10, 16, 1); else K8SLLM_LL(10, 16, 2);
    }
#undef K8SLLM_LL
    return (int)hipGetLastError();
  }
  if (split != 0 && split != 1 && split != 2 && split != 4 && split != 8) return -1;
  const int nw = split == 4 || split == 8 ? split : ((split == 1 || split == 2) ? 1 : 8);
  const int qt = (cu != nullptr && split == 2) ? 2 : 1;
  const dim3 grid((unsigned)(qt == 1 ? T : T / qt + S), hgs);
#define K8SLLM_LA(KS, DT, NW, QT)                                                                                      \
  hipLaunchKernelGGL((latent_attn_mfma_kernel<KS, DT, NW, QT>), grid, dim3(64 * NW), 0, s, (bf16_t*)out,                \
                     (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, cu, ctx, seq_lens,     \
                     block_tables, bt_stride, S, H, dkp, dv, scale, window, sinks)
#define K8SLLM_LAS(KS, DT)                                            \
  if (nw == 8) K8SLLM_LA(KS, DT, 8, 1);                               \
  else if (nw == 4) K8SLLM_LA(KS, DT, 4, 1);                          \
  else if (qt == 2) K8SLLM_LA(KS, DT, 1, 2);                          \
  else K8SLLM_LA(KS, DT, 1, 1)
  if (dkp <= 128 && dv <= 128) { K8SLLM_LAS(4, 8); }
  else { K8SLLM_LAS(10, 16); }
#undef K8SLLM_LAS
#undef K8SLLM_LA
  return (int)hipGetLastError();
}
}
