// PyTorch bindings of the layer-list decoders' kernels (_k8sllm_hybrid).  Validates tensors (every
// shape the kernels index by is checked here, on the host), picks the current HIP stream (so every
// op is hipGraph-capturable) and calls the C launchers.  Activations are bfloat16 or float32.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

extern "C" {
int k8sllm_hy_embed_pos(float* out, const int* ids, const int* positions, const void* emb, const void* pos,
                        const int* src, const int* prev, long T, int d, int vocab, int max_pos, float scale, int f32,
                        hipStream_t s);
int k8sllm_hy_sum_norm(void* out, float* residual, const void* a0, int t0, float s0, const void* a1, int t1, float s1,
                       const void* y, int ty, const float* wy, const float* w, long rows, int d, float eps, int center,
                       int one_plus, int f32, hipStream_t s);
int k8sllm_hy_gated_lookup(void* out, const void* gate, const void* table, long t_stride, int col, const int* ids,
                           const int* src, const int* prev, long rows, int n, int vocab, int f32, hipStream_t s);
int k8sllm_hy_rotary_norm_cache(void* qkv, long stride, long T, int Hq, int G, int dk, int dv, const int* positions,
                                const float* freq, int nf, int pairs, int norm, const float* qw, const float* kw,
                                float eps, const float* q_scale, void* k_cache, void* v_cache, const int* slots, int bs,
                                int v_from_k, int f32, hipStream_t s);
int k8sllm_hy_decay_scan(float* o, const void* qkv, long stride, int q_col, int k_col, int v_col, const void* z,
                         long z_stride, const float* z_bias, const float* a_log, float inv_tau, const void* beta,
                         long b_stride, float* state, const int* cu, const int* ctx, const int* slot, int S, int H, int Gk,
                         int dk, int dv, float q_scale, int unit, int f32, float* ws, long T, hipStream_t s);
long k8sllm_hy_decay_scan_ws(long T, int H, int Gk, int dk);
int k8sllm_hy_router_grouped(int* ids, float* wts, const void* h, long T, int d, const float* wr, int E, int K,
                             int groups, int keep, float scale, int f32, hipStream_t s);
int k8sllm_hy_add_norm(void* out, float* residual, const void* a0, int t0, const void* a1, int t1, const void* a2,
                       int t2, const float* vec, const float* w, long rows, int d, float eps, int one_plus, int f32,
                       hipStream_t s);
int k8sllm_hy_gated_group_norm(void* out, const float* y, const void* z, long z_stride, const float* w, long rows,
                               int n, int groups, float eps, int after, int f32, hipStream_t s);
int k8sllm_hy_gated_add_norm(void* out, float* residual, const void* y, int yt, const void* gate, long g_stride,
                             const float* bias, float mult, const float* w, long rows, int d, float eps, int one_plus,
                             int vec, int f32, hipStream_t s);
int k8sllm_hy_glu(void* out, const void* gu, long g_stride, long rows, int f, int kind, float limit, int vec, int f32,
                  hipStream_t s);
int k8sllm_hy_activation_cols(void* out, const void* x, long x_stride, long rows, int n, int kind, int vec, int f32,
                              hipStream_t s);
int k8sllm_hy_sigmoid_gate(void* x, const void* z, long z_stride, long rows, int n, int vec, int f32, hipStream_t s);
int k8sllm_hy_softcap(float* x, long n, float cap, hipStream_t s);
int k8sllm_hy_rotary_cache(void* qkv, long stride, long T, int Hq, int G, int dk, int dv, const int* positions,
                           const float* freq, int nf, int pairs, int rot_off, int rot_k, const float* q_scale,
                           void* k_cache, void* v_cache, const int* slots, int bs, int f32, hipStream_t s);
int k8sllm_hy_swiglu(void* out, const void* gu, long rows, int f, int f32, hipStream_t s);
int k8sllm_hy_qk_norm_cache(void* qkv, long stride, const float* qw, const float* kw, float eps, long T, int nq,
                            int nk, int nv, void* k_cache, void* v_cache, const int* slots, int bs, int f32, hipStream_t s);
int k8sllm_hy_window_prefill(void* out, const void* qkv, long q_stride, const void* k_cache, const void* v_cache,
                             const int* cu, const int* ctx, const int* block_tables, int bt_stride, int S, long T,
                             int Hq, int G, int dk, int dv, int bs, float scale, int window, int sink,
                             const float* sinks, int f32, int mfma, hipStream_t s);
int k8sllm_hy_window_decode(void* out, const void* qkv, long q_stride, const void* k_cache, const void* v_cache,
                            const int* block_tables, int bt_stride, const int* seq_lens, int B, int Hq, int G, int dk,
                            int dv, int bs, float scale, int window, int sink, const float* sinks, int f32, int vec,
                            hipStream_t s);
int k8sllm_hy_conv_silu(void* out, const void* proj, long stride, int col0, int C, const float* cw, const float* cb,
                        int taps, void* state, const int* cu, const int* ctx, const int* slot, int S, long T, int f32,
                        hipStream_t s);
int k8sllm_hy_ssm_scan(float* y, const void* xbc, const void* proj, long p_stride, int dt_col, const float* dt_bias,
                       const float* a_log, const float* d_skip, const float* decay, float* state, const int* cu,
                       const int* ctx, const int* slot, int S, long T, int nh, int P, int N, int G, int f32, int mode,
                       hipStream_t s);
int k8sllm_hy_linear_attn_chunk(float* y, const void* vkq, const float* decay, float* state, const int* cu,
                                const int* ctx, const int* slot, int S, int H, int dk, int dv, int nt, hipStream_t s);
int k8sllm_hy_router(int* ids, float* wts, float* gate, const void* h, long T, int d, const float* wr,
                     const float* bias, int E, int K, int rows_w, int over_all, int f32, hipStream_t s);
int k8sllm_hy_grouped_gemm(void* Y, const void* A, const void* W, const int* offsets, const int* sorted_idx, int div,
                           int E, long rows, int N, int Kd, long w_es, int act, int il, int f32, int mfma, float limit,
                           hipStream_t s);
int k8sllm_hy_combine(float* out, const void* ys, const int* inv, const float* wts, const void* shared,
                      const float* gate, long T, int K, int d, int f32, hipStream_t s);
int k8sllm_hy_norm_shift(void* out, const float* x, const float* w, const float* mu, float* state, const int* cu,
                         const int* ctx, const int* slot, int S, long rows, int d, float eps, int one_plus,
                         int advance, int multi, int f32, hipStream_t s);
int k8sllm_hy_depth_mix(float* stack, long plane, int n, const void* addend, int adt, const float* coef,
                        hipStream_t s);
int k8sllm_hy_activation(void* out, const void* x, long n, int kind, float a, float b, int f32, hipStream_t s);
int k8sllm_hy_latent_prep(void* proj, long stride, long T, int Q, int R, int dr, const float* qw, const float* kw,
                          float eps, const int* positions, const float* freq, int nf, int pairs, void* k_cache,
                          int kw_pitch, void* v_cache, const int* slots, int bs, int f32, hipStream_t s);
int k8sllm_hy_latent_queries(void* out, const void* q, long q_stride, const void* q_lat, long T, int H, int dn, int dr,
                             int R, int w, const int* positions, const float* freq, int nf, int pairs, int f32,
                             hipStream_t s);
int k8sllm_hy_latent_attention(void* out, const void* q, long q_stride, const void* k_cache, const void* v_cache,
                               const int* cu, const int* ctx, const int* seq_lens, const int* block_tables,
                               int bt_stride, int S, long T, int H, int dkp, int dv, int bs, float scale, int window,
                               const float* sinks, int split, hipStream_t s);
int k8sllm_moe_align(const int* topk_ids, long n, int E, int* expert_offsets, int* sorted_idx, int* inv_idx,
                     hipStream_t s);
}

namespace {

using torch::Tensor;
using OptT = c10::optional<Tensor>;

hipStream_t cur() { return c10::hip::getCurrentHIPStream().stream(); }
void check(int rc, const char* what) { TORCH_CHECK(rc == 0, "k8sllm hybrid kernel launch failed: ", what, " rc=", rc); }

// activation dtype: 1 = fp32, 0 = bf16
int act(const Tensor& t, const char* n) {
  TORCH_CHECK(t.is_cuda(), n, " must be a GPU tensor");
  TORCH_CHECK(t.scalar_type() == torch::kBFloat16 || t.scalar_type() == torch::kFloat32, n, " must be bf16 or fp32");
  return t.scalar_type() == torch::kFloat32;
}
void same(const Tensor& t, int f32, const char* n) { TORCH_CHECK(act(t, n) == f32, n, ": activation dtype mismatch"); }
void f32c(const Tensor& t, const char* n) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kFloat32 && t.is_contiguous(), n, " must be contiguous fp32 on the GPU");
}
void i32c(const Tensor& t, const char* n) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kInt32 && t.is_contiguous(), n, " must be contiguous int32 on the GPU");
}
const int* iptr(const OptT& t, const char* n) {
  if (!t.has_value()) return nullptr;
  i32c(*t, n);
  return t->data_ptr<int>();
}
int any_dt(const OptT& t, int64_t numel, const char* n) {  // 0 none, 1 bf16, 2 fp32
  if (!t.has_value()) return 0;
  const int f = act(*t, n);
  TORCH_CHECK(t->is_contiguous() && t->numel() == numel, n, " must be contiguous and match the residual");
  return f ? 2 : 1;
}

void embed_pos(Tensor out, Tensor ids, Tensor positions, Tensor emb, OptT pos, OptT src, OptT prev, double scale) {
  const int f = act(emb, "embed");
  f32c(out, "out");
  i32c(ids, "ids");
  i32c(positions, "positions");
  TORCH_CHECK(emb.dim() == 2 && emb.is_contiguous(), "embed [V, d]");
  const int64_t T = ids.numel(), d = emb.size(1);
  TORCH_CHECK(out.numel() == T * d && positions.numel() >= T, "embed_pos: sizes");
  int maxp = 1;
  if (pos.has_value()) {
    same(*pos, f, "pos");
    TORCH_CHECK(pos->dim() == 2 && pos->is_contiguous() && pos->size(1) == d, "pos [P, d]");
    maxp = (int)pos->size(0);
  }
  const int* sp = iptr(src, "src");
  const int* pp = iptr(prev, "prev");
  TORCH_CHECK((sp == nullptr) == (pp == nullptr), "src and prev come together");
  if (sp) {
    TORCH_CHECK(src->numel() >= T && prev->numel() >= 1, "src / prev sizes");
  }
  check(k8sllm_hy_embed_pos(out.data_ptr<float>(), ids.data_ptr<int>(), positions.data_ptr<int>(), emb.data_ptr(),
                            pos.has_value() ? pos->data_ptr() : nullptr, sp, pp, T, (int)d, (int)emb.size(0), maxp, (float)scale, f, cur()),
        "embed_pos");
}

void add_norm(Tensor out, Tensor residual, OptT a0, OptT a1, OptT a2, OptT vec, Tensor w, double eps, bool one_plus) {
  const int f = act(out, "out");
  f32c(residual, "residual");
  f32c(w, "w");
  TORCH_CHECK(residual.dim() == 2 && out.is_contiguous() && out.numel() == residual.numel(), "add_norm: out shape");
  const int64_t rows = residual.size(0), d = residual.size(1);
  TORCH_CHECK(w.numel() == d, "add_norm: w [d]");
  const int t0 = any_dt(a0, rows * d, "addend 0"), t1 = any_dt(a1, rows * d, "addend 1"), t2 = any_dt(a2, rows * d, "addend 2");
  if (vec.has_value()) {
    f32c(*vec, "vec");
    TORCH_CHECK(vec->numel() == d, "add_norm: vec [d]");
  }
  check(k8sllm_hy_add_norm(out.data_ptr(), residual.data_ptr<float>(), t0 ? a0->data_ptr() : nullptr, t0,
                           t1 ? a1->data_ptr() : nullptr, t1, t2 ? a2->data_ptr() : nullptr, t2,
                           vec.has_value() ? vec->data_ptr<float>() : nullptr, w.data_ptr<float>(), rows, (int)d, (float)eps,
                           one_plus, f, cur()),
        "add_norm");
}

// after 0: norm(y * silu(z)) * w;  1: norm(y) * w * sigmoid(z);  2: norm(y) * w * silu(z)
void gated_group_norm(Tensor out, Tensor y, Tensor proj, int64_t z_col, Tensor w, double eps, int64_t groups,
                      int64_t after) {
  TORCH_CHECK(after >= 0 && after <= 2, "gated_group_norm: mode");
  const int f = act(out, "out");
  same(proj, f, "proj");
  f32c(y, "y");
  f32c(w, "w");
  TORCH_CHECK(y.dim() == 2 && proj.dim() == 2 && proj.stride(1) == 1 && proj.size(0) == y.size(0), "gated_group_norm: rows");
  const int64_t n = y.size(1);
  TORCH_CHECK(out.is_contiguous() && out.numel() == y.numel() && w.numel() == n && z_col >= 0 && z_col + n <= proj.size(1) &&
                  groups >= 1 && n % groups == 0,
              "gated_group_norm: shapes");
  check(k8sllm_hy_gated_group_norm(out.data_ptr(), y.data_ptr<float>(),
                                   (const char*)proj.data_ptr() + z_col * proj.element_size(), proj.stride(0),
                                   w.data_ptr<float>(), y.size(0), (int)n, (int)groups, (float)eps, (int)after, f, cur()),
        "gated_group_norm");
}

// true when 8-wide accesses of a column range [col, col + n) of rows `stride` apart are aligned
bool vec8(const Tensor& t, int64_t col, int64_t n) {
  return n % 8 == 0 && col % 8 == 0 && t.stride(0) % 8 == 0 &&
         reinterpret_cast<uintptr_t>(t.data_ptr()) % (8 * t.element_size()) == 0;
}

void gated_add_norm(Tensor out, Tensor residual, Tensor y, Tensor proj, int64_t g_col, Tensor bias, double mult, Tensor w,
                    double eps, bool one_plus) {
  const int f = act(out, "out");
  same(proj, f, "gate");
  f32c(residual, "residual");
  f32c(w, "w");
  f32c(bias, "gate bias");
  TORCH_CHECK(residual.dim() == 2 && out.is_contiguous() && out.numel() == residual.numel(), "gated_add_norm: out shape");
  const int64_t rows = residual.size(0), d = residual.size(1);
  TORCH_CHECK(w.numel() == d && bias.numel() == d, "gated_add_norm: w, bias [d]");
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1 && proj.size(0) == rows && g_col >= 0 && g_col + d <= proj.size(1),
              "gated_add_norm: gate columns");
  const int yt = any_dt(y, rows * d, "y");
  const bool v = vec8(proj, g_col, d);
  check(k8sllm_hy_gated_add_norm(out.data_ptr(), residual.data_ptr<float>(), y.data_ptr(), yt,
                                 (const char*)proj.data_ptr() + g_col * proj.element_size(), proj.stride(0),
                                 bias.data_ptr<float>(), (float)mult, w.data_ptr<float>(), rows, (int)d, (float)eps, one_plus,
                                 v, f, cur()),
        "gated_add_norm");
}

// out [rows, f] = act(proj[:, col : col + f]) * proj[:, col + f : col + 2f]; kind 1 tanh GELU, 3 SiLU, 4 ReLU,
// 5 the clamped unit g sigmoid(1.702 g) (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit)
void glu(Tensor out, Tensor proj, int64_t col, int64_t kind, double limit) {
  const int f = act(proj, "proj");
  same(out, f, "out");
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1 && out.dim() == 2 && out.is_contiguous() && out.size(0) == proj.size(0),
              "glu: layouts");
  const int64_t n = out.size(1);
  TORCH_CHECK(col >= 0 && col + 2 * n <= proj.size(1) && (kind == 1 || kind == 3 || kind == 4 || (kind == 5 && limit > 0)),
              "glu: columns / kind");
  check(k8sllm_hy_glu(out.data_ptr(), (const char*)proj.data_ptr() + col * proj.element_size(), proj.stride(0), proj.size(0),
                      (int)n, (int)kind, (float)limit, vec8(proj, col, n), f, cur()),
        "glu");
}

// out [rows, n] = act(proj[:, col : col + n]); kind 0 erf GELU, 1 tanh GELU, 3 SiLU
void activation_cols(Tensor out, Tensor proj, int64_t col, int64_t kind) {
  const int f = act(proj, "proj");
  same(out, f, "out");
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1 && out.dim() == 2 && out.is_contiguous() && out.size(0) == proj.size(0),
              "activation_cols: layouts");
  const int64_t n = out.size(1);
  TORCH_CHECK(col >= 0 && col + n <= proj.size(1) && (kind == 0 || kind == 1 || kind == 3), "activation_cols: columns / kind");
  check(k8sllm_hy_activation_cols(out.data_ptr(), (const char*)proj.data_ptr() + col * proj.element_size(), proj.stride(0),
                                  proj.size(0), (int)n, (int)kind, vec8(proj, col, n), f, cur()),
        "activation_cols");
}

// x [rows, n] *= sigmoid(proj[:, col : col + n])
void sigmoid_gate(Tensor x, Tensor proj, int64_t col) {
  const int f = act(x, "x");
  same(proj, f, "gate");
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous() && proj.dim() == 2 && proj.stride(1) == 1 && proj.size(0) == x.size(0),
              "sigmoid_gate: layouts");
  const int64_t n = x.size(1);
  TORCH_CHECK(col >= 0 && col + n <= proj.size(1), "sigmoid_gate: columns");
  check(k8sllm_hy_sigmoid_gate(x.data_ptr(), (const char*)proj.data_ptr() + col * proj.element_size(), proj.stride(0),
                               x.size(0), (int)n, vec8(proj, col, n), f, cur()),
        "sigmoid_gate");
}

void softcap(Tensor x, double cap) {
  f32c(x, "logits");
  TORCH_CHECK(cap > 0, "softcap: cap > 0");
  check(k8sllm_hy_softcap(x.data_ptr<float>(), x.numel(), (float)cap, cur()), "softcap");
}

void swiglu(Tensor out, Tensor gu) {
  const int f = act(gu, "gu");
  same(out, f, "out");
  TORCH_CHECK(gu.dim() == 2 && gu.is_contiguous() && out.is_contiguous() && gu.size(1) % 2 == 0 &&
                  out.numel() * 2 == gu.numel(),
              "swiglu: shapes");
  check(k8sllm_hy_swiglu(out.data_ptr(), gu.data_ptr(), gu.size(0), (int)(gu.size(1) / 2), f, cur()), "swiglu");
}

// key pages [blocks, bs, width]
void pages(const Tensor& c, int f, int64_t width, const char* n) {
  same(c, f, n);
  TORCH_CHECK(c.dim() == 3 && c.is_contiguous() && c.size(2) == width, n, " must be [blocks, block, heads*dim]");
}
// value pages [blocks, G, dv, bs] matching the key pages' block count and size
void vpages(const Tensor& c, const Tensor& k, int f, int64_t G, int64_t dv) {
  same(c, f, "v_cache");
  TORCH_CHECK(c.dim() == 4 && c.is_contiguous() && c.size(0) == k.size(0) && c.size(1) == G && c.size(2) == dv &&
                  c.size(3) == k.size(1),
              "v_cache must be [blocks, kv_heads, vdim, block]");
}

// learned sink logits, one per query head (absent: every sink's logit is 0)
const float* sink_ptr(const OptT& sinks, int64_t Hq) {
  if (!sinks.has_value()) return nullptr;
  f32c(*sinks, "sinks");
  TORCH_CHECK(sinks->numel() == Hq, "sinks [Hq]");
  return sinks->data_ptr<float>();
}

void qk_norm_cache(Tensor qkv, Tensor qw, Tensor kw, double eps, int64_t Hq, int64_t G, int64_t dk, int64_t dv,
                   OptT k_cache, OptT v_cache, OptT slots) {
  const int f = act(qkv, "qkv");
  f32c(qw, "qw");
  f32c(kw, "kw");
  const int64_t nq = Hq * dk, nk = G * dk, nv = G * dv;
  TORCH_CHECK(qkv.dim() == 2 && qkv.stride(1) == 1 && qkv.size(1) == nq + nk + nv, "qkv [T, Hq*dk + G*dk + G*dv]");
  TORCH_CHECK(qw.numel() == nq && kw.numel() == nk, "q / k norm weights");
  void *kc = nullptr, *vc = nullptr;
  const int* sp = nullptr;
  if (k_cache.has_value()) {
    TORCH_CHECK(v_cache.has_value() && slots.has_value(), "k_cache, v_cache and slot_mapping come together");
    pages(*k_cache, f, nk, "k_cache");
    vpages(*v_cache, *k_cache, f, G, dv);
    sp = iptr(slots, "slot_mapping");
    TORCH_CHECK(slots->numel() >= qkv.size(0), "slot_mapping [T]");
    kc = k_cache->data_ptr();
    vc = v_cache->data_ptr();
  }
  check(k8sllm_hy_qk_norm_cache(qkv.data_ptr(), qkv.stride(0), qw.data_ptr<float>(), kw.data_ptr<float>(), (float)eps,
                                qkv.size(0), (int)nq, (int)nk, (int)nv, kc, vc, sp,
                                k_cache.has_value() ? (int)k_cache->size(1) : 16, f, cur()),
        "qk_norm_cache");
}

void window_attention_prefill(Tensor out, Tensor qkv, Tensor k_cache, Tensor v_cache, Tensor cu, Tensor ctx,
                              Tensor block_tables, int64_t Hq, int64_t G, int64_t dk, int64_t dv, double scale,
                              int64_t window, bool sink, OptT sinks, int64_t mfma) {
  const int f = act(qkv, "qkv");
  same(out, f, "out");
  pages(k_cache, f, G * dk, "k_cache");
  vpages(v_cache, k_cache, f, G, dv);
  i32c(cu, "cu");
  i32c(ctx, "ctx");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == torch::kInt32 && block_tables.dim() == 2 &&
                  block_tables.stride(1) == 1,
              "block_tables [S, W] int32");
  const int64_t T = qkv.size(0), S = ctx.numel();
  TORCH_CHECK(qkv.dim() == 2 && qkv.stride(1) == 1 && qkv.size(1) >= Hq * dk, "qkv rows");
  TORCH_CHECK(out.is_contiguous() && out.numel() == T * Hq * dv, "out [T, Hq*dv]");
  TORCH_CHECK(cu.numel() == S + 1 && block_tables.size(0) >= S, "cu [S+1], block_tables [S, W]");
  TORCH_CHECK(window >= 0 && G >= 1 && Hq % G == 0, "heads / window");
  check(k8sllm_hy_window_prefill(out.data_ptr(), qkv.data_ptr(), qkv.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
                                 cu.data_ptr<int>(), ctx.data_ptr<int>(), block_tables.data_ptr<int>(),
                                 (int)block_tables.stride(0), (int)S, T, (int)Hq, (int)G, (int)dk, (int)dv,
                                 (int)k_cache.size(1), (float)scale, (int)window, sink, sink_ptr(sinks, Hq), f,
                                 (int)mfma, cur()),
        "window_attention_prefill");
}

void window_attention_decode(Tensor out, Tensor qkv, Tensor k_cache, Tensor v_cache, Tensor block_tables,
                             Tensor seq_lens, int64_t Hq, int64_t G, int64_t dk, int64_t dv, double scale,
                             int64_t window, bool sink, OptT sinks, bool vec) {
  const int f = act(qkv, "qkv");
  same(out, f, "out");
  pages(k_cache, f, G * dk, "k_cache");
  vpages(v_cache, k_cache, f, G, dv);
  i32c(seq_lens, "seq_lens");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == torch::kInt32 && block_tables.dim() == 2 &&
                  block_tables.stride(1) == 1,
              "block_tables [B, W] int32");
  const int64_t B = qkv.size(0);
  TORCH_CHECK(qkv.dim() == 2 && qkv.stride(1) == 1 && qkv.size(1) >= Hq * dk, "qkv rows");
  TORCH_CHECK(out.is_contiguous() && out.numel() == B * Hq * dv, "out [B, Hq*dv]");
  TORCH_CHECK(seq_lens.numel() >= B && block_tables.size(0) >= B, "seq_lens [B], block_tables [B, W]");
  TORCH_CHECK(window >= 0 && G >= 1 && Hq % G == 0, "heads / window");
  check(k8sllm_hy_window_decode(out.data_ptr(), qkv.data_ptr(), qkv.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
                                block_tables.data_ptr<int>(), (int)block_tables.stride(0), seq_lens.data_ptr<int>(),
                                (int)B, (int)Hq, (int)G, (int)dk, (int)dv, (int)k_cache.size(1), (float)scale,
                                (int)window, sink, sink_ptr(sinks, Hq), f, vec, cur()),
        "window_attention_decode");
}

void segs(const Tensor& cu, const Tensor& ctx, const Tensor& slot) {
  i32c(cu, "seg_cu");
  i32c(ctx, "seg_ctx");
  i32c(slot, "seg_slot");
  TORCH_CHECK(cu.numel() == ctx.numel() + 1 && slot.numel() == ctx.numel(), "segments: cu [R+1], ctx [R], slot [R]");
}

void conv_silu(Tensor out, Tensor proj, int64_t col0, Tensor cw, OptT cb, Tensor state, Tensor cu, Tensor ctx,
               Tensor slot) {
  const int f = act(proj, "proj");
  same(out, f, "out");
  same(state, f, "conv_state");
  f32c(cw, "conv_w");
  if (cb.has_value()) f32c(*cb, "conv_b");
  segs(cu, ctx, slot);
  const int64_t T = proj.size(0), C = cw.size(0), taps = cw.size(1);
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1 && col0 >= 0 && col0 + C <= proj.size(1), "proj columns");
  TORCH_CHECK(out.is_contiguous() && out.numel() == T * C && (!cb.has_value() || cb->numel() == C), "conv_silu: out / bias");
  TORCH_CHECK(state.dim() == 3 && state.is_contiguous() && state.size(2) == C && state.size(1) >= taps - 1 &&
                  (taps == 1 || state.size(1) == taps - 1),
              "conv_state [slots, taps-1, C]");
  check(k8sllm_hy_conv_silu(out.data_ptr(), proj.data_ptr(), proj.stride(0), (int)col0, (int)C, cw.data_ptr<float>(),
                            cb.has_value() ? cb->data_ptr<float>() : nullptr, (int)taps, state.data_ptr(), cu.data_ptr<int>(), ctx.data_ptr<int>(),
                            slot.data_ptr<int>(), (int)ctx.numel(), T, f, cur()),
        "conv_silu");
}

// decay given: the fixed-decay recurrence (dt = 1, no skip term); proj, dt_bias, a_log, d_skip are then not read
void ssm_scan(Tensor y, Tensor xbc, OptT proj, int64_t dt_col, OptT dt_bias, OptT a_log, OptT d_skip, OptT decay,
              Tensor state, Tensor cu, Tensor ctx, Tensor slot, int64_t nh, int64_t P, int64_t N, int64_t G,
              int64_t mode) {
  const int f = act(xbc, "xbc");
  f32c(y, "y");
  f32c(state, "ssm_state");
  segs(cu, ctx, slot);
  const int64_t T = xbc.size(0);
  TORCH_CHECK(xbc.dim() == 2 && xbc.is_contiguous() && xbc.size(1) == nh * P + 2 * G * N, "xbc [T, nh*P + 2*G*N]");
  const void* pp = nullptr;
  long pstride = 0;
  const float *bp = nullptr, *ap = nullptr, *dp = nullptr, *cp = nullptr;
  if (decay.has_value()) {
    f32c(*decay, "decay");
    TORCH_CHECK(decay->numel() == nh, "decay [heads]");
    cp = decay->data_ptr<float>();
  } else {
    TORCH_CHECK(proj.has_value() && dt_bias.has_value() && a_log.has_value() && d_skip.has_value(), "ssm: dt inputs");
    same(*proj, f, "proj");
    f32c(*dt_bias, "dt_bias");
    f32c(*a_log, "A_log");
    f32c(*d_skip, "D");
    TORCH_CHECK(proj->dim() == 2 && proj->stride(1) == 1 && proj->size(0) == T && dt_col >= 0 && dt_col + nh <= proj->size(1),
                "proj dt columns");
    TORCH_CHECK(dt_bias->numel() == nh && a_log->numel() == nh && d_skip->numel() == nh, "ssm sizes");
    pp = proj->data_ptr();
    pstride = proj->stride(0);
    bp = dt_bias->data_ptr<float>();
    ap = a_log->data_ptr<float>();
    dp = d_skip->data_ptr<float>();
  }
  TORCH_CHECK(y.numel() == T * nh * P, "ssm: y [T, nh*P]");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == nh && state.size(2) == N && state.size(3) == P, "ssm_state [slots, nh, N, P]");
  TORCH_CHECK(G >= 1 && nh % G == 0 && N <= 256, "ssm: groups / state size (<= 256)");
  check(k8sllm_hy_ssm_scan(y.data_ptr<float>(), xbc.data_ptr(), pp, pstride, (int)dt_col, bp, ap, dp, cp,
                           state.data_ptr<float>(), cu.data_ptr<int>(), ctx.data_ptr<int>(), slot.data_ptr<int>(),
                           (int)ctx.numel(), T, (int)nh, (int)P, (int)N, (int)G, f, (int)mode, cur()),
        "ssm_scan");
}

// The matrix-core (chunked) linear attention for bf16 prompts; false: these sizes or dtype are not the
// kernel's, nothing was launched.
bool linear_attention_chunked(Tensor y, Tensor vkq, Tensor decay, Tensor state, Tensor cu, Tensor ctx, Tensor slot,
                              int64_t H, int64_t dk, int64_t dv, int64_t nt) {
  if (act(vkq, "vkq") != 0) return false;
  f32c(y, "y");
  f32c(decay, "decay");
  f32c(state, "state");
  segs(cu, ctx, slot);
  const int64_t T = vkq.size(0);
  TORCH_CHECK(vkq.dim() == 2 && vkq.is_contiguous() && vkq.size(1) == H * dv + 2 * H * dk, "vkq [T, H*dv + 2*H*dk]");
  TORCH_CHECK(y.numel() == T * H * dv && decay.numel() == H, "linear attention: y [T, H*dv], decay [H]");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == dk && state.size(3) == dv,
              "state [slots, H, dk, dv]");
  const int rc = k8sllm_hy_linear_attn_chunk(y.data_ptr<float>(), vkq.data_ptr(), decay.data_ptr<float>(),
                                             state.data_ptr<float>(), cu.data_ptr<int>(), ctx.data_ptr<int>(),
                                             slot.data_ptr<int>(), (int)ctx.numel(), (int)H, (int)dk, (int)dv, (int)nt, cur());
  if (rc == 1) return false;
  check(rc, "linear_attention_chunked");
  return true;
}

// In place on the fused rows [T, Hq*dk | G*dk | G*dv | ...]: rotary positions on the first 2 * len(freq)
// entries of every q / k head (pairs: entry 2i with 2i + 1, else i with i + len(freq)), q heads times
// q_scale [Hq] (optional), k and v to the pages.  rot_off: the turning entries start there in every head;
// rot_k false: the keys are copied as they are.
void rotary_cache(Tensor qkv, int64_t Hq, int64_t G, int64_t dk, int64_t dv, Tensor positions, Tensor freq, bool pairs,
                  OptT q_scale, OptT k_cache, OptT v_cache, OptT slots, int64_t rot_off, bool rot_k) {
  const int f = act(qkv, "qkv");
  f32c(freq, "freq");
  i32c(positions, "positions");
  const int64_t nq = Hq * dk, nk = G * dk, nv = G * dv, T = qkv.size(0);
  TORCH_CHECK(qkv.dim() == 2 && qkv.stride(1) == 1 && qkv.size(1) >= nq + nk + nv, "qkv [T, Hq*dk + G*dk + G*dv (+ more)]");
  TORCH_CHECK(Hq >= 1 && G >= 1 && positions.numel() >= T && rot_off >= 0 && rot_off + 2 * freq.numel() <= dk,
              "rotary_cache: heads / positions / freq");
  const float* qs = nullptr;
  if (q_scale.has_value()) {
    f32c(*q_scale, "q_scale");
    TORCH_CHECK(q_scale->numel() == Hq, "q_scale [Hq]");
    qs = q_scale->data_ptr<float>();
  }
  void *kc = nullptr, *vc = nullptr;
  const int* sp = nullptr;
  if (k_cache.has_value()) {
    TORCH_CHECK(v_cache.has_value() && slots.has_value(), "k_cache, v_cache and slot_mapping come together");
    pages(*k_cache, f, nk, "k_cache");
    vpages(*v_cache, *k_cache, f, G, dv);
    sp = iptr(slots, "slot_mapping");
    TORCH_CHECK(slots->numel() >= T, "slot_mapping [T]");
    kc = k_cache->data_ptr();
    vc = v_cache->data_ptr();
  }
  check(k8sllm_hy_rotary_cache(qkv.data_ptr(), qkv.stride(0), T, (int)Hq, (int)G, (int)dk, (int)dv, positions.data_ptr<int>(),
                               freq.data_ptr<float>(), (int)freq.numel(), pairs, (int)rot_off, rot_k, qs, kc, vc, sp,
                               k_cache.has_value() ? (int)k_cache->size(1) : 16, f, cur()),
        "rotary_cache");
}

void moe_router(Tensor ids, Tensor wts, OptT gate, Tensor h, Tensor wr, OptT bias, int64_t E, int64_t K,
                bool over_all) {
  const int f = act(h, "h");
  i32c(ids, "ids");
  f32c(wts, "wts");
  f32c(wr, "router weight");
  if (bias.has_value()) {
    f32c(*bias, "router bias");
    TORCH_CHECK(bias->numel() >= E, "router bias [E]");
  }
  const int64_t T = h.size(0), d = h.size(1);
  TORCH_CHECK(h.dim() == 2 && h.is_contiguous() && wr.dim() == 2 && wr.size(1) == d, "router: h [T, d], wr [E(+1), d]");
  TORCH_CHECK(wr.size(0) == E || wr.size(0) == E + 1, "router rows");
  TORCH_CHECK(ids.numel() == T * K && wts.numel() == T * K, "router: outputs");
  TORCH_CHECK(E <= 256 && K >= 1 && K <= 16 && K <= E, "router: up to 256 experts, top 16");
  float* gp = nullptr;
  if (gate.has_value()) {
    f32c(*gate, "gate");
    TORCH_CHECK(gate->numel() == T && wr.size(0) == E + 1, "gate [T] needs the extra router row");
    gp = gate->data_ptr<float>();
  }
  check(k8sllm_hy_router(ids.data_ptr<int>(), wts.data_ptr<float>(), gp, h.data_ptr(), T, (int)d, wr.data_ptr<float>(),
                         bias.has_value() ? bias->data_ptr<float>() : nullptr, (int)E, (int)K, (int)wr.size(0), over_all,
                         f, cur()),
        "moe_router");
}

// addends: any float dtype, contiguous [rows, d]; returns 0 / 1 (bf16) / 2 (fp32)
void sum_norm(Tensor out, Tensor residual, OptT a0, double s0, OptT a1, double s1, OptT y, OptT wy, OptT w, double eps,
              bool center, bool one_plus) {
  const int f = act(out, "out");
  f32c(residual, "residual");
  TORCH_CHECK(residual.dim() == 2 && out.is_contiguous() && out.numel() == residual.numel(), "sum_norm: out shape");
  const int64_t rows = residual.size(0), d = residual.size(1);
  const int t0 = any_dt(a0, rows * d, "addend 0"), t1 = any_dt(a1, rows * d, "addend 1"), ty = any_dt(y, rows * d, "normed addend");
  const float *wyp = nullptr, *wp = nullptr;
  if (ty) {
    TORCH_CHECK(wy.has_value(), "sum_norm: the normed addend needs its weight");
    f32c(*wy, "normed addend weight");
    TORCH_CHECK(wy->numel() == d, "sum_norm: wy [d]");
    wyp = wy->data_ptr<float>();
  }
  if (w.has_value()) {
    f32c(*w, "w");
    TORCH_CHECK(w->numel() == d, "sum_norm: w [d]");
    wp = w->data_ptr<float>();
  }
  check(k8sllm_hy_sum_norm(out.data_ptr(), residual.data_ptr<float>(), t0 ? a0->data_ptr() : nullptr, t0, (float)s0,
                           t1 ? a1->data_ptr() : nullptr, t1, (float)s1, ty ? y->data_ptr() : nullptr, ty, wyp, wp, rows,
                           (int)d, (float)eps, center, one_plus, f, cur()),
        "sum_norm");
}

// out [T, n] = gelu_tanh(gate) * table[id, col : col + n]
void gated_lookup(Tensor out, Tensor gate, Tensor table, Tensor ids, int64_t col, OptT src, OptT prev) {
  const int f = act(gate, "gate");
  same(out, f, "out");
  same(table, f, "table");
  i32c(ids, "ids");
  TORCH_CHECK(gate.dim() == 2 && gate.is_contiguous() && out.is_contiguous() && out.numel() == gate.numel(), "gated_lookup: gate / out");
  TORCH_CHECK(table.dim() == 2 && table.stride(1) == 1, "gated_lookup: table [V, *]");
  const int64_t T = gate.size(0), n = gate.size(1);
  TORCH_CHECK(ids.numel() >= T && col >= 0 && col + n <= table.size(1), "gated_lookup: ids / columns");
  const int* sp = iptr(src, "src");
  const int* pp = iptr(prev, "prev");
  TORCH_CHECK((sp == nullptr) == (pp == nullptr), "src and prev come together");
  if (sp) {
    TORCH_CHECK(src->numel() >= T && prev->numel() >= 1, "src / prev sizes");
  }
  check(k8sllm_hy_gated_lookup(out.data_ptr(), gate.data_ptr(), table.data_ptr(), table.stride(0), (int)col,
                               ids.data_ptr<int>(), sp, pp, T, (int)n, (int)table.size(0), f, cur()),
        "gated_lookup");
}

// rotary_cache with an RMS norm of every q / k head (norm 1: before the turn, weights qw / kw [dk]; 2: after
// it, no weight); v_from_k: rows are [q | k | ...] and the value pages take the keys as projected
void rotary_norm_cache(Tensor qkv, int64_t Hq, int64_t G, int64_t dk, int64_t dv, Tensor positions, Tensor freq, bool pairs,
                       int64_t norm, OptT qw, OptT kw, double eps, OptT q_scale, OptT k_cache, OptT v_cache, OptT slots,
                       bool v_from_k) {
  const int f = act(qkv, "qkv");
  f32c(freq, "freq");
  i32c(positions, "positions");
  const int64_t nq = Hq * dk, nk = G * dk, nv = v_from_k ? 0 : G * dv, T = qkv.size(0);
  TORCH_CHECK(qkv.dim() == 2 && qkv.stride(1) == 1 && qkv.size(1) >= nq + nk + nv, "qkv [T, Hq*dk + G*dk (+ G*dv) (+ more)]");
  TORCH_CHECK(Hq >= 1 && G >= 1 && positions.numel() >= T && 2 * freq.numel() <= dk && dk <= 1024 && norm >= 0 && norm <= 2 &&
                  (!v_from_k || dv == dk),
              "rotary_norm_cache: heads / positions / freq / norm");
  const float *qs = nullptr, *qwp = nullptr, *kwp = nullptr;
  if (q_scale.has_value()) {
    f32c(*q_scale, "q_scale");
    TORCH_CHECK(q_scale->numel() == Hq, "q_scale [Hq]");
    qs = q_scale->data_ptr<float>();
  }
  if (norm == 1) {
    TORCH_CHECK(qw.has_value() && kw.has_value(), "rotary_norm_cache: norm weights");
    f32c(*qw, "qw");
    f32c(*kw, "kw");
    TORCH_CHECK(qw->numel() == dk && kw->numel() == dk, "q / k norm weights [dk]");
    qwp = qw->data_ptr<float>();
    kwp = kw->data_ptr<float>();
  }
  void *kc = nullptr, *vc = nullptr;
  const int* sp = nullptr;
  if (k_cache.has_value()) {
    TORCH_CHECK(v_cache.has_value() && slots.has_value(), "k_cache, v_cache and slot_mapping come together");
    pages(*k_cache, f, nk, "k_cache");
    vpages(*v_cache, *k_cache, f, G, dv);
    sp = iptr(slots, "slot_mapping");
    TORCH_CHECK(slots->numel() >= T, "slot_mapping [T]");
    kc = k_cache->data_ptr();
    vc = v_cache->data_ptr();
  }
  check(k8sllm_hy_rotary_norm_cache(qkv.data_ptr(), qkv.stride(0), T, (int)Hq, (int)G, (int)dk, (int)dv,
                                    positions.data_ptr<int>(), freq.data_ptr<float>(), (int)freq.numel(), pairs, (int)norm,
                                    qwp, kwp, (float)eps, qs, kc, vc, sp, k_cache.has_value() ? (int)k_cache->size(1) : 16,
                                    v_from_k, f, cur()),
        "rotary_norm_cache");
}

// The per-channel-decay recurrence (optionally with the delta rule: beta given); see decay_scan.hip
// ws: fp32 workspace of decay_scan_ws(T, ...) floats - given, the two-launch form for prompts runs
void decay_scan(Tensor o, Tensor qkv, int64_t q_col, int64_t k_col, int64_t v_col, Tensor z, Tensor z_bias, OptT a_log,
                double tau, OptT beta, int64_t beta_col, Tensor state, Tensor cu, Tensor ctx, Tensor slot, int64_t H,
                int64_t Gk, int64_t dk, int64_t dv, double q_scale, bool unit, OptT ws) {
  const int f = act(qkv, "qkv");
  same(z, f, "z");
  f32c(o, "o");
  f32c(z_bias, "z_bias");
  f32c(state, "state");
  segs(cu, ctx, slot);
  const int64_t T = qkv.size(0);
  TORCH_CHECK(H >= 1 && Gk >= 1 && H % Gk == 0 && dk >= 1 && dk <= 256 && dv >= 1 && tau > 0, "decay_scan: sizes (dim <= 256)");
  TORCH_CHECK(qkv.dim() == 2 && qkv.stride(1) == 1 && q_col >= 0 && k_col >= 0 && v_col >= 0 &&
                  q_col + Gk * dk <= qkv.size(1) && k_col + Gk * dk <= qkv.size(1) && v_col + H * dv <= qkv.size(1),
              "decay_scan: q / k / v columns");
  TORCH_CHECK(z.dim() == 2 && z.stride(1) == 1 && z.size(0) == T && z.size(1) == H * dk && z_bias.numel() == H * dk,
              "decay_scan: z [T, H*dk], z_bias [H*dk]");
  TORCH_CHECK(o.numel() == T * H * dv, "decay_scan: o [T, H*dv]");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == dv && state.size(3) == dk, "state [slots, H, dv, dk]");
  const float* ap = nullptr;
  if (a_log.has_value()) {
    f32c(*a_log, "A_log");
    TORCH_CHECK(a_log->numel() == H, "A_log [H]");
    ap = a_log->data_ptr<float>();
  }
  const void* bp = nullptr;
  long bstride = 0;
  if (beta.has_value()) {
    same(*beta, f, "beta");
    TORCH_CHECK(beta->dim() == 2 && beta->stride(1) == 1 && beta->size(0) == T && beta_col >= 0 && beta_col + H <= beta->size(1),
                "decay_scan: beta columns");
    bp = (const char*)beta->data_ptr() + beta_col * beta->element_size();
    bstride = beta->stride(0);
  }
  float* wp = nullptr;
  if (ws.has_value()) {
    f32c(*ws, "workspace");
    TORCH_CHECK(ws->numel() >= k8sllm_hy_decay_scan_ws(T, (int)H, (int)Gk, (int)dk), "decay_scan: workspace too small");
    wp = ws->data_ptr<float>();
  }
  check(k8sllm_hy_decay_scan(o.data_ptr<float>(), qkv.data_ptr(), qkv.stride(0), (int)q_col, (int)k_col, (int)v_col,
                             z.data_ptr(), z.stride(0), z_bias.data_ptr<float>(), ap, (float)(1.0 / tau), bp, bstride,
                             state.data_ptr<float>(), cu.data_ptr<int>(), ctx.data_ptr<int>(), slot.data_ptr<int>(),
                             (int)ctx.numel(), (int)H, (int)Gk, (int)dk, (int)dv, (float)q_scale, unit, f, wp, (long)T, cur()),
        "decay_scan");
}

void moe_router_grouped(Tensor ids, Tensor wts, Tensor h, Tensor wr, int64_t E, int64_t K, int64_t groups, int64_t keep,
                        double scale) {
  const int f = act(h, "h");
  i32c(ids, "ids");
  f32c(wts, "wts");
  f32c(wr, "router weight");
  const int64_t T = h.size(0), d = h.size(1);
  TORCH_CHECK(h.dim() == 2 && h.is_contiguous() && wr.dim() == 2 && wr.size(1) == d && wr.size(0) == E, "router: h [T, d], wr [E, d]");
  TORCH_CHECK(ids.numel() == T * K && wts.numel() == T * K, "router: outputs");
  TORCH_CHECK(E <= 256 && K >= 1 && K <= 16 && groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups &&
                  K <= keep * (E / groups),
              "router: up to 256 experts, top 16 within the kept groups");
  check(k8sllm_hy_router_grouped(ids.data_ptr<int>(), wts.data_ptr<float>(), h.data_ptr(), T, (int)d, wr.data_ptr<float>(),
                                 (int)E, (int)K, (int)groups, (int)keep, (float)scale, f, cur()),
        "moe_router_grouped");
}

void moe_align(Tensor ids, int64_t E, Tensor offsets, Tensor sorted_idx, Tensor inv_idx) {
  i32c(ids, "ids");
  i32c(offsets, "offsets");
  i32c(sorted_idx, "sorted_idx");
  i32c(inv_idx, "inv_idx");
  TORCH_CHECK(offsets.numel() == E + 1 && sorted_idx.numel() == ids.numel() && inv_idx.numel() == ids.numel() && E <= 256,
              "moe_align sizes");
  check(k8sllm_moe_align(ids.data_ptr<int>(), ids.numel(), (int)E, offsets.data_ptr<int>(), sorted_idx.data_ptr<int>(),
                         inv_idx.data_ptr<int>(), cur()),
        "moe_align");
}

// y [rows, N] = W[e] a over expert-sorted rows; sorted_idx given: a's row of sorted row r is sorted_idx[r] / div
// act_code: 0 none, 1 SwiGLU (w = [gate rows ; up rows]), 2 erf GELU
// 3 the clamped gated unit (w = [gate rows ; up rows], limit)
void grouped_gemm(Tensor y, Tensor a, Tensor w, Tensor offsets, OptT sorted_idx, int64_t div, int64_t act_code, bool il,
                  bool mfma, double limit) {
  TORCH_CHECK(act_code >= 0 && act_code <= 3 && (act_code != 3 || limit > 0), "grouped_gemm: activation code");
  const bool swiglu = act_code == 1 || act_code == 3;
  const int f = act(a, "a");
  same(y, f, "y");
  same(w, f, "w");
  i32c(offsets, "offsets");
  TORCH_CHECK(a.dim() == 2 && a.is_contiguous() && w.dim() == 3 && w.is_contiguous() && y.dim() == 2 && y.is_contiguous(),
              "grouped_gemm: layouts");
  const int64_t E = w.size(0), Kd = w.size(2), rows = y.size(0);
  const int64_t N = swiglu ? w.size(1) / 2 : w.size(1);
  TORCH_CHECK(a.size(1) == Kd && y.size(1) == N && offsets.numel() == E + 1 && (!swiglu || w.size(1) % 2 == 0),
              "grouped_gemm: shapes");
  TORCH_CHECK(!il || (act_code == 1 && N % 64 == 0), "grouped_gemm: interleaved gate/up needs swiglu and ff % 64 == 0");
  const int* sp = iptr(sorted_idx, "sorted_idx");
  if (sp) {
    TORCH_CHECK(sorted_idx->numel() == rows && div >= 1 && a.size(0) * div >= rows, "grouped_gemm: gather index");
  } else {
    TORCH_CHECK(a.size(0) == rows, "grouped_gemm: a rows");
  }
  check(k8sllm_hy_grouped_gemm(y.data_ptr(), a.data_ptr(), w.data_ptr(), offsets.data_ptr<int>(), sp, (int)div, (int)E,
                               rows, (int)N, (int)Kd, w.size(1) * Kd, (int)act_code, il, f, mfma, (float)limit, cur()),
        "grouped_gemm");
}

void moe_combine(Tensor out, Tensor ys, Tensor inv, Tensor wts, OptT shared, OptT gate) {
  const int f = act(ys, "ys");
  f32c(out, "out");
  f32c(wts, "wts");
  i32c(inv, "inv_idx");
  const int64_t T = out.size(0), d = out.size(1), K = wts.numel() / std::max<int64_t>(T, 1);
  TORCH_CHECK(out.dim() == 2 && ys.dim() == 2 && ys.is_contiguous() && ys.size(1) == d && ys.size(0) == T * K &&
                  inv.numel() == T * K && wts.numel() == T * K,
              "moe_combine: shapes");
  const void* sh = nullptr;
  const float* gp = nullptr;
  if (shared.has_value()) {
    same(*shared, f, "shared");
    TORCH_CHECK(shared->is_contiguous() && shared->numel() == T * d, "shared [T, d]");
    sh = shared->data_ptr();
    if (gate.has_value()) {
      f32c(*gate, "gate");
      TORCH_CHECK(gate->numel() == T, "gate [T]");
      gp = gate->data_ptr<float>();
    }
  }
  check(k8sllm_hy_combine(out.data_ptr<float>(), ys.data_ptr(), inv.data_ptr<int>(), wts.data_ptr<float>(), sh, gp, T,
                          (int)K, (int)d, f, cur()),
        "moe_combine");
}

void norm_shift(Tensor out, Tensor x, Tensor w, double eps, bool one_plus, Tensor mu, Tensor state, Tensor cu, Tensor ctx,
                Tensor slot, bool advance, bool multi) {
  const int f = act(out, "out");
  f32c(x, "residual");
  f32c(w, "w");
  f32c(mu, "shift");
  f32c(state, "shift state");
  segs(cu, ctx, slot);
  TORCH_CHECK(x.dim() == 2 && out.is_contiguous() && out.numel() == x.numel(), "norm_shift: out shape");
  const int64_t rows = x.size(0), d = x.size(1);
  TORCH_CHECK(w.numel() == d && mu.numel() == d && state.dim() == 2 && state.size(1) == d, "norm_shift: w, shift [d], state [slots, d]");
  check(k8sllm_hy_norm_shift(out.data_ptr(), x.data_ptr<float>(), w.data_ptr<float>(), mu.data_ptr<float>(),
                             state.data_ptr<float>(), cu.data_ptr<int>(), ctx.data_ptr<int>(), slot.data_ptr<int>(),
                             (int)ctx.numel(), rows, (int)d, (float)eps, one_plus, advance, multi, f, cur()),
        "norm_shift");
}

void depth_mix(Tensor stack, int64_t n, OptT addend, Tensor coef) {
  f32c(stack, "stack");
  f32c(coef, "coef");
  TORCH_CHECK(stack.dim() == 3 && n >= 0 && n + 1 < stack.size(0) && coef.numel() == n + 1 && n < 256,
              "depth_mix: stack [L, T, d], coef [n + 1], n + 1 < L");
  const int64_t plane = stack.size(1) * stack.size(2);
  const int adt = any_dt(addend, plane, "addend");
  check(k8sllm_hy_depth_mix(stack.data_ptr<float>(), plane, (int)n, adt ? addend->data_ptr() : nullptr, adt,
                            coef.data_ptr<float>(), cur()),
        "depth_mix");
}

void activation(Tensor out, Tensor x, int64_t kind, double a, double b) {
  const int f = act(x, "x");
  same(out, f, "out");
  TORCH_CHECK(x.is_contiguous() && out.is_contiguous() && out.numel() == x.numel() && kind >= 0 && kind <= 3, "activation: shapes / kind");
  check(k8sllm_hy_activation(out.data_ptr(), x.data_ptr(), x.numel(), (int)kind, (float)a, (float)b, f, cur()), "activation");
}

void latent_prep(Tensor proj, int64_t Q, int64_t R, int64_t dr, Tensor qw, OptT kw, double eps, Tensor positions,
                 Tensor freq, OptT k_cache, OptT v_cache, OptT slots, bool pairs) {
  const int f = act(proj, "proj");
  f32c(qw, "dq.norm");
  f32c(freq, "freq");
  i32c(positions, "positions");
  const int64_t T = proj.size(0);
  const bool own = kw.has_value();
  TORCH_CHECK(proj.dim() == 2 && proj.stride(1) == 1 && proj.size(1) == (own ? Q + R + dr : Q), "proj [T, q_rank (+ kv_rank + rot)]");
  TORCH_CHECK(qw.numel() == Q && positions.numel() >= T && 2 * freq.numel() <= dr, "latent_prep: norm weight / positions / freq");
  void *kc = nullptr, *vc = nullptr;
  const int* sp = nullptr;
  const float* kwp = nullptr;
  int bs = 16, pitch = 0;
  if (own) {
    f32c(*kw, "dkv.norm");
    TORCH_CHECK(kw->numel() == R, "dkv.norm [kv_rank]");
    kwp = kw->data_ptr<float>();
    if (k_cache.has_value()) {
      TORCH_CHECK(v_cache.has_value() && slots.has_value(), "k_cache, v_cache and slot_mapping come together");
      TORCH_CHECK(k_cache->dim() == 3 && k_cache->size(2) >= R + dr, "k_cache rows hold [latent | rotated part]");
      pitch = (int)k_cache->size(2);
      pages(*k_cache, f, pitch, "k_cache");
      vpages(*v_cache, *k_cache, f, 1, R);
      sp = iptr(slots, "slot_mapping");
      TORCH_CHECK(slots->numel() >= T, "slot_mapping [T]");
      kc = k_cache->data_ptr();
      vc = v_cache->data_ptr();
      bs = (int)k_cache->size(1);
    }
  }
  check(k8sllm_hy_latent_prep(proj.data_ptr(), proj.stride(0), T, (int)Q, (int)R, (int)dr, qw.data_ptr<float>(), kwp,
                              (float)eps, positions.data_ptr<int>(), freq.data_ptr<float>(), (int)freq.numel(), pairs, kc, pitch,
                              vc, sp, bs, f, cur()),
        "latent_prep");
}

void latent_queries(Tensor out, Tensor q, Tensor q_lat, int64_t H, int64_t dn, int64_t dr, Tensor positions, Tensor freq,
                    bool pairs) {
  const int f = act(q, "q");
  same(out, f, "out");
  same(q_lat, f, "q_lat");
  f32c(freq, "freq");
  i32c(positions, "positions");
  const int64_t T = q.size(0);
  TORCH_CHECK(q.dim() == 2 && q.stride(1) == 1 && q.size(1) == H * (dn + dr), "q [T, H * (dim + rot)]");
  TORCH_CHECK(q_lat.dim() == 3 && q_lat.is_contiguous() && q_lat.size(0) == H && q_lat.size(1) == T, "q_lat [H, T, R]");
  const int64_t R = q_lat.size(2);
  TORCH_CHECK(out.dim() == 2 && out.is_contiguous() && out.size(0) == T && out.size(1) % H == 0 && out.size(1) / H >= R + dr &&
                  positions.numel() >= T && 2 * freq.numel() <= dr,
              "latent_queries: out [T, H * pitch] / positions / freq");
  check(k8sllm_hy_latent_queries(out.data_ptr(), q.data_ptr(), q.stride(0), q_lat.data_ptr(), T, (int)H, (int)dn, (int)dr,
                                 (int)R, (int)(out.size(1) / H), positions.data_ptr<int>(), freq.data_ptr<float>(), (int)freq.numel(),
                                 pairs, f, cur()),
        "latent_queries");
}

// The matrix-core latent attention; false: these sizes or dtype are not the kernel's, nothing was
// launched.  cu / ctx given: prompt chunks (block_tables per segment); else one row per sequence.
bool latent_attention(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache, OptT cu, OptT ctx, OptT seq_lens,
                      Tensor block_tables, int64_t H, double scale, int64_t window, OptT sinks, int64_t split) {
  if (act(q, "q") != 0) return false;
  same(out, 0, "out");
  TORCH_CHECK(k_cache.dim() == 3 && v_cache.dim() == 4, "pages");
  const int64_t dkp = k_cache.size(2), dv = v_cache.size(2), T = q.size(0);
  pages(k_cache, 0, dkp, "k_cache");
  vpages(v_cache, k_cache, 0, 1, dv);
  TORCH_CHECK(q.dim() == 2 && q.stride(1) == 1 && q.size(1) == H * dkp, "q [T, H * key pitch]");
  TORCH_CHECK(out.is_contiguous() && out.numel() == T * H * dv, "out [T, H * dv]");
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == torch::kInt32 && block_tables.dim() == 2 &&
                  block_tables.stride(1) == 1,
              "block_tables [S, W] int32");
  const int *cup = nullptr, *ctxp = nullptr, *slp = nullptr;
  int64_t S = 0;
  if (cu.has_value()) {
    TORCH_CHECK(ctx.has_value(), "cu and ctx come together");
    cup = iptr(cu, "cu");
    ctxp = iptr(ctx, "ctx");
    S = ctx->numel();
    TORCH_CHECK(cu->numel() == S + 1 && block_tables.size(0) >= S, "cu [S+1], block_tables [S, W]");
  } else {
    slp = iptr(seq_lens, "seq_lens");
    TORCH_CHECK(slp != nullptr && seq_lens->numel() >= T && block_tables.size(0) >= T, "seq_lens [T], block_tables [T, W]");
  }
  TORCH_CHECK(window >= 0 && H >= 1, "heads / window");
  const int rc = k8sllm_hy_latent_attention(out.data_ptr(), q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
                                            cup, ctxp, slp, block_tables.data_ptr<int>(), (int)block_tables.stride(0), (int)S, T,
                                            (int)H, (int)dkp, (int)dv, (int)k_cache.size(1), (float)scale, (int)window,
                                            sink_ptr(sinks, H), (int)split, cur());
  if (rc == 1) return false;
  check(rc, "latent_attention");
  return true;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_pos", &embed_pos);
  m.def("add_norm", &add_norm);
  m.def("gated_group_norm", &gated_group_norm);
  m.def("swiglu", &swiglu);
  m.def("gated_add_norm", &gated_add_norm);
  m.def("glu", &glu);
  m.def("activation_cols", &activation_cols);
  m.def("sigmoid_gate", &sigmoid_gate);
  m.def("softcap", &softcap);
  m.def("rotary_cache", &rotary_cache);
  m.def("linear_attention_chunked", &linear_attention_chunked);
  m.def("qk_norm_cache", &qk_norm_cache);
  m.def("window_attention_prefill", &window_attention_prefill);
  m.def("window_attention_decode", &window_attention_decode);
  m.def("conv_silu", &conv_silu);
  m.def("ssm_scan", &ssm_scan);
  m.def("moe_router", &moe_router);
  m.def("moe_align", &moe_align);
  m.def("grouped_gemm", &grouped_gemm);
  m.def("moe_combine", &moe_combine);
  m.def("norm_shift", &norm_shift);
  m.def("depth_mix", &depth_mix);
  m.def("activation", &activation);
  m.def("latent_prep", &latent_prep);
  m.def("latent_queries", &latent_queries);
  m.def("latent_attention", &latent_attention);
  m.def("sum_norm", &sum_norm);
  m.def("gated_lookup", &gated_lookup);
  m.def("rotary_norm_cache", &rotary_norm_cache);
  m.def("decay_scan", &decay_scan);
  m.def("moe_router_grouped", &moe_router_grouped);
}
