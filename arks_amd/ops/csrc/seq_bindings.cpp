// Python bindings of the sequence-state kernels (arks_amd_seq_C). Shapes,
// dtypes and strides are validated here; the kernels are in seq_*.hip.
#include <torch/extension.h>

#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

#include "attn_bindings.h"

extern "C" {
void arks_seq_token_shift(void* xs, void* xa, const void* x, const void* w,
                          void* state, const void* cu, const void* seq_lens,
                          const void* slots, const void* token_seq, int T,
                          int W, int act_f32, hipStream_t stream);
void arks_seq_gated_norm_residual(void* x, void* xa, const void* y,
                                  const void* g, int64_t ldg, const void* gb,
                                  const void* w, float eps, int T, int W,
                                  int act_f32, hipStream_t stream);
void arks_seq_rms_norm_f32(void* out, const void* x, const void* w,
                           const void* gate, int64_t ldg, float eps, int T,
                           int W, int act_f32, hipStream_t stream);
void arks_seq_gelu_tanh(void* out, const void* x, int64_t ldx, int64_t rows,
                        int n, int act_f32, hipStream_t stream);
int arks_seq_qk_norm_rope_cache(
    void* qo, const void* q, const void* k, const void* v, int64_t ldq,
    int64_t ldk, int64_t ldv, const void* qw, const void* kw, float eps,
    const void* positions, const void* freq_qk, int n_rot, const void* freq_v,
    int n_vrot, void* k_cache, void* v_cache, const void* slot_mapping, int T,
    int H, int G, int D, int V, int block_size, int interleaved, int act_f32,
    float rot_mag, int norm_after, hipStream_t stream);
int arks_seq_unrotate_rows(void* out, const void* positions, const void* freq,
                            int T, int H, int V, int interleaved, int act_f32,
                            hipStream_t stream);
int arks_seq_attn_sink_generic(
    void* out, const void* q, const void* k_cache, const void* v_cache,
    const void* block_tables, const void* seq_lens, const void* cu,
    const void* token_seq, float scale, int sink, const void* freq_v,
    int interleaved, int T, int H, int G, int D, int V, int block_size,
    int max_blocks, int act_f32, const void* sink_w, float softcap,
    int window, int keep_first, int64_t ldk, int64_t ldv, int64_t ldo,
    float out_scale, int maps, hipStream_t stream);
int arks_seq_lightning_scan(void* out, const void* q, const void* k,
                            const void* v, int64_t ldq, int64_t ldk,
                            int64_t ldv, const void* decay, void* state,
                            const void* cu, const void* seq_lens,
                            const void* slots, int S, int H, int D, int V,
                            int act_f32, int mode, const void* positions,
                            const void* freq, int n_rot, int interleaved,
                            float k_scale, hipStream_t stream);
int arks_seq_causal_conv_silu(void* out, const void* x, int64_t ldx,
                              const void* w, const void* w_t, const void* bias,
                              void* state,
                              const void* cu, const void* seq_lens,
                              const void* slots, const void* token_seq, int T,
                              int S, int C, int taps, int act_f32,
                              hipStream_t stream);
int arks_seq_selective_scan(void* out, const void* u, const void* dbc,
                            int64_t ldd, const void* z, int64_t ldz,
                            const void* dt_w, const void* dt_b, const void* A,
                            const void* Dp, void* state, const void* cu,
                            const void* seq_lens, const void* slots, int S,
                            int C, int N, int R, const void* dt_pre,
                            void* dsum, int act_f32, hipStream_t stream);
void arks_seq_scan_combine(void* part, const void* dsum, const void* A,
                           void* state, const void* chunk_off, const void* cu,
                           const void* seq_lens, const void* slots, int S,
                           int C, int N, hipStream_t stream);
int arks_seq_lightning_mfma(void* out, void* part, const void* q, const void* k,
                            const void* v, int64_t ldq, int64_t ldk,
                            int64_t ldv, const void* decay, const void* cu,
                            int chunks, int H, int D, int V, int pass,
                            int mode, const void* positions, const void* freq,
                            int n_rot, int interleaved, float k_scale,
                            hipStream_t stream);
int arks_seq_stream_mix_norm(void* xs, void* n_out, const void* y, int64_t ldy,
                             const void* y_bias, const void* mix,
                             const void* out_w, const void* in_w,
                             const void* norm_w, const void* norm_b, float eps,
                             int S, int64_t T, int C, int act_f32,
                             hipStream_t stream);
int arks_seq_short_conv_residual(void* out, const void* h, const void* w,
                                 void* state, const void* cu,
                                 const void* seq_lens, const void* slots,
                                 const void* token_seq, int T, int S, int C,
                                 int taps, int act_f32, hipStream_t stream);
void arks_seq_head_norm_gate(void* out, int64_t ldo, const void* o,
                             const void* gate, int64_t ldg, float eps, int T,
                             int H, int V, float out_scale, int act_f32,
                             hipStream_t stream);
void arks_seq_glu_act(void* out, int64_t ldo, const void* gu, int64_t ldg,
                      int64_t rows, int F, int mode, float limit, float alpha,
                      const void* row_scale, int act_f32, hipStream_t stream);
void arks_seq_kv_write_pooled(const void* k, const void* v, int64_t ldk,
                              int64_t ldv, void* k_cache, void* v_cache,
                              void* kp_cache, void* vp_cache,
                              const void* slot_mapping, const void* positions,
                              const void* block_tables, const void* token_seq,
                              int T, int max_blocks, int G, int D, int V,
                              int bs, int pool, int spp, int act_f32,
                              hipStream_t stream);
int arks_seq_attn_window_pool(void* out, int64_t ldo, const void* q,
                              int64_t ldq, const void* k_cache,
                              const void* v_cache, const void* kp_cache,
                              const void* vp_cache, const void* block_tables,
                              const void* seq_lens, const void* cu,
                              const void* token_seq, float scale, int window,
                              int pool, int spp, float out_scale, int T, int H,
                              int G, int D, int V, int bs, int max_blocks,
                              int act_f32, hipStream_t stream);
int arks_seq_attn_window_pool_mfma(void* out, int64_t ldo, const void* q,
                                   int64_t ldq, const void* k_cache,
                                   const void* v_cache, const void* kp_cache,
                                   const void* vp_cache,
                                   const void* block_tables,
                                   const void* seq_lens, const void* cu,
                                   const void* token_seq, float scale,
                                   int window, int pool, int spp,
                                   float out_scale, int T, int H, int G, int D,
                                   int V, int bs, int max_blocks,
                                   int num_seqs, int single_rows,
                                   hipStream_t stream);
void arks_seq_residual_tanh_norm(void* x, void* h, void* xa, int64_t ldxa,
                                 const void* y, float mult, const void* alpha,
                                 const void* w, const void* b, int64_t T, int C,
                                 int act_f32, hipStream_t stream);
void arks_seq_latent_prepare(void* cqn, const void* cq, int64_t ldq,
                             const void* ckv, int64_t ldk, const void* qw,
                             const void* kw, float eps, const void* positions,
                             const void* freq, void* cache,
                             const void* slot_mapping, int T, int Rq, int Rk,
                             int P, int act_f32, hipStream_t stream);
void arks_seq_latent_query(void* out, const void* q, const void* q_abs,
                           const void* positions, const void* freq, int T,
                           int H, int D, int Rk, int P, int act_f32,
                           hipStream_t stream);
int arks_seq_mamba2_scan(void* out, const void* xbc, int64_t ldx,
                         const void* dt_raw, int64_t ldd, const void* dt_bias,
                         const void* rate, const void* Dp, void* state,
                         const void* cu, const void* seq_lens,
                         const void* slots, void* dsum, int S, int P, int V,
                         int N, int G, int act_f32, hipStream_t stream);
void arks_seq_mamba2_combine(void* part, const void* dsum, const void* rate,
                             void* state, const void* chunk_off,
                             const void* cu, const void* seq_lens,
                             const void* slots, int S, int P, int NV,
                             hipStream_t stream);
void arks_seq_gate_group_norm(void* out, int64_t ldo, const void* y,
                              const void* z, int64_t ldz, const void* w,
                              float eps, int T, int C, int groups,
                              float out_scale, int act_f32,
                              hipStream_t stream);
int arks_seq_attn_masked_mfma(void* out, int64_t ldo, const void* q,
                              const void* k_cache, int64_t ldk,
                              const void* v_cache, int64_t ldv,
                              const void* block_tables, const void* seq_lens,
                              const void* cu, const void* token_seq,
                              float scale, const void* sink_w, float softcap,
                              int window, int keep_first, float out_scale,
                              int T, int H, int G, int D, int V, int bs,
                              int max_blocks, int num_seqs, int single_rows,
                              void* ws, int ksplit, int maps,
                              hipStream_t stream);
int arks_seq_attn_masked_ksplit(int T, int H, int G, int max_blocks);
int arks_seq_moe_route_grouped(void* weights, void* ids, const void* logits,
                               int T, int E, int top, int groups, int keep,
                               int sigmoid, int renorm, void* matrix,
                               hipStream_t stream);
void arks_seq_moe_mix_rows(void* out, const void* y, const void* weights,
                           const void* rows, int T, int H, int k, int dense,
                           const void* add, int act_f32, hipStream_t stream);
void arks_seq_residual_pair_norm(void* x, void* h1, void* h2, const void* y1,
                                 const void* s1, const void* y2,
                                 const void* s2, const void* w1,
                                 const void* w2, float eps, int64_t T, int C,
                                 int act_f32, hipStream_t stream);
int arks_seq_conv_qkv_cache(void* qo, const void* p, int64_t ldp,
                            const void* w, const void* w_t, void* state,
                            const void* cu, const void* seq_lens,
                            const void* slots, const void* token_seq,
                            const void* positions, void* k_cache,
                            void* v_cache, const void* slot_mapping, int T,
                            int S, int n_q, int n_k, int n_v, int heads,
                            int kv_heads, int maps, int block_size, int taps,
                            float temp_coef, int temp_every, int act_f32,
                            hipStream_t stream);
int arks_seq_diff_head_norm_gate(void* out, int64_t ldo, const void* a,
                                 const void* gate, int64_t ldg, float lam,
                                 float eps, float mult, int T, int H, int G,
                                 int V, int act_f32, hipStream_t stream);
void arks_seq_moe_glu_scaled(void* out, const void* gu, int64_t ldg,
                             const void* scale, int64_t T, int E, int ff,
                             int sff, int act_f32, hipStream_t stream);
void arks_seq_lightning_combine(void* part, const void* decay, void* state,
                                const void* chunk_off, const void* chunk_rows,
                                const void* cu, const void* seq_lens,
                                const void* slots, int S, int H, int D, int V,
                                int transposed, hipStream_t stream);
}

namespace {

using torch::Tensor;
using OptTensor = c10::optional<Tensor>;

hipStream_t current_stream() {
  return c10::hip::getCurrentHIPStream().stream();
}

int act_flag(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be on the GPU");
  TORCH_CHECK(t.scalar_type() == torch::kBFloat16 ||
                  t.scalar_type() == torch::kFloat32,
              name, " must be bfloat16 or float32");
  return t.scalar_type() == torch::kFloat32 ? 1 : 0;
}

void check_f32(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kFloat32 &&
                  t.is_contiguous(),
              name, " must be a contiguous float32 GPU tensor");
}

void check_i32(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kInt32 &&
                  t.is_contiguous(),
              name, " must be a contiguous int32 GPU tensor");
}

void check_i64(const Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kInt64 &&
                  t.is_contiguous(),
              name, " must be a contiguous int64 GPU tensor");
}

// rows x cols view whose last dim is dense; returns the row stride
int64_t row_stride(const Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 2 && t.stride(1) == 1, name,
              " must be 2-D with a dense last dim");
  return t.stride(0);
}

// [T, heads, dim] view of a wider row: heads dense
int64_t head_row_stride(const Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 3 && t.stride(2) == 1 && t.stride(1) == t.size(2),
              name, " must be [T, heads, dim] with dense heads");
  return t.stride(0);
}

// [pages, G, bs, dim] cache, or a view of the leading columns of one:
// token rows a fixed stride apart through heads and pages; returns it
int64_t paged_row_stride(const Tensor& t, const char* name) {
  TORCH_CHECK(t.dim() == 4 && t.stride(3) == 1 &&
                  t.stride(1) == t.size(2) * t.stride(2) &&
                  t.stride(0) == t.size(1) * t.stride(1) &&
                  t.stride(2) >= t.size(3),
              name, " must be [pages, heads, tokens, dim] rows of one stride");
  return t.stride(2);
}

struct SeqMeta {
  int S;
};

SeqMeta check_meta(const Tensor& cu, const Tensor& seq_lens,
                   const Tensor* slots, const Tensor* token_seq, int64_t T) {
  check_i32(cu, "cu_seqlens");
  check_i32(seq_lens, "seq_lens");
  const int64_t S = seq_lens.numel();
  TORCH_CHECK(cu.numel() == S + 1, "cu_seqlens must have num_seqs + 1 entries");
  if (slots) {
    check_i32(*slots, "state_slots");
    TORCH_CHECK(slots->numel() == S, "state_slots must have num_seqs entries");
  }
  if (token_seq) {
    check_i32(*token_seq, "token_seq");
    TORCH_CHECK(token_seq->numel() == T, "token_seq must have one entry per row");
  }
  return {(int)S};
}

void token_shift(Tensor xs, Tensor xa, Tensor x, Tensor w, Tensor state,
                 Tensor cu, Tensor seq_lens, Tensor slots, Tensor token_seq) {
  check_f32(x, "x");
  check_f32(w, "shift weight");
  check_f32(state, "shift state");
  const int T = x.size(0), W = x.size(1);
  const int f32 = act_flag(xs, "xs");
  TORCH_CHECK(xs.is_contiguous() && xs.sizes() == x.sizes());
  TORCH_CHECK(w.numel() == W && state.dim() == 2 && state.size(1) == W);
  check_meta(cu, seq_lens, &slots, &token_seq, T);
  void* xa_p = nullptr;
  if (!f32) {
    TORCH_CHECK(xa.scalar_type() == xs.scalar_type() && xa.is_contiguous() &&
                xa.sizes() == x.sizes());
    xa_p = xa.data_ptr();
  }
  arks_seq_token_shift(xs.data_ptr(), xa_p, x.data_ptr(), w.data_ptr(),
                       state.data_ptr(), cu.data_ptr(), seq_lens.data_ptr(),
                       slots.data_ptr(), token_seq.data_ptr(), T, W, f32,
                       current_stream());
}

void gated_norm_residual(Tensor x, OptTensor xa, Tensor y, OptTensor gate,
                         OptTensor gate_bias, Tensor w, double eps) {
  check_f32(x, "x");
  check_f32(w, "norm weight");
  const int T = x.size(0), W = x.size(1);
  const int f32 = act_flag(y, "y");
  TORCH_CHECK(y.is_contiguous() && y.dim() == 2 && y.size(0) == T &&
              y.size(1) == W, "y must be contiguous [T, W]");
  TORCH_CHECK(w.numel() == W);
  const void* g_p = nullptr;
  const void* gb_p = nullptr;
  int64_t ldg = 0;
  if (gate.has_value()) {
    TORCH_CHECK(gate->scalar_type() == y.scalar_type() && gate->size(0) == T &&
                gate->size(1) == W);
    ldg = row_stride(*gate, "gate");
    TORCH_CHECK(gate_bias.has_value());
    check_f32(*gate_bias, "gate bias");
    TORCH_CHECK(gate_bias->numel() == W);
    g_p = gate->data_ptr();
    gb_p = gate_bias->data_ptr();
  }
  void* xa_p = nullptr;
  if (xa.has_value()) {
    TORCH_CHECK(xa->scalar_type() == y.scalar_type() && xa->is_contiguous() &&
                xa->sizes() == x.sizes());
    xa_p = xa->data_ptr();
  }
  arks_seq_gated_norm_residual(x.data_ptr(), xa_p, y.data_ptr(), g_p, ldg, gb_p,
                               w.data_ptr(), (float)eps, T, W, f32,
                               current_stream());
}

void rms_norm_f32(Tensor out, Tensor x, Tensor w, double eps) {
  check_f32(x, "x");
  check_f32(w, "norm weight");
  const int f32 = act_flag(out, "out");
  TORCH_CHECK(out.is_contiguous() && out.sizes() == x.sizes() && x.dim() == 2);
  TORCH_CHECK(w.numel() == x.size(1));
  arks_seq_rms_norm_f32(out.data_ptr(), x.data_ptr(), w.data_ptr(), nullptr, 0,
                        (float)eps, x.size(0), x.size(1), f32, current_stream());
}

void gated_rmsnorm(Tensor out, Tensor o, Tensor w, Tensor gate, double eps) {
  check_f32(o, "o");
  check_f32(w, "norm weight");
  const int f32 = act_flag(out, "out");
  TORCH_CHECK(out.is_contiguous() && out.sizes() == o.sizes() && o.dim() == 2);
  TORCH_CHECK(gate.scalar_type() == out.scalar_type() &&
              gate.size(0) == o.size(0) && gate.size(1) == o.size(1));
  TORCH_CHECK(w.numel() == o.size(1));
  arks_seq_rms_norm_f32(out.data_ptr(), o.data_ptr(), w.data_ptr(),
                        gate.data_ptr(), row_stride(gate, "gate"), (float)eps,
                        o.size(0), o.size(1), f32, current_stream());
}

void gelu_tanh(Tensor out, Tensor x) {
  const int f32 = act_flag(x, "x");
  TORCH_CHECK(out.scalar_type() == x.scalar_type() && out.is_contiguous() &&
              out.sizes() == x.sizes());
  arks_seq_gelu_tanh(out.data_ptr(), x.data_ptr(), row_stride(x, "x"),
                     x.size(0), x.size(1), f32, current_stream());
}

void qk_norm_rope_cache(Tensor qo, Tensor q, Tensor k, Tensor v, OptTensor qw,
                        OptTensor kw, double eps, Tensor positions,
                        Tensor freq_qk, OptTensor freq_v, Tensor k_cache,
                        Tensor v_cache, Tensor slot_mapping, bool interleaved,
                        double rot_mag, bool norm_after) {
  const int f32 = act_flag(q, "q");
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  const int G = k.size(1), V = v.size(2);
  TORCH_CHECK(k.scalar_type() == q.scalar_type() &&
              v.scalar_type() == q.scalar_type() &&
              qo.scalar_type() == q.scalar_type() &&
              k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type(),
              "q, k, v and the cache must share one dtype");
  TORCH_CHECK(k.size(0) == T && v.size(0) == T && k.size(2) == D &&
              v.size(1) == G);
  TORCH_CHECK(qo.is_contiguous() && qo.sizes() == q.sizes());
  TORCH_CHECK(k_cache.is_contiguous() && v_cache.is_contiguous() &&
              k_cache.dim() == 4 && v_cache.dim() == 4);
  TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == D &&
              v_cache.size(1) == G && v_cache.size(3) == V &&
              v_cache.size(2) == k_cache.size(2) &&
              v_cache.size(0) == k_cache.size(0), "cache shape mismatch");
  check_i64(positions, "positions");
  check_i64(slot_mapping, "slot_mapping");
  TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
  check_f32(freq_qk, "inv_freq_qk");
  const int n_rot = freq_qk.numel();
  TORCH_CHECK(2 * n_rot <= D, "rotary dims exceed the head size");
  const void* qw_p = nullptr;
  const void* kw_p = nullptr;
  if (qw.has_value()) {
    check_f32(*qw, "q norm weight");
    TORCH_CHECK(kw.has_value());
    check_f32(*kw, "k norm weight");
    TORCH_CHECK(qw->numel() == D && kw->numel() == D);
    qw_p = qw->data_ptr();
    kw_p = kw->data_ptr();
  }
  const void* fv_p = nullptr;
  int n_vrot = 0;
  if (freq_v.has_value()) {
    check_f32(*freq_v, "inv_freq_v");
    n_vrot = freq_v->numel();
    TORCH_CHECK(2 * n_vrot == V, "value rotation covers all value dims");
    fv_p = freq_v->data_ptr();
  }
  const int rc = arks_seq_qk_norm_rope_cache(
      qo.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
      head_row_stride(q, "q"), head_row_stride(k, "k"), head_row_stride(v, "v"),
      qw_p, kw_p, (float)eps, positions.data_ptr(), freq_qk.data_ptr(), n_rot,
      fv_p, n_vrot, k_cache.data_ptr(), v_cache.data_ptr(),
      slot_mapping.data_ptr(), T, H, G, D, V, (int)k_cache.size(2),
      interleaved ? 1 : 0, f32, (float)rot_mag, norm_after ? 1 : 0,
      current_stream());
  TORCH_CHECK(rc == 0, "more rotary pairs than the kernel's table holds");
}

void attention_sink_paged(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                          Tensor block_tables, Tensor seq_lens, Tensor cu,
                          Tensor token_seq, double scale, bool sink,
                          OptTensor freq_v, bool interleaved,
                          int64_t max_q_len, OptTensor sink_w, double softcap,
                          int64_t window, int64_t keep_first,
                          double out_scale, int64_t maps) {
  const int f32 = act_flag(q, "q");
  TORCH_CHECK(q.is_contiguous() && q.dim() == 3 && maps >= 1);
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  TORCH_CHECK(k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type() &&
              out.scalar_type() == q.scalar_type());
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.size(3) == D * maps);
  const int G = k_cache.size(1), bs = k_cache.size(2), V = v_cache.size(3);
  TORCH_CHECK(H % (G * maps) == 0 && v_cache.size(1) == G &&
              v_cache.size(2) == bs);
  TORCH_CHECK(maps == 1 || (!sink_w.has_value() && !freq_v.has_value()),
              "several key maps: no per-head sink, no turned values");
  const int64_t ldk = paged_row_stride(k_cache, "k_cache");
  const int64_t ldv = paged_row_stride(v_cache, "v_cache");
  const int64_t ldo = head_row_stride(out, "out");
  TORCH_CHECK(out.size(0) == T && out.size(1) == H && out.size(2) == V);
  const void* sw_p = nullptr;
  if (sink_w.has_value()) {
    check_f32(*sink_w, "sink_w");
    TORCH_CHECK(sink_w->numel() == H);
    sw_p = sink_w->data_ptr();
  }
  TORCH_CHECK(window >= 0 && keep_first >= 0 && softcap >= 0);
  check_i32(block_tables, "block_tables");
  TORCH_CHECK(block_tables.dim() == 2 &&
              block_tables.size(0) == seq_lens.numel());
  check_meta(cu, seq_lens, nullptr, &token_seq, T);
  const void* fv_p = nullptr;
  if (freq_v.has_value()) {
    check_f32(*freq_v, "inv_freq_v");
    TORCH_CHECK(2 * freq_v->numel() == V);
    fv_p = freq_v->data_ptr();
  }
  const int rc = arks_seq_attn_sink_generic(
      out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
      block_tables.data_ptr(), seq_lens.data_ptr(), cu.data_ptr(),
      token_seq.data_ptr(), (float)scale, sink ? 1 : 0, fv_p,
      interleaved ? 1 : 0, T, H, G, D, V, bs, (int)block_tables.size(1), f32,
      sw_p, (float)softcap, (int)window, (int)keep_first, ldk, ldv, ldo,
      (float)out_scale, (int)maps, current_stream());
  TORCH_CHECK(rc == 0, "attention head sizes beyond the kernel's limits (",
              D, ", ", V, ")");
}

void unrotate_rows(Tensor out, Tensor positions, Tensor freq_v,
                   bool interleaved) {
  const int f32 = act_flag(out, "out");
  TORCH_CHECK(out.is_contiguous() && out.dim() == 3);
  check_i64(positions, "positions");
  check_f32(freq_v, "inv_freq_v");
  TORCH_CHECK(positions.numel() == out.size(0) &&
              2 * freq_v.numel() == out.size(2));
  const int rc = arks_seq_unrotate_rows(
      out.data_ptr(), positions.data_ptr(), freq_v.data_ptr(), out.size(0),
      out.size(1), out.size(2), interleaved ? 1 : 0, f32, current_stream());
  TORCH_CHECK(rc == 0, "more rotary pairs than the kernel's table holds");
}

// Input convention of the lightning kernels: without positions, rows pass
// through silu (mode 0); with positions, plain rows whose q and k are turned
// over their first 2 * freq.numel() dims (mode 1; freq may be absent).
struct RotArgs {
  int mode, n_rot;
  const void* positions;
  const void* freq;
};

RotArgs rot_args(const OptTensor& positions, const OptTensor& freq, int64_t T,
                 int64_t D) {
  RotArgs r{0, 0, nullptr, nullptr};
  if (!positions.has_value()) return r;
  check_i64(*positions, "positions");
  TORCH_CHECK(positions->numel() == T, "one position per row");
  r.mode = 1;
  r.positions = positions->data_ptr();
  if (freq.has_value() && freq->numel() > 0) {
    check_f32(*freq, "rotary frequencies");
    TORCH_CHECK(2 * freq->numel() <= D, "more rotary dims than the head has");
    r.n_rot = (int)freq->numel();
    r.freq = freq->data_ptr();
  }
  return r;
}

void lightning_scan(Tensor out, Tensor q, Tensor k, Tensor v, Tensor decay,
                    Tensor state, Tensor cu, Tensor seq_lens, Tensor slots,
                    int64_t max_q_len, OptTensor positions, OptTensor freq,
                    bool interleaved, double k_scale) {
  const int f32 = act_flag(q, "q");
  const RotArgs rot = rot_args(positions, freq, q.size(0), q.size(2));
  const int T = q.size(0), H = q.size(1), D = q.size(2), V = v.size(2);
  TORCH_CHECK(k.scalar_type() == q.scalar_type() &&
              v.scalar_type() == q.scalar_type());
  TORCH_CHECK(k.size(0) == T && k.size(1) == H && k.size(2) == D &&
              v.size(0) == T && v.size(1) == H);
  check_f32(out, "out");
  TORCH_CHECK(out.size(0) == T && out.size(1) == H && out.size(2) == V);
  check_f32(decay, "decay");
  TORCH_CHECK(decay.numel() == H);
  check_f32(state, "state");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D &&
              state.size(3) == V, "state must be [slots, H, D, V]");
  const SeqMeta m = check_meta(cu, seq_lens, &slots, nullptr, T);
  const int rc = arks_seq_lightning_scan(
      out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
      head_row_stride(q, "q"), head_row_stride(k, "k"), head_row_stride(v, "v"),
      decay.data_ptr(), state.data_ptr(), cu.data_ptr(), seq_lens.data_ptr(),
      slots.data_ptr(), m.S, H, D, V, f32, rot.mode, rot.positions, rot.freq,
      rot.n_rot, interleaved ? 1 : 0, (float)k_scale, current_stream());
  TORCH_CHECK(rc == 0, "lightning head size beyond the kernel's limit (", D, ")");
}

void causal_conv_silu(Tensor out, Tensor x, Tensor w, OptTensor w_t,
                      Tensor bias, OptTensor state, Tensor cu, Tensor seq_lens,
                      Tensor slots, Tensor token_seq) {
  const int f32 = act_flag(x, "x");
  const int T = x.size(0), C = x.size(1);
  TORCH_CHECK(out.scalar_type() == x.scalar_type() && out.is_contiguous() &&
              out.sizes() == x.sizes());
  check_f32(w, "conv weight");
  check_f32(bias, "conv bias");
  TORCH_CHECK(w.dim() == 2 && w.size(0) == C && bias.numel() == C);
  const int taps = w.size(1);
  const void* wt_p = nullptr;
  if (w_t.has_value()) {  // [taps, C] copy for the vectorised kernel
    check_f32(*w_t, "transposed conv weight");
    TORCH_CHECK(w_t->dim() == 2 && w_t->size(0) == taps && w_t->size(1) == C);
    wt_p = w_t->data_ptr();
  }
  void* st_p = nullptr;
  if (taps > 1) {
    TORCH_CHECK(state.has_value());
    check_f32(*state, "conv state");
    TORCH_CHECK(state->dim() == 3 && state->size(1) == taps - 1 &&
                state->size(2) == C, "conv state must be [slots, taps-1, C]");
    st_p = state->data_ptr();
  }
  const SeqMeta m = check_meta(cu, seq_lens, &slots, &token_seq, T);
  const int rc = arks_seq_causal_conv_silu(
      out.data_ptr(), x.data_ptr(), row_stride(x, "x"), w.data_ptr(), wt_p,
      bias.data_ptr(), st_p, cu.data_ptr(), seq_lens.data_ptr(),
      slots.data_ptr(), token_seq.data_ptr(), T, m.S, C, taps, f32,
      current_stream());
  TORCH_CHECK(rc == 0, "conv taps beyond the kernel's limit (", taps, ")");
}

void selective_scan(OptTensor out_, Tensor u, Tensor dbc, Tensor z, Tensor dt_w,
                    Tensor dt_b, Tensor A, Tensor Dp, Tensor state, Tensor cu,
                    Tensor seq_lens, Tensor slots, OptTensor dt_pre,
                    OptTensor dsum) {
  const int f32 = act_flag(u, "u");
  const int T = u.size(0), C = u.size(1);
  TORCH_CHECK(u.is_contiguous());
  void* out_p = nullptr;  // none: state-only pass (needs dt_pre, N <= 64)
  if (out_.has_value()) {
    const Tensor& out = *out_;
    TORCH_CHECK(out.is_contiguous() && out.scalar_type() == u.scalar_type() &&
                out.sizes() == u.sizes());
    out_p = out.data_ptr();
  } else {
    TORCH_CHECK(dt_pre.has_value() && A.size(1) <= 64,
                "a state-only scan needs dt_pre and a state size <= 64");
  }
  TORCH_CHECK(dbc.scalar_type() == u.scalar_type() &&
              z.scalar_type() == u.scalar_type());
  check_f32(dt_w, "dt weight");
  check_f32(dt_b, "dt bias");
  check_f32(A, "A");
  check_f32(Dp, "D");
  check_f32(state, "ssm state");
  const int R = dt_w.size(1), N = A.size(1);
  TORCH_CHECK(dt_w.size(0) == C && dt_b.numel() == C && A.size(0) == C &&
              Dp.numel() == C);
  TORCH_CHECK(dbc.size(0) == T && dbc.size(1) == R + 2 * N,
              "dbc must be [T, dt_rank + 2 * state]");
  TORCH_CHECK(z.size(0) == T && z.size(1) == C);
  TORCH_CHECK(state.dim() == 3 && state.size(1) == C && state.size(2) == N,
              "ssm state must be [slots, C, N]");
  const SeqMeta m = check_meta(cu, seq_lens, &slots, nullptr, T);
  const void* dtp_p = nullptr;
  void* dsum_p = nullptr;
  if (dt_pre.has_value()) {
    check_f32(*dt_pre, "dt_pre");
    TORCH_CHECK(dt_pre->dim() == 2 && dt_pre->size(0) == T &&
                dt_pre->size(1) == C, "dt_pre must be [T, C]");
    dtp_p = dt_pre->data_ptr();
  }
  if (dsum.has_value()) {
    check_f32(*dsum, "dsum");
    TORCH_CHECK(dsum->numel() == (int64_t)m.S * C, "dsum must be [S, C]");
    dsum_p = dsum->data_ptr();
  }
  const int rc = arks_seq_selective_scan(
      out_p, u.data_ptr(), dbc.data_ptr(), row_stride(dbc, "dbc"),
      z.data_ptr(), row_stride(z, "z"), dt_w.data_ptr(), dt_b.data_ptr(),
      A.data_ptr(), Dp.data_ptr(), state.data_ptr(), cu.data_ptr(),
      seq_lens.data_ptr(), slots.data_ptr(), m.S, C, N, R, dtp_p, dsum_p, f32,
      current_stream());
  TORCH_CHECK(rc == 0, "ssm state size beyond the kernel's limit (", N, ")");
}

// part [chunks, C, N], dsum [chunks, C]; chunk_off [S + 1] = each real
// sequence's range of chunks
void scan_combine(Tensor part, Tensor dsum, Tensor A, Tensor state,
                  Tensor chunk_off, Tensor cu, Tensor seq_lens, Tensor slots) {
  check_f32(part, "part");
  check_f32(dsum, "dsum");
  check_f32(A, "A");
  check_f32(state, "ssm state");
  const int C = A.size(0), N = A.size(1);
  TORCH_CHECK(part.dim() == 3 && part.size(1) == C && part.size(2) == N &&
              dsum.dim() == 2 && dsum.size(0) == part.size(0) &&
              dsum.size(1) == C && state.size(1) == C && state.size(2) == N);
  const SeqMeta m = check_meta(cu, seq_lens, &slots, nullptr, 0);
  check_i32(chunk_off, "chunk_off");
  TORCH_CHECK(chunk_off.numel() == m.S + 1);
  arks_seq_scan_combine(part.data_ptr(), dsum.data_ptr(), A.data_ptr(),
                        state.data_ptr(), chunk_off.data_ptr(), cu.data_ptr(),
                        seq_lens.data_ptr(), slots.data_ptr(), m.S, C, N,
                        current_stream());
}

// One pass of the matrix-core lightning prefill over chunks of <= 64 rows
// (cu = chunk row starts). pass 1 fills part with chunk end states, pass 2
// reads chunk start states from part and writes out. False: no kernel for
// these head sizes (the caller runs the general kernel).
bool lightning_mfma(Tensor out, Tensor part, Tensor q, Tensor k, Tensor v,
                    Tensor decay, Tensor cu, int64_t pass, OptTensor positions,
                    OptTensor freq, bool interleaved, double k_scale) {
  const RotArgs rot = rot_args(positions, freq, q.size(0), q.size(2));
  TORCH_CHECK(q.is_cuda() && q.scalar_type() == torch::kBFloat16 &&
              k.scalar_type() == torch::kBFloat16 &&
              v.scalar_type() == torch::kBFloat16, "bf16 rows only");
  const int T = q.size(0), H = q.size(1), D = q.size(2), V = v.size(2);
  TORCH_CHECK(k.size(0) == T && k.size(1) == H && k.size(2) == D &&
              v.size(0) == T && v.size(1) == H);
  check_f32(out, "out");
  check_f32(part, "part");
  check_f32(decay, "decay");
  check_i32(cu, "chunk starts");
  const int chunks = cu.numel() - 1;
  TORCH_CHECK(out.size(0) == T && out.size(1) == H && out.size(2) == V);
  TORCH_CHECK(part.dim() == 4 && part.size(0) == chunks && part.size(1) == H &&
              part.size(2) == D && part.size(3) == V && decay.numel() == H);
  TORCH_CHECK(pass == 1 || pass == 2);
  return arks_seq_lightning_mfma(
             out.data_ptr(), part.data_ptr(), q.data_ptr(), k.data_ptr(),
             v.data_ptr(), head_row_stride(q, "q"), head_row_stride(k, "k"),
             head_row_stride(v, "v"), decay.data_ptr(), cu.data_ptr(), chunks,
             H, D, V, (int)pass, rot.mode, rot.positions, rot.freq, rot.n_rot,
             interleaved ? 1 : 0, (float)k_scale, current_stream()) == 0;
}

void lightning_combine(Tensor part, Tensor decay, Tensor state,
                       Tensor chunk_off, Tensor chunk_rows, Tensor cu,
                       Tensor seq_lens, Tensor slots, bool transposed) {
  check_f32(part, "part");
  check_f32(decay, "decay");
  check_f32(state, "state");
  // part: [chunks, H, D, V], or its states stored [v][d] (transposed)
  TORCH_CHECK(part.dim() == 4 && state.dim() == 4 &&
              part.size(1) == state.size(1) &&
              part.size(2) * part.size(3) == state.size(2) * state.size(3));
  const int H = state.size(1), D = state.size(2), V = state.size(3);
  TORCH_CHECK(decay.numel() == H);
  const SeqMeta m = check_meta(cu, seq_lens, &slots, nullptr, 0);
  check_i32(chunk_off, "chunk_off");
  check_i32(chunk_rows, "chunk_rows");
  TORCH_CHECK(chunk_off.numel() == m.S + 1 &&
              chunk_rows.numel() == part.size(0));
  arks_seq_lightning_combine(part.data_ptr(), decay.data_ptr(),
                             state.data_ptr(), chunk_off.data_ptr(),
                             chunk_rows.data_ptr(), cu.data_ptr(),
                             seq_lens.data_ptr(), slots.data_ptr(), m.S, H, D,
                             V, transposed ? 1 : 0, current_stream());
}

// ---- stream arrangement, window/pool attention, grouped routing

void stream_mix_norm(Tensor xs, OptTensor n_out, OptTensor y, OptTensor y_bias,
                     OptTensor mix, OptTensor out_w, OptTensor in_w,
                     OptTensor norm_w, OptTensor norm_b, double eps) {
  check_f32(xs, "xs");
  TORCH_CHECK(xs.dim() == 3, "xs must be [streams, T, C]");
  const int S = xs.size(0), C = xs.size(2);
  const int64_t T = xs.size(1);
  int f32 = 1;
  int64_t ldy = 0;
  if (y.has_value()) {
    f32 = act_flag(*y, "y");
    TORCH_CHECK(y->size(0) == T && y->size(1) == C);
    ldy = row_stride(*y, "y");
    TORCH_CHECK(mix.has_value() && out_w.has_value());
    check_f32(*mix, "mix");
    check_f32(*out_w, "out weights");
    TORCH_CHECK(mix->numel() == S * S && out_w->numel() == S);
    if (y_bias.has_value()) {
      check_f32(*y_bias, "y bias");
      TORCH_CHECK(y_bias->numel() == C);
    }
  }
  if (in_w.has_value()) {
    check_f32(*in_w, "in weights");
    check_f32(*norm_w, "norm weight");
    check_f32(*norm_b, "norm bias");
    check_f32(*n_out, "norm output");
    TORCH_CHECK(in_w->numel() == S && norm_w->numel() == C &&
                norm_b->numel() == C && n_out->size(0) == T &&
                n_out->size(1) == C);
  }
  const int rc = arks_seq_stream_mix_norm(
      xs.data_ptr(), in_w.has_value() ? n_out->data_ptr() : nullptr,
      y.has_value() ? y->data_ptr() : nullptr, ldy,
      y.has_value() && y_bias.has_value() ? y_bias->data_ptr() : nullptr,
      y.has_value() ? mix->data_ptr() : nullptr,
      y.has_value() ? out_w->data_ptr() : nullptr,
      in_w.has_value() ? in_w->data_ptr() : nullptr,
      in_w.has_value() ? norm_w->data_ptr() : nullptr,
      in_w.has_value() ? norm_b->data_ptr() : nullptr, (float)eps, S, T, C,
      f32, current_stream());
  TORCH_CHECK(rc == 0, "more residual copies or a wider row than the kernel holds");
}

void short_conv_residual(Tensor out, Tensor h, Tensor w, OptTensor state,
                         Tensor cu, Tensor seq_lens, Tensor slots,
                         Tensor token_seq) {
  check_f32(h, "h");
  check_f32(w, "conv weight");
  const int f32 = act_flag(out, "out");
  const int T = h.size(0), C = h.size(1), taps = w.size(1);
  TORCH_CHECK(out.is_contiguous() && out.sizes() == h.sizes());
  TORCH_CHECK(w.dim() == 2 && w.size(0) == C && taps >= 1);
  const SeqMeta m = check_meta(cu, seq_lens, &slots, &token_seq, T);
  if (taps > 1) {
    TORCH_CHECK(state.has_value(), "a conv with history needs its state");
    check_f32(*state, "conv state");
    TORCH_CHECK(state->dim() == 3 && state->size(1) == taps - 1 &&
                state->size(2) == C, "state must be [slots, taps-1, C]");
  }
  const int rc = arks_seq_short_conv_residual(
      out.data_ptr(), h.data_ptr(), w.data_ptr(),
      taps > 1 ? state->data_ptr() : nullptr, cu.data_ptr(),
      seq_lens.data_ptr(), slots.data_ptr(), token_seq.data_ptr(), T, m.S, C,
      taps, f32, current_stream());
  TORCH_CHECK(rc == 0, "more conv taps than the kernel holds");
}

void head_norm_gate(Tensor out, Tensor o, Tensor gate, double eps,
                    int64_t heads, double out_scale) {
  check_f32(o, "o");
  const int f32 = act_flag(out, "out");
  TORCH_CHECK(o.dim() == 2 && o.size(1) % heads == 0);
  TORCH_CHECK(gate.scalar_type() == out.scalar_type() &&
              gate.sizes() == o.sizes() && out.sizes() == o.sizes());
  arks_seq_head_norm_gate(out.data_ptr(), row_stride(out, "out"), o.data_ptr(),
                          gate.data_ptr(), row_stride(gate, "gate"),
                          (float)eps, o.size(0), heads, o.size(1) / heads,
                          (float)out_scale, f32, current_stream());
}

void glu_act(Tensor out, Tensor gu, int64_t mode, double limit, double alpha,
             OptTensor row_scale) {
  const int f32 = act_flag(gu, "gate|up");
  TORCH_CHECK(gu.dim() == 2 && gu.size(1) % 2 == 0);
  const int F = gu.size(1) / 2;
  TORCH_CHECK(out.scalar_type() == gu.scalar_type() &&
              out.size(0) == gu.size(0) && out.size(1) == F);
  const void* rs_p = nullptr;
  if (row_scale.has_value()) {
    check_f32(*row_scale, "row_scale");
    TORCH_CHECK(row_scale->numel() == gu.size(0));
    rs_p = row_scale->data_ptr();
  }
  arks_seq_glu_act(out.data_ptr(), row_stride(out, "out"), gu.data_ptr(),
                   row_stride(gu, "gate|up"), gu.size(0), F, (int)mode,
                   (float)limit, (float)alpha, rs_p, f32, current_stream());
}

struct WindowShapes {
  int T, H, G, D, V, bs, spp, max_blocks, f32;
};

WindowShapes check_window(const Tensor& q, const Tensor& k_cache,
                          const Tensor& v_cache, const Tensor& kp,
                          const Tensor& vp, const Tensor& block_tables,
                          int64_t pool) {
  WindowShapes w;
  w.f32 = act_flag(q, "q");
  TORCH_CHECK(q.dim() == 3);
  w.T = q.size(0); w.H = q.size(1); w.D = q.size(2);
  for (const Tensor* c : {&k_cache, &v_cache, &kp, &vp})
    TORCH_CHECK(c->is_cuda() && c->is_contiguous() && c->dim() == 4 &&
                c->scalar_type() == q.scalar_type(),
                "caches must be contiguous [pages, G, n, dim] of q's dtype");
  w.G = k_cache.size(1); w.bs = k_cache.size(2); w.V = v_cache.size(3);
  w.spp = kp.size(2);
  TORCH_CHECK(pool >= 1 && w.spp == (w.bs - 1) / pool + 1,
              "pooled cache does not fit the pool size");
  TORCH_CHECK(k_cache.size(3) == w.D && kp.size(3) == w.D &&
              vp.size(3) == w.V && v_cache.size(1) == w.G &&
              kp.size(1) == w.G && vp.size(1) == w.G &&
              v_cache.size(2) == w.bs && vp.size(2) == w.spp &&
              kp.size(0) == k_cache.size(0) && vp.size(0) == k_cache.size(0) &&
              v_cache.size(0) == k_cache.size(0) && w.H % w.G == 0);
  check_i32(block_tables, "block_tables");
  TORCH_CHECK(block_tables.dim() == 2);
  w.max_blocks = block_tables.size(1);
  return w;
}

void kv_write_pooled(Tensor k, Tensor v, Tensor k_cache, Tensor v_cache,
                     Tensor kp, Tensor vp, Tensor slot_mapping,
                     Tensor positions, Tensor block_tables, Tensor token_seq,
                     int64_t pool) {
  const int f32 = act_flag(k, "k");
  TORCH_CHECK(k.dim() == 3 && v.dim() == 3 &&
              v.scalar_type() == k.scalar_type());
  for (const Tensor* c : {&k_cache, &v_cache, &kp, &vp})
    TORCH_CHECK(c->is_cuda() && c->is_contiguous() && c->dim() == 4 &&
                c->scalar_type() == k.scalar_type());
  const int T = k.size(0), G = k.size(1), D = k.size(2), V = v.size(2);
  const int bs = k_cache.size(2), spp = kp.size(2);
  TORCH_CHECK(v.size(0) == T && v.size(1) == G && k_cache.size(1) == G &&
              k_cache.size(3) == D && v_cache.size(1) == G &&
              v_cache.size(2) == bs && v_cache.size(3) == V &&
              kp.size(1) == G && kp.size(3) == D && vp.size(1) == G &&
              vp.size(2) == spp && vp.size(3) == V);
  TORCH_CHECK(pool >= 1 && spp == (bs - 1) / pool + 1);
  check_i64(slot_mapping, "slot_mapping");
  check_i64(positions, "positions");
  check_i32(block_tables, "block_tables");
  check_i32(token_seq, "token_seq");
  TORCH_CHECK(slot_mapping.numel() == T && positions.numel() == T &&
              token_seq.numel() == T && block_tables.dim() == 2);
  arks_seq_kv_write_pooled(
      k.data_ptr(), v.data_ptr(), head_row_stride(k, "k"),
      head_row_stride(v, "v"), k_cache.data_ptr(), v_cache.data_ptr(),
      kp.data_ptr(), vp.data_ptr(), slot_mapping.data_ptr(),
      positions.data_ptr(), block_tables.data_ptr(), token_seq.data_ptr(), T,
      (int)block_tables.size(1), G, D, V, bs, (int)pool, spp, f32,
      current_stream());
}

void attention_window_pool(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                           Tensor kp, Tensor vp, Tensor block_tables,
                           Tensor seq_lens, Tensor cu, Tensor token_seq,
                           double scale, int64_t window, int64_t pool,
                           double out_scale) {
  const WindowShapes w = check_window(q, k_cache, v_cache, kp, vp,
                                      block_tables, pool);
  TORCH_CHECK(out.scalar_type() == q.scalar_type() && out.dim() == 3 &&
              out.size(0) == w.T && out.size(1) == w.H && out.size(2) == w.V);
  check_meta(cu, seq_lens, nullptr, &token_seq, w.T);
  TORCH_CHECK(block_tables.size(0) == seq_lens.numel() && window >= 1);
  const int rc = arks_seq_attn_window_pool(
      out.data_ptr(), head_row_stride(out, "out"), q.data_ptr(),
      head_row_stride(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(),
      kp.data_ptr(), vp.data_ptr(), block_tables.data_ptr(),
      seq_lens.data_ptr(), cu.data_ptr(), token_seq.data_ptr(), (float)scale,
      (int)window, (int)pool, w.spp, (float)out_scale, w.T, w.H, w.G, w.D, w.V,
      w.bs, w.max_blocks, w.f32, current_stream());
  TORCH_CHECK(rc == 0, "head size beyond the kernel's limit");
}

// The matrix-core kernel; false: not built for these sizes (the caller
// runs the general kernel). single_rows: every sequence has one row in
// this step (a workgroup then takes the query heads of one group).
bool attention_window_pool_mfma(Tensor out, Tensor q, Tensor k_cache,
                                Tensor v_cache, Tensor kp, Tensor vp,
                                Tensor block_tables, Tensor seq_lens, Tensor cu,
                                Tensor token_seq, double scale, int64_t window,
                                int64_t pool, double out_scale,
                                bool single_rows) {
  const WindowShapes w = check_window(q, k_cache, v_cache, kp, vp,
                                      block_tables, pool);
  TORCH_CHECK(w.f32 == 0, "bf16 rows only");
  TORCH_CHECK(out.scalar_type() == q.scalar_type() && out.dim() == 3 &&
              out.size(0) == w.T && out.size(1) == w.H && out.size(2) == w.V);
  check_meta(cu, seq_lens, nullptr, &token_seq, w.T);
  TORCH_CHECK(block_tables.size(0) == seq_lens.numel() && window >= 1);
  return arks_seq_attn_window_pool_mfma(
             out.data_ptr(), head_row_stride(out, "out"), q.data_ptr(),
             head_row_stride(q, "q"), k_cache.data_ptr(), v_cache.data_ptr(),
             kp.data_ptr(), vp.data_ptr(), block_tables.data_ptr(),
             seq_lens.data_ptr(), cu.data_ptr(), token_seq.data_ptr(),
             (float)scale, (int)window, (int)pool, w.spp, (float)out_scale,
             w.T, w.H, w.G, w.D, w.V, w.bs, w.max_blocks,
             (int)seq_lens.numel(), single_rows ? 1 : 0,
             current_stream()) == 0;
}

void moe_route_grouped(Tensor weights, Tensor ids, Tensor logits, int64_t top,
                       int64_t groups, int64_t keep, bool sigmoid, bool renorm,
                       OptTensor matrix) {
  check_f32(logits, "router logits");
  check_f32(weights, "weights");
  check_i32(ids, "ids");
  const int T = logits.size(0), E = logits.size(1);
  TORCH_CHECK(weights.size(0) == T && weights.size(1) == top &&
              ids.size(0) == T && ids.size(1) == top);
  void* mat_p = nullptr;
  if (matrix.has_value()) {
    check_f32(*matrix, "scale matrix");
    TORCH_CHECK(matrix->dim() == 2 && matrix->size(0) == T &&
                matrix->size(1) == E);
    mat_p = matrix->data_ptr();
  }
  const int rc = arks_seq_moe_route_grouped(
      weights.data_ptr(), ids.data_ptr(), logits.data_ptr(), T, E, (int)top,
      (int)groups, (int)keep, sigmoid ? 1 : 0, renorm ? 1 : 0, mat_p,
      current_stream());
  TORCH_CHECK(rc == 0, "routing sizes the kernel does not hold");
}

void moe_mix_common(Tensor out, Tensor y, Tensor weights, Tensor rows,
                    int dense, const OptTensor& add = c10::nullopt) {
  const int f32 = act_flag(y, "y");
  check_f32(weights, "weights");
  check_i32(rows, "rows");
  TORCH_CHECK(y.is_contiguous() && out.is_contiguous() &&
              out.scalar_type() == y.scalar_type());
  const int T = weights.size(0), k = weights.size(1), H = out.size(1);
  TORCH_CHECK(out.size(0) == T && rows.numel() == (int64_t)T * k &&
              y.size(-1) == H);
  if (dense) TORCH_CHECK(y.dim() == 3 && y.size(1) == T);
  const void* add_p = nullptr;
  if (add.has_value()) {
    TORCH_CHECK(add->scalar_type() == y.scalar_type() && add->is_contiguous() &&
                add->is_cuda() && add->sizes() == out.sizes());
    add_p = add->data_ptr();
  }
  arks_seq_moe_mix_rows(out.data_ptr(), y.data_ptr(), weights.data_ptr(),
                        rows.data_ptr(), T, H, k, dense, add_p, f32,
                        current_stream());
}

void moe_mix(Tensor out, Tensor y, Tensor weights, Tensor ids) {
  moe_mix_common(out, y, weights, ids, 1);
}

void moe_mix_rows(Tensor out, Tensor y, Tensor weights, Tensor rows,
                  OptTensor add) {
  moe_mix_common(out, y, weights, rows, 0, add);
}

void residual_pair_norm(Tensor x, OptTensor h1, OptTensor h2, OptTensor y1,
                        OptTensor s1, OptTensor y2, OptTensor s2, OptTensor w1,
                        OptTensor w2, double eps) {
  check_f32(x, "x");
  TORCH_CHECK(x.dim() == 2);
  const int64_t T = x.size(0);
  const int C = x.size(1);
  int f32 = -1;
  auto rows = [&](const OptTensor& t, const char* name) -> void* {
    if (!t.has_value()) return nullptr;
    const int f = act_flag(*t, name);
    TORCH_CHECK(f32 < 0 || f == f32, "activation dtypes differ");
    f32 = f;
    TORCH_CHECK(t->dim() == 2 && t->size(0) == T && t->size(1) == C &&
                t->is_contiguous(), name, " must be contiguous [T, C]");
    return t->data_ptr();
  };
  auto vec = [&](const OptTensor& t, const char* name) -> const void* {
    if (!t.has_value()) return nullptr;
    check_f32(*t, name);
    TORCH_CHECK(t->numel() == C, name, " must have C entries");
    return t->data_ptr();
  };
  void* h1_p = rows(h1, "h1");
  void* h2_p = rows(h2, "h2");
  const void* y1_p = rows(y1, "y1");
  const void* y2_p = rows(y2, "y2");
  TORCH_CHECK(h1.has_value() == w1.has_value() &&
              h2.has_value() == w2.has_value() &&
              y1.has_value() == s1.has_value() &&
              y2.has_value() == s2.has_value());
  if (f32 < 0) return;  // nothing to add, nothing to write
  arks_seq_residual_pair_norm(x.data_ptr(), h1_p, h2_p, y1_p, vec(s1, "s1"),
                              y2_p, vec(s2, "s2"), vec(w1, "w1"),
                              vec(w2, "w2"), (float)eps, T, C, f32,
                              current_stream());
}

void conv_qkv_cache(Tensor qo, Tensor p, int64_t n_q, int64_t n_k, int64_t n_v,
                    Tensor w, OptTensor w_t, OptTensor state, Tensor cu,
                    Tensor seq_lens, Tensor slots, Tensor token_seq,
                    Tensor positions, double temp_coef, int64_t temp_every,
                    int64_t heads, int64_t kv_heads, int64_t maps,
                    OptTensor k_cache, OptTensor v_cache, Tensor slot_mapping) {
  const int f32 = act_flag(p, "p");
  const int64_t ldp = row_stride(p, "p");
  const int T = p.size(0);
  const int64_t C = n_q + n_k + n_v;
  TORCH_CHECK(p.size(1) >= C && n_q > 0 && heads > 0 && kv_heads > 0 &&
              maps > 0 && heads % kv_heads == 0 &&
              n_q % (heads * maps) == 0 && n_k % kv_heads == 0 &&
              n_v % kv_heads == 0);
  TORCH_CHECK(qo.scalar_type() == p.scalar_type() && qo.is_contiguous() &&
              qo.dim() == 2 && qo.size(0) == T && qo.size(1) == n_q);
  check_f32(w, "taps");
  TORCH_CHECK(w.dim() == 2 && w.size(0) == C);
  const int taps = w.size(1);
  const void* wt_p = nullptr;
  if (w_t.has_value()) {
    check_f32(*w_t, "transposed taps");
    TORCH_CHECK(w_t->dim() == 2 && w_t->size(0) == taps && w_t->size(1) == C);
    wt_p = w_t->data_ptr();
  }
  const SeqMeta m = check_meta(cu, seq_lens, &slots, &token_seq, T);
  void* st_p = nullptr;
  if (taps > 1) {
    TORCH_CHECK(state.has_value(), "a convolution with history needs state");
    check_f32(*state, "conv state");
    TORCH_CHECK(state->dim() == 3 && state->size(1) == taps - 1 &&
                state->size(2) == C);
    st_p = state->data_ptr();
  }
  check_i64(positions, "positions");
  check_i64(slot_mapping, "slot_mapping");
  TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
  void* kc_p = nullptr;
  void* vc_p = nullptr;
  int bs = 1;
  if (n_k > 0 || n_v > 0) {
    TORCH_CHECK(k_cache.has_value() && v_cache.has_value());
    TORCH_CHECK(k_cache->scalar_type() == p.scalar_type() &&
                v_cache->scalar_type() == p.scalar_type() &&
                k_cache->is_contiguous() && v_cache->is_contiguous() &&
                k_cache->dim() == 4 && v_cache->dim() == 4);
    TORCH_CHECK(k_cache->size(1) == kv_heads && v_cache->size(1) == kv_heads &&
                k_cache->size(3) * kv_heads == n_k &&
                v_cache->size(3) * kv_heads == n_v &&
                k_cache->size(2) == v_cache->size(2) &&
                k_cache->size(0) == v_cache->size(0), "cache shape mismatch");
    kc_p = k_cache->data_ptr();
    vc_p = v_cache->data_ptr();
    bs = k_cache->size(2);
  }
  const int rc = arks_seq_conv_qkv_cache(
      qo.data_ptr(), p.data_ptr(), ldp, w.data_ptr(), wt_p, st_p,
      cu.data_ptr(), seq_lens.data_ptr(), slots.data_ptr(),
      token_seq.data_ptr(), positions.data_ptr(), kc_p, vc_p,
      slot_mapping.data_ptr(), T, m.S, (int)n_q, (int)n_k, (int)n_v,
      (int)heads, (int)kv_heads, (int)maps, bs, taps, (float)temp_coef,
      (int)temp_every, f32, current_stream());
  TORCH_CHECK(rc == 0, "more taps than the convolution kernel holds");
}

void diff_head_norm_gate(Tensor out, Tensor a, Tensor gate, double lam,
                         double eps, double mult, int64_t heads,
                         int64_t kv_heads) {
  const int f32 = act_flag(a, "a");
  TORCH_CHECK(a.is_contiguous() && a.dim() == 3 && a.size(1) == 2 * heads &&
              heads % kv_heads == 0);
  const int T = a.size(0), V = a.size(2);
  TORCH_CHECK(out.scalar_type() == a.scalar_type() &&
              gate.scalar_type() == a.scalar_type() && out.dim() == 2 &&
              gate.dim() == 2 && out.size(0) == T && gate.size(0) == T &&
              out.size(1) == heads * V && gate.size(1) == heads * V);
  const int rc = arks_seq_diff_head_norm_gate(
      out.data_ptr(), row_stride(out, "out"), a.data_ptr(), gate.data_ptr(),
      row_stride(gate, "gate"), (float)lam, (float)eps, (float)mult, T,
      (int)heads, (int)kv_heads, V, f32, current_stream());
  TORCH_CHECK(rc == 0, "value size beyond the kernel's limit (", V, ")");
}

void moe_glu_scaled(Tensor out, Tensor gu, Tensor scale, int64_t experts,
                    int64_t ff, int64_t shared_ff) {
  const int f32 = act_flag(gu, "gate|up");
  check_f32(scale, "scale");
  const int64_t T = gu.size(0);
  TORCH_CHECK(gu.dim() == 2 &&
              gu.size(1) == experts * 2 * ff + 2 * shared_ff &&
              scale.dim() == 2 && scale.size(0) == T &&
              scale.size(1) == experts);
  TORCH_CHECK(out.scalar_type() == gu.scalar_type() && out.is_contiguous() &&
              out.dim() == 2 && out.size(0) == T &&
              out.size(1) == experts * ff + shared_ff);
  arks_seq_moe_glu_scaled(out.data_ptr(), gu.data_ptr(),
                          row_stride(gu, "gate|up"), scale.data_ptr(), T,
                          (int)experts, (int)ff, (int)shared_ff, f32,
                          current_stream());
}

}  // namespace

void residual_tanh_norm(Tensor x, OptTensor h, OptTensor xa, OptTensor y,
                        double mult, OptTensor alpha, OptTensor w,
                        OptTensor b) {
  check_f32(x, "x");
  TORCH_CHECK(x.dim() == 2);
  const int64_t T = x.size(0);
  const int C = x.size(1);
  int f32 = -1;
  auto same = [&](const Tensor& t, const char* name) {
    const int f = act_flag(t, name);
    TORCH_CHECK(f32 < 0 || f == f32, "activation dtypes differ");
    f32 = f;
    TORCH_CHECK(t.dim() == 2 && t.size(0) == T && t.size(1) == C, name,
                " must be [T, C]");
  };
  void* h_p = nullptr;
  void* xa_p = nullptr;
  const void* y_p = nullptr;
  int64_t ldxa = C;
  if (h.has_value()) {
    same(*h, "h");
    TORCH_CHECK(h->is_contiguous() && alpha.has_value() && w.has_value() &&
                b.has_value());
    check_f32(*alpha, "alpha");
    check_f32(*w, "weight");
    check_f32(*b, "bias");
    TORCH_CHECK(alpha->numel() == 1 && w->numel() == C && b->numel() == C);
    h_p = h->data_ptr();
  }
  if (xa.has_value()) {
    same(*xa, "xa");
    ldxa = row_stride(*xa, "xa");
    xa_p = xa->data_ptr();
  }
  if (y.has_value()) {
    same(*y, "y");
    TORCH_CHECK(y->is_contiguous());
    y_p = y->data_ptr();
  }
  if (f32 < 0) return;  // nothing to add, nothing to write
  arks_seq_residual_tanh_norm(
      x.data_ptr(), h_p, xa_p, ldxa, y_p, (float)mult,
      alpha.has_value() ? alpha->data_ptr() : nullptr,
      w.has_value() ? w->data_ptr() : nullptr,
      b.has_value() ? b->data_ptr() : nullptr, T, C, f32, current_stream());
}

void latent_prepare(Tensor cqn, Tensor cq, Tensor ckv, Tensor qw, Tensor kw,
                    double eps, Tensor positions, Tensor freq, Tensor cache,
                    Tensor slot_mapping) {
  const int f32 = act_flag(cq, "cq");
  const int T = cq.size(0), Rq = cq.size(1);
  check_f32(qw, "q norm");
  check_f32(kw, "kv norm");
  check_f32(freq, "inv_freq");
  const int Rk = kw.numel(), P = freq.numel();
  TORCH_CHECK(cqn.scalar_type() == cq.scalar_type() && cqn.is_contiguous() &&
              cqn.size(0) == T && cqn.size(1) == Rq && qw.numel() == Rq);
  TORCH_CHECK(ckv.scalar_type() == cq.scalar_type() && ckv.dim() == 2 &&
              ckv.size(0) == T && ckv.size(1) == Rk + 2 * P);
  TORCH_CHECK(cache.scalar_type() == cq.scalar_type() && cache.is_contiguous() &&
              cache.dim() == 4 && cache.size(1) == 1 &&
              cache.size(3) == Rk + 2 * P);
  check_i64(positions, "positions");
  check_i64(slot_mapping, "slot_mapping");
  TORCH_CHECK(positions.numel() == T && slot_mapping.numel() == T);
  arks_seq_latent_prepare(cqn.data_ptr(), cq.data_ptr(), row_stride(cq, "cq"),
                          ckv.data_ptr(), row_stride(ckv, "ckv"), qw.data_ptr(),
                          kw.data_ptr(), (float)eps, positions.data_ptr(),
                          freq.data_ptr(), cache.data_ptr(),
                          slot_mapping.data_ptr(), T, Rq, Rk, P, f32,
                          current_stream());
}

void latent_query(Tensor out, Tensor q, OptTensor q_abs, Tensor positions,
                  Tensor freq) {
  const int f32 = act_flag(q, "q");
  check_f32(freq, "inv_freq");
  check_i64(positions, "positions");
  TORCH_CHECK(q.dim() == 3 && q.is_contiguous() && out.dim() == 3 &&
              out.is_contiguous());
  const int T = q.size(0), H = q.size(1), P = freq.numel();
  const int D = q.size(2) - 2 * P;
  const int Rk = q_abs.has_value() ? (int)q_abs->size(2) : D;
  if (q_abs.has_value())
    TORCH_CHECK(q_abs->dim() == 3 && q_abs->is_contiguous() &&
                q_abs->size(0) == H && q_abs->size(1) == T &&
                q_abs->scalar_type() == q.scalar_type());
  TORCH_CHECK(D >= 0 && out.size(0) == T && out.size(1) == H &&
              out.size(2) == Rk + 2 * P && positions.numel() == T &&
              out.scalar_type() == q.scalar_type());
  arks_seq_latent_query(out.data_ptr(), q.data_ptr(),
                        q_abs.has_value() ? q_abs->data_ptr() : nullptr,
                        positions.data_ptr(), freq.data_ptr(), T, H, D, Rk, P,
                        f32, current_stream());
}

void mamba2_scan(OptTensor out, Tensor xbc, Tensor dt_raw, Tensor dt_bias,
                 Tensor rate, Tensor Dp, Tensor state, Tensor cu,
                 Tensor seq_lens, Tensor slots, int64_t P, int64_t V,
                 int64_t N, int64_t G, OptTensor dsum) {
  const int f32 = act_flag(xbc, "xbc");
  const int64_t T = xbc.size(0);
  TORCH_CHECK(dt_raw.scalar_type() == xbc.scalar_type() && dt_raw.dim() == 2 &&
              dt_raw.size(0) == T && dt_raw.size(1) == P);
  TORCH_CHECK(xbc.dim() == 2 && xbc.size(1) == P * V + 2 * G * N && G >= 1 &&
              P % G == 0);
  check_f32(dt_bias, "dt_bias");
  check_f32(rate, "rate");
  check_f32(Dp, "D");
  check_f32(state, "state");
  TORCH_CHECK(dt_bias.numel() == P && rate.numel() == P && Dp.numel() == P);
  TORCH_CHECK(state.dim() == 4 && state.size(1) == P && state.size(2) == N &&
              state.size(3) == V);
  const SeqMeta m = check_meta(cu, seq_lens, &slots, nullptr, 0);
  void* out_p = nullptr;
  if (out.has_value()) {
    check_f32(*out, "out");
    TORCH_CHECK(out->dim() == 2 && out->size(0) == T && out->size(1) == P * V);
    out_p = out->data_ptr();
  }
  void* ds_p = nullptr;
  if (dsum.has_value()) {
    check_f32(*dsum, "dsum");
    TORCH_CHECK(dsum->dim() == 2 && dsum->size(0) == state.size(0) &&
                dsum->size(1) == P);
    ds_p = dsum->data_ptr();
  }
  const int rc = arks_seq_mamba2_scan(
      out_p, xbc.data_ptr(), row_stride(xbc, "xbc"), dt_raw.data_ptr(),
      row_stride(dt_raw, "dt"), dt_bias.data_ptr(), rate.data_ptr(),
      Dp.data_ptr(), state.data_ptr(), cu.data_ptr(), seq_lens.data_ptr(),
      slots.data_ptr(), ds_p, m.S, (int)P, (int)V, (int)N, (int)G, f32,
      current_stream());
  TORCH_CHECK(rc == 0, "mamba2 state size beyond the kernel's limit (", N, ")");
}

void mamba2_combine(Tensor part, Tensor dsum, Tensor rate, Tensor state,
                    Tensor chunk_off, Tensor cu, Tensor seq_lens,
                    Tensor slots) {
  check_f32(part, "part");
  check_f32(dsum, "dsum");
  check_f32(rate, "rate");
  check_f32(state, "state");
  const int P = rate.numel();
  TORCH_CHECK(part.dim() == 4 && state.dim() == 4 && part.size(1) == P &&
              state.size(1) == P && part.size(2) == state.size(2) &&
              part.size(3) == state.size(3) && dsum.dim() == 2 &&
              dsum.size(0) == part.size(0) && dsum.size(1) == P);
  const SeqMeta m = check_meta(cu, seq_lens, &slots, nullptr, 0);
  check_i32(chunk_off, "chunk_off");
  TORCH_CHECK(chunk_off.numel() == m.S + 1);
  arks_seq_mamba2_combine(part.data_ptr(), dsum.data_ptr(), rate.data_ptr(),
                          state.data_ptr(), chunk_off.data_ptr(), cu.data_ptr(),
                          seq_lens.data_ptr(), slots.data_ptr(), m.S, P,
                          (int)(part.size(2) * part.size(3)), current_stream());
}

void gate_group_norm(Tensor out, Tensor y, Tensor z, Tensor w, int64_t groups,
                     double eps, double out_scale) {
  check_f32(y, "y");
  check_f32(w, "weight");
  const int f32 = act_flag(z, "z");
  TORCH_CHECK(y.dim() == 2);
  const int T = y.size(0), C = y.size(1);
  TORCH_CHECK(groups >= 1 && C % groups == 0 && w.numel() == C);
  TORCH_CHECK(out.scalar_type() == z.scalar_type() && z.dim() == 2 &&
              z.size(0) == T && z.size(1) == C && out.dim() == 2 &&
              out.size(0) == T && out.size(1) == C);
  arks_seq_gate_group_norm(out.data_ptr(), row_stride(out, "out"), y.data_ptr(),
                           z.data_ptr(), row_stride(z, "z"), w.data_ptr(),
                           (float)eps, T, C, (int)groups, (float)out_scale, f32,
                           current_stream());
}

// false: no matrix-core kernel for these sizes (the caller runs the general
// one)
bool attention_masked_mfma(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                           Tensor block_tables, Tensor seq_lens, Tensor cu,
                           Tensor token_seq, double scale, OptTensor sink_w,
                           double softcap, int64_t window, int64_t keep_first,
                           double out_scale, bool single_rows, int64_t maps) {
  TORCH_CHECK(q.is_cuda() && q.scalar_type() == torch::kBFloat16 &&
              q.is_contiguous() && q.dim() == 3 && maps >= 1);
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  TORCH_CHECK(k_cache.scalar_type() == q.scalar_type() &&
              v_cache.scalar_type() == q.scalar_type() &&
              out.scalar_type() == q.scalar_type());
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.size(3) == D * maps);
  // key groups: every key/value head of the cache once per map
  const int G = k_cache.size(1) * maps, bs = k_cache.size(2),
            V = v_cache.size(3);
  TORCH_CHECK(H % G == 0 && v_cache.size(1) * maps == G &&
              v_cache.size(2) == bs);
  TORCH_CHECK(maps == 1 || !sink_w.has_value());
  const int64_t ldk = paged_row_stride(k_cache, "k_cache");
  const int64_t ldv = paged_row_stride(v_cache, "v_cache");
  const int64_t ldo = head_row_stride(out, "out");
  TORCH_CHECK(out.size(0) == T && out.size(1) == H && out.size(2) == V);
  const void* sw_p = nullptr;
  if (sink_w.has_value()) {
    check_f32(*sink_w, "sink_w");
    TORCH_CHECK(sink_w->numel() == H);
    sw_p = sink_w->data_ptr();
  }
  check_i32(block_tables, "block_tables");
  TORCH_CHECK(block_tables.dim() == 2 &&
              block_tables.size(0) == seq_lens.numel());
  const SeqMeta m = check_meta(cu, seq_lens, nullptr, &token_seq, T);
  // partial sums of a key-split launch (fp32 [T, H, ksplit, V + 2])
  int ksplit = 1;
  Tensor ws;
  if (single_rows) {
    ksplit = arks_seq_attn_masked_ksplit(T, H, G, (int)block_tables.size(1));
    if (ksplit > 1)
      ws = torch::empty({(int64_t)T * H * ksplit * (V + 2)},
                        q.options().dtype(torch::kFloat32));
  }
  return arks_seq_attn_masked_mfma(
             out.data_ptr(), ldo, q.data_ptr(), k_cache.data_ptr(), ldk,
             v_cache.data_ptr(), ldv, block_tables.data_ptr(),
             seq_lens.data_ptr(), cu.data_ptr(), token_seq.data_ptr(),
             (float)scale, sw_p, (float)softcap, (int)window, (int)keep_first,
             (float)out_scale, T, H, G, D, V, bs, (int)block_tables.size(1),
             m.S, single_rows ? 1 : 0, ksplit > 1 ? ws.data_ptr() : nullptr,
             ksplit, (int)maps, current_stream()) == 0;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("residual_tanh_norm", &residual_tanh_norm);
  m.def("latent_prepare", &latent_prepare);
  m.def("latent_query", &latent_query);
  m.def("mamba2_scan", &mamba2_scan);
  m.def("mamba2_combine", &mamba2_combine);
  m.def("gate_group_norm", &gate_group_norm);
  m.def("residual_pair_norm", &residual_pair_norm);
  m.def("conv_qkv_cache", &conv_qkv_cache);
  m.def("diff_head_norm_gate", &diff_head_norm_gate);
  m.def("moe_glu_scaled", &moe_glu_scaled);
  m.def("attention_masked_mfma", &attention_masked_mfma);
  m.def("stream_mix_norm", &stream_mix_norm);
  m.def("short_conv_residual", &short_conv_residual);
  m.def("head_norm_gate", &head_norm_gate);
  m.def("glu_act", &glu_act);
  m.def("kv_write_pooled", &kv_write_pooled);
  m.def("attention_window_pool", &attention_window_pool);
  m.def("attention_window_pool_mfma", &attention_window_pool_mfma);
  m.def("moe_route_grouped", &moe_route_grouped);
  m.def("moe_mix", &moe_mix);
  m.def("moe_mix_rows", &moe_mix_rows);
  def_paged_attention(m);
  m.def("unrotate_rows", &unrotate_rows);
  m.def("token_shift", &token_shift);
  m.def("gated_norm_residual", &gated_norm_residual);
  m.def("rms_norm_f32", &rms_norm_f32);
  m.def("gated_rmsnorm", &gated_rmsnorm);
  m.def("gelu_tanh", &gelu_tanh);
  m.def("qk_norm_rope_cache", &qk_norm_rope_cache);
  m.def("attention_sink_paged", &attention_sink_paged);
  m.def("lightning_scan", &lightning_scan);
  m.def("causal_conv_silu", &causal_conv_silu);
  m.def("selective_scan", &selective_scan);
  m.def("scan_combine", &scan_combine);
  m.def("lightning_combine", &lightning_combine);
  m.def("lightning_mfma", &lightning_mfma);
}
