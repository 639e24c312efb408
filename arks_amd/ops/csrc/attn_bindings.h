// Bindings of the paged attention kernels (attn_decode.hip, attn_extend.hip,
// attn_extend2.hip). Both extensions compile those kernels and include this
// header: arks_amd_C serves them to the llama-family models, arks_amd_seq_C
// to the sink attention of the layer-list decoders (sink = 1: every softmax
// also holds a value-less key of score 0).
#pragma once

#include <torch/extension.h>

#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

extern "C" {
void arks_attn_decode_paged(void* out, void* part_out, const void* q,
                            const void* k_cache, const void* v_cache,
                            const void* block_tables, const void* seq_lens,
                            float scale, int num_seqs, int num_q_heads,
                            int num_kv_heads, int head_dim, int max_blocks,
                            int nparts, int64_t q_stride, int kv_fp8,
                            int window, int sink, hipStream_t stream);
void arks_attn_extend_paged(void* out, const void* q, const void* k_cache,
                            const void* v_cache, const void* block_tables,
                            const void* kv_lens, const void* cu_seqlens_q,
                            const void* tile_info, int ntiles, float scale,
                            int num_q_heads, int num_kv_heads, int head_dim,
                            int max_blocks, int64_t q_stride, int kv_fp8,
                            int window, int sink, int maps,
                            hipStream_t stream);
void arks_attn_extend_paged2(void* out, const void* q, const void* k_cache,
                             const void* v_cache, const void* block_tables,
                             const void* kv_lens, const void* cu_seqlens_q,
                             const void* tile_info, void* part_ws, int ntiles,
                             float scale, int num_q_heads, int num_kv_heads,
                             int head_dim, int max_blocks, int64_t q_stride,
                             int window, int sink, int maps,
                             hipStream_t stream);
void arks_attn_extend2_combine(void* out, const void* part_ws,
                               const void* combine_table,
                               const void* cu_seqlens_q, int n_split,
                               float scale, int num_q_heads, int head_dim,
                               hipStream_t stream);
}

namespace {

inline hipStream_t attn_current_stream() {
  return c10::hip::getCurrentHIPStream().stream();
}

inline bool check_kv_cache(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be on GPU");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
  if (t.scalar_type() == torch::kFloat8_e4m3fn) return true;
  TORCH_CHECK(t.scalar_type() == torch::kBFloat16, name, " must be bf16/fp8");
  return false;
}
inline void check_bf16_contig(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be on GPU");
  TORCH_CHECK(t.scalar_type() == torch::kBFloat16, name, " must be bf16");
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}
inline void check_bf16_rowstrided(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be on GPU");
  TORCH_CHECK(t.scalar_type() == torch::kBFloat16, name, " must be bf16");
  TORCH_CHECK(t.stride(-1) == 1, name, " last dim must be contiguous");
  if (t.dim() == 3) {
    TORCH_CHECK(t.stride(1) == t.size(2), name, " inner dims must be dense");
  }
}
inline void attention_decode_paged(torch::Tensor out, torch::Tensor q,
                            torch::Tensor k_cache, torch::Tensor v_cache,
                            torch::Tensor block_tables, torch::Tensor seq_lens,
                            double scale, torch::Tensor part_out,
                            int64_t nparts, int64_t window, int64_t sink) {
  check_bf16_contig(out, "out");
  check_bf16_rowstrided(q, "q");
  const bool kv_fp8 = check_kv_cache(k_cache, "k_cache");
  check_kv_cache(v_cache, "v_cache");
  TORCH_CHECK(block_tables.scalar_type() == torch::kInt32);
  TORCH_CHECK(seq_lens.scalar_type() == torch::kInt32);
  const int num_seqs = q.size(0);
  const int num_q_heads = q.size(1);
  const int head_dim = q.size(2);
  const int num_kv_heads = k_cache.size(1);
  TORCH_CHECK(k_cache.size(2) == 16, "KV block size must be 16");
  TORCH_CHECK(head_dim == 64 || head_dim == 128, "head_dim must be 64 or 128");
  const int gq = num_q_heads / num_kv_heads;
  TORCH_CHECK(gq >= 1 && gq <= 8 && gq * num_kv_heads == num_q_heads,
              "q/kv head ratio must be integral and <= 8");
  const int max_blocks = block_tables.size(1);
  if (nparts > 1) {
    TORCH_CHECK(part_out.scalar_type() == torch::kFloat32 &&
                part_out.numel() >=
                    (int64_t)num_seqs * num_kv_heads * nparts * gq *
                        (head_dim + 2),
                "part_out workspace too small");
  }
  arks_attn_decode_paged(out.data_ptr(),
                         nparts > 1 ? part_out.data_ptr() : nullptr,
                         q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                         block_tables.data_ptr(), seq_lens.data_ptr(),
                         (float)scale, num_seqs, num_q_heads, num_kv_heads,
                         head_dim, max_blocks, (int)nparts, q.stride(0),
                         kv_fp8 ? 1 : 0, (int)window, (int)sink,
                         attn_current_stream());
}
inline void attention_extend_paged(torch::Tensor out, torch::Tensor q,
                            torch::Tensor k_cache, torch::Tensor v_cache,
                            torch::Tensor block_tables, torch::Tensor kv_lens,
                            torch::Tensor cu_seqlens_q, torch::Tensor tile_info,
                            double scale, int64_t window, int64_t sink,
                            int64_t maps) {
  check_bf16_contig(out, "out");
  check_bf16_rowstrided(q, "q");
  const bool kv_fp8 = check_kv_cache(k_cache, "k_cache");
  check_kv_cache(v_cache, "v_cache");
  TORCH_CHECK(block_tables.scalar_type() == torch::kInt32);
  TORCH_CHECK(kv_lens.scalar_type() == torch::kInt32);
  TORCH_CHECK(cu_seqlens_q.scalar_type() == torch::kInt32);
  TORCH_CHECK(tile_info.scalar_type() == torch::kInt32);
  TORCH_CHECK(tile_info.dim() == 2 && tile_info.size(1) == 2);
  const int num_q_heads = q.size(1);
  const int head_dim = q.size(2);
  // key groups: every head of the cache once per key map of its rows
  const int num_kv_heads = k_cache.size(1) * maps;
  TORCH_CHECK(maps >= 1 && k_cache.size(3) == head_dim * maps &&
                  v_cache.size(3) == head_dim &&
                  v_cache.size(1) == k_cache.size(1) &&
                  num_q_heads % num_kv_heads == 0,
              "cache rows do not fit the heads and key maps");
  TORCH_CHECK(k_cache.size(2) == 16, "KV block size must be 16");
  TORCH_CHECK(head_dim == 32 || head_dim == 64 || head_dim == 96 ||
                  head_dim == 128 || head_dim == 256,
              "head_dim must be 32, 64, 96, 128 or 256");
  TORCH_CHECK(!kv_fp8 || head_dim == 64 || head_dim == 128,
              "fp8 KV needs head_dim 64 or 128");
  const int ntiles = tile_info.size(0);
  const int max_blocks = block_tables.size(1);
  arks_attn_extend_paged(out.data_ptr(), q.data_ptr(), k_cache.data_ptr(),
                         v_cache.data_ptr(), block_tables.data_ptr(),
                         kv_lens.data_ptr(), cu_seqlens_q.data_ptr(),
                         tile_info.data_ptr(), ntiles, (float)scale,
                         num_q_heads, num_kv_heads, head_dim, max_blocks,
                         q.stride(0), kv_fp8 ? 1 : 0, (int)window, (int)sink,
                         (int)maps, attn_current_stream());
}
inline void attention_extend_paged2(torch::Tensor out, torch::Tensor q,
                             torch::Tensor k_cache, torch::Tensor v_cache,
                             torch::Tensor block_tables, torch::Tensor kv_lens,
                             torch::Tensor cu_seqlens_q,
                             torch::Tensor tile_info, torch::Tensor part_ws,
                             double scale, int64_t window, int64_t sink,
                             int64_t maps) {
  check_bf16_contig(out, "out");
  check_bf16_rowstrided(q, "q");
  check_bf16_contig(k_cache, "k_cache");
  check_bf16_contig(v_cache, "v_cache");
  TORCH_CHECK(block_tables.scalar_type() == torch::kInt32);
  TORCH_CHECK(kv_lens.scalar_type() == torch::kInt32);
  TORCH_CHECK(cu_seqlens_q.scalar_type() == torch::kInt32);
  TORCH_CHECK(tile_info.scalar_type() == torch::kInt32);
  TORCH_CHECK(tile_info.dim() == 2 && tile_info.size(1) == 4,
              "tile_info rows are (seq, q0, part, nparts)");
  const int num_q_heads = q.size(1);
  const int head_dim = q.size(2);
  const int num_kv_heads = k_cache.size(1) * maps;
  TORCH_CHECK(maps >= 1 && k_cache.size(3) == head_dim * maps &&
                  v_cache.size(3) == head_dim &&
                  v_cache.size(1) == k_cache.size(1) &&
                  num_q_heads % num_kv_heads == 0,
              "cache rows do not fit the heads and key maps");
  TORCH_CHECK(k_cache.size(2) == 16, "KV block size must be 16");
  TORCH_CHECK(head_dim == 64 || head_dim == 128, "head_dim must be 64 or 128");
  const int ntiles = tile_info.size(0);
  const int max_blocks = block_tables.size(1);
  void* ws = nullptr;
  if (part_ws.numel() > 0) {
    // sized by the host: split rows sort first, so only their slabs exist
    TORCH_CHECK(part_ws.scalar_type() == torch::kFloat32);
    ws = part_ws.data_ptr();
  }
  arks_attn_extend_paged2(out.data_ptr(), q.data_ptr(), k_cache.data_ptr(),
                          v_cache.data_ptr(), block_tables.data_ptr(),
                          kv_lens.data_ptr(), cu_seqlens_q.data_ptr(),
                          tile_info.data_ptr(), ws, ntiles, (float)scale,
                          num_q_heads, num_kv_heads, head_dim, max_blocks,
                          q.stride(0), (int)window, (int)sink, (int)maps,
                          attn_current_stream());
}
inline void attention_extend2_combine(torch::Tensor out, torch::Tensor part_ws,
                               torch::Tensor combine_table,
                               torch::Tensor cu_seqlens_q, double scale) {
  check_bf16_rowstrided(out, "out");
  TORCH_CHECK(part_ws.scalar_type() == torch::kFloat32);
  TORCH_CHECK(combine_table.scalar_type() == torch::kInt32 &&
              combine_table.dim() == 2 && combine_table.size(1) == 4);
  const int num_q_heads = out.size(1);
  const int head_dim = out.size(2);
  arks_attn_extend2_combine(out.data_ptr(), part_ws.data_ptr(),
                            combine_table.data_ptr(), cu_seqlens_q.data_ptr(),
                            combine_table.size(0), (float)scale, num_q_heads,
                            head_dim, attn_current_stream());
}

inline void def_paged_attention(pybind11::module_& m) {
  m.def("attention_decode_paged", &attention_decode_paged);
  m.def("attention_extend_paged", &attention_extend_paged);
  m.def("attention_extend_paged2", &attention_extend_paged2);
  m.def("attention_extend2_combine", &attention_extend2_combine);
}

}  // namespace
