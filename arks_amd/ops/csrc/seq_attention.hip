// Causal grouped-query attention of packed new rows over paged keys, any
// head sizes, any activation type, fp32 arithmetic throughout: the general
// kernel of the sink attention (arks_amd/models/mixers.py). The bf16 MFMA
// kernels in seq_attention_mfma.hip take over where their tiling fits.
//
// One wave per (row, query head). Keys are visited 64 at a time: lane j
// scores key j (dot over D against the query held in LDS), the wave takes
// the running maximum and rescales, then every lane accumulates its own
// value dims over the tile's 64 weights. The softmax may carry a sink: a
// key of score 0 without a value, i.e. the running state starts at
// (max 0, sum 1) instead of (-inf, 0); with sink_w the sink's score is a
// number per head, (max sink_w[h], sum 1). softcap c > 0 turns a score s
// into c tanh(s / c). window w > 0: the row at position i sees key j <= i
// only if i - j < w or j < keep_first; tiles with no visible key are
// skipped. Key and value rows have their own strides (ldk, ldv), so the
// value may be a leading part of the key's row (latent attention keeps one
// row per token for both). The output is a row-strided view (ldo), scaled
// by out_scale. After the sum each row's output is turned back by its own
// position when the cache holds position-turned values. maps M > 1: a key
// row holds M keys of D dims side by side (row stride ldk >= M * D) that
// share the row's value; H counts all query heads, in H / (G * M)-head
// groups, and group g * M + m reads key m of key/value head g.
#include "seq_common.h"

namespace arks {

constexpr int ATT_MAX_D = 1024;  // query dims held in LDS
constexpr int ATT_VPT = 8;      // value dims per lane (V <= 512)

template <typename AT>
__global__ __launch_bounds__(64) void attn_sink_generic_kernel(
    AT* __restrict__ out, const AT* __restrict__ q,
    const AT* __restrict__ k_cache, const AT* __restrict__ v_cache,
    const int* __restrict__ block_tables, const int* __restrict__ seq_lens,
    const int* __restrict__ cu, const int* __restrict__ token_seq,
    float scale, int sink, const float* __restrict__ freq_v, int interleaved,
    int H, int G, int D, int V, int block_size, int max_blocks,
    const float* __restrict__ sink_w, float softcap, int window,
    int keep_first, int64_t ldk, int64_t ldv, int64_t ldo, float out_scale,
    int maps) {
  __shared__ float q_s[ATT_MAX_D];
  __shared__ float p_s[64];
  __shared__ int64_t voff_s[64];
  __shared__ float o_s[64 * ATT_VPT];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int s = token_seq[t];
  const int first_row = cu[s];
  const int rows = cu[s + 1] - first_row;
  const int pos = seq_lens[s] - rows + (t - first_row);
  const int nkeys = pos + 1;
  const int gm = h / (H / (G * maps));  // key group: (kv head, map)
  const int g = gm / maps;
  const int kcol = (gm % maps) * D;
  const int* bt = block_tables + (int64_t)s * max_blocks;
  for (int d = lane; d < D; d += 64)
    q_s[d] = Act<AT>::ld(q + ((int64_t)t * H + h) * D + d);
  __syncthreads();
  float m = sink_w ? sink_w[h] : (sink ? 0.f : -INFINITY);
  float l = (sink_w || sink) ? 1.f : 0.f;
  float acc[ATT_VPT];
#pragma unroll
  for (int i = 0; i < ATT_VPT; ++i) acc[i] = 0.f;
  // first key of the window; keys in [keep_first, lo) are hidden
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  for (int j0 = 0; j0 < nkeys; j0 += 64) {
    if (j0 >= keep_first && j0 + 64 <= lo) continue;
    const int j = j0 + lane;
    const bool valid = j < nkeys && (j >= lo || j < keep_first);
    float sc = -INFINITY;
    int64_t rowoff = 0;
    if (valid) {
      const int page = bt[j / block_size];
      rowoff = ((int64_t)page * G + g) * block_size + (j % block_size);
      const AT* kr = k_cache + rowoff * ldk + kcol;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot += q_s[d] * Act<AT>::ld(kr + d);
      sc = dot * scale;
      if (softcap > 0.f) sc = softcap * tanhf(sc / softcap);
    }
    const float m_new = fmaxf(m, wave_reduce_max(sc));
    const float p = valid ? expf(sc - m_new) : 0.f;
    const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * corr + wave_reduce_sum(p);
#pragma unroll
    for (int i = 0; i < ATT_VPT; ++i) acc[i] *= corr;
    m = m_new;
    __syncthreads();  // previous tile's readers are done
    p_s[lane] = p;
    voff_s[lane] = rowoff * ldv;
    __syncthreads();
    const int cnt = min(64, nkeys - j0);
    for (int jj = 0; jj < cnt; ++jj) {
      const float pj = p_s[jj];
      if (pj == 0.f) continue;  // hidden key (uniform over the wave)
      const AT* vr = v_cache + voff_s[jj];
#pragma unroll
      for (int i = 0; i < ATT_VPT; ++i) {
        const int d = lane + 64 * i;
        if (d < V) acc[i] += pj * Act<AT>::ld(vr + d);
      }
    }
  }
  const float inv = l > 0.f ? out_scale / l : 0.f;
  AT* orow = out + (int64_t)t * ldo + (int64_t)h * V;
  if (!freq_v) {
#pragma unroll
    for (int i = 0; i < ATT_VPT; ++i) {
      const int d = lane + 64 * i;
      if (d < V) Act<AT>::st(orow + d, acc[i] * inv);
    }
    return;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < ATT_VPT; ++i) {
    const int d = lane + 64 * i;
    if (d < V) o_s[d] = acc[i] * inv;
  }
  __syncthreads();
  const int npairs = V / 2;
  for (int i = lane; i < npairs; i += 64) {
    const int d0 = interleaved ? 2 * i : i;
    const int d1 = interleaved ? 2 * i + 1 : i + npairs;
    const float a = o_s[d0], b = o_s[d1];
    float sn, cs;
    sincosf(-(float)pos * freq_v[i], &sn, &cs);
    Act<AT>::st(orow + d0, a * cs - b * sn);
    Act<AT>::st(orow + d1, b * cs + a * sn);
  }
}

}  // namespace arks

using namespace arks;

extern "C" int arks_seq_attn_sink_generic(
    void* out, const void* q, const void* k_cache, const void* v_cache,
    const void* block_tables, const void* seq_lens, const void* cu,
    const void* token_seq, float scale, int sink, const void* freq_v,
    int interleaved, int T, int H, int G, int D, int V, int block_size,
    int max_blocks, int act_f32, const void* sink_w, float softcap,
    int window, int keep_first, int64_t ldk, int64_t ldv, int64_t ldo,
    float out_scale, int maps, hipStream_t stream) {
  if (D > ATT_MAX_D || V > 64 * ATT_VPT) return 1;
  if (T == 0) return 0;
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (attn_sink_generic_kernel<AT>), dim3(T, H), dim3(64), 0, stream,
      (AT*)out, (const AT*)q, (const AT*)k_cache, (const AT*)v_cache,
      (const int*)block_tables, (const int*)seq_lens, (const int*)cu,
      (const int*)token_seq, scale, sink, (const float*)freq_v, interleaved, H,
      G, D, V, block_size, max_blocks, (const float*)sink_w, softcap, window,
      keep_first, ldk, ldv, ldo, out_scale, maps));
  return 0;
}
