// Row kernels of the two-norm parallel block and of difference attention
// (arks_amd/models/hybrid.py DualNormBlock, models/mixers.py DiffAttention,
// models/feedforward.py InputScaledMoE), bf16 or float rows, fp32
// arithmetic:
//
//   residual_pair_norm   x += s1 * y1 + s2 * y2 (per-channel s, each branch
//       optional) on the fp32 residual, then both norms of the new row from
//       one sum of squares: h_q = x / sqrt(mean(x^2) + eps) * (1 + w_q)
//   conv_qkv_cache       causal depthwise convolution over time of the
//       q | k | v channels of the in-projection's rows (taps per channel, no
//       bias, no activation; inputs before the step's first row come from
//       the sequence's stored history, zeros at position 0); q times
//       1 + coef ln(floor((pos + 1) / every) + 1) and regrouped from
//       [head, map, dim] to [kv head, map, head of the group, dim]; k and v
//       rows to their pages; then the new histories (second launch, so every
//       reader of the first sees the old ones)
//   diff_head_norm_gate  (a1 - lambda a2) / rms * mult * sigmoid(gate) per
//       head from the two maps' attention outputs
//   moe_glu_scaled       silu(s g) * (s u) for every expert's [gate | up]
//       columns with the row's factor for that expert, silu(g) * u for the
//       shared expert's
#include "seq_common.h"

namespace arks {

// ---------------------------------------------------------------- norms
// One block per row, any width.
template <typename AT>
__global__ __launch_bounds__(256) void residual_pair_norm_kernel(
    float* __restrict__ x, AT* __restrict__ h1, AT* __restrict__ h2,
    const AT* __restrict__ y1, const float* __restrict__ s1,
    const AT* __restrict__ y2, const float* __restrict__ s2,
    const float* __restrict__ w1, const float* __restrict__ w2, float eps,
    int C) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  float* xr = x + t * C;
  float ss = 0.f;
  for (int c = threadIdx.x; c < C; c += 256) {
    float v = xr[c];
    if (y1 || y2) {
      float add = 0.f;
      if (y1) add += s1[c] * Act<AT>::ld(y1 + t * C + c);
      if (y2) add += s2[c] * Act<AT>::ld(y2 + t * C + c);
      v += add;
      xr[c] = v;
    }
    ss += v * v;
  }
  if (!h1 && !h2) return;
  ss = block_reduce_sum<256>(ss, red);
  const float rstd = 1.f / sqrtf(ss / (float)C + eps);
  for (int c = threadIdx.x; c < C; c += 256) {
    const float n = xr[c] * rstd;  // this thread's own writes
    if (h1) Act<AT>::st(h1 + t * C + c, n * (1.f + w1[c]));
    if (h2) Act<AT>::st(h2 + t * C + c, n * (1.f + w2[c]));
  }
}

// bf16 rows, C % 8 == 0, C <= 256 * 8 * PAIR_NORM_IT: every thread keeps
// its pieces of the new row in registers between the two passes; 16-byte
// accesses of the bf16 rows, two float4 of the residual.
constexpr int PAIR_NORM_IT = 4;

__global__ __launch_bounds__(256) void residual_pair_norm_vec8_kernel(
    float* __restrict__ x, bf16* __restrict__ h1, bf16* __restrict__ h2,
    const bf16* __restrict__ y1, const float* __restrict__ s1,
    const bf16* __restrict__ y2, const float* __restrict__ s2,
    const float* __restrict__ w1, const float* __restrict__ w2, float eps,
    int C) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  float* xr = x + t * C;
  float v[PAIR_NORM_IT][8];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < PAIR_NORM_IT; ++it) {
    const int c = (it * 256 + threadIdx.x) * 8;
    if (c < C) {
      const float4v a = *reinterpret_cast<const float4v*>(xr + c);
      const float4v b = *reinterpret_cast<const float4v*>(xr + c + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { v[it][e] = a[e]; v[it][4 + e] = b[e]; }
      if (y1) {
        const ushort8 u = *reinterpret_cast<const ushort8*>(y1 + t * C + c);
        const float4v sa = *reinterpret_cast<const float4v*>(s1 + c);
        const float4v sb = *reinterpret_cast<const float4v*>(s1 + c + 4);
#pragma unroll
        for (int e = 0; e < 8; ++e)
          v[it][e] += (e < 4 ? sa[e] : sb[e - 4]) * bf16_bits_to_float(u[e]);
      }
      if (y2) {
        const ushort8 u = *reinterpret_cast<const ushort8*>(y2 + t * C + c);
        const float4v sa = *reinterpret_cast<const float4v*>(s2 + c);
        const float4v sb = *reinterpret_cast<const float4v*>(s2 + c + 4);
#pragma unroll
        for (int e = 0; e < 8; ++e)
          v[it][e] += (e < 4 ? sa[e] : sb[e - 4]) * bf16_bits_to_float(u[e]);
      }
      if (y1 || y2) {
        float4v a2, b2;
#pragma unroll
        for (int e = 0; e < 4; ++e) { a2[e] = v[it][e]; b2[e] = v[it][4 + e]; }
        *reinterpret_cast<float4v*>(xr + c) = a2;
        *reinterpret_cast<float4v*>(xr + c + 4) = b2;
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += v[it][e] * v[it][e];
    }
  }
  if (!h1 && !h2) return;
  ss = block_reduce_sum<256>(ss, red);
  const float rstd = 1.f / sqrtf(ss / (float)C + eps);
#pragma unroll
  for (int it = 0; it < PAIR_NORM_IT; ++it) {
    const int c = (it * 256 + threadIdx.x) * 8;
    if (c < C) {
      if (h1) {
        const float4v wa = *reinterpret_cast<const float4v*>(w1 + c);
        const float4v wb = *reinterpret_cast<const float4v*>(w1 + c + 4);
        ushort8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          o[e] = float_to_bf16_bits(v[it][e] * rstd *
                                    (1.f + (e < 4 ? wa[e] : wb[e - 4])));
        *reinterpret_cast<ushort8*>(h1 + t * C + c) = o;
      }
      if (h2) {
        const float4v wa = *reinterpret_cast<const float4v*>(w2 + c);
        const float4v wb = *reinterpret_cast<const float4v*>(w2 + c + 4);
        ushort8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          o[e] = float_to_bf16_bits(v[it][e] * rstd *
                                    (1.f + (e < 4 ? wa[e] : wb[e - 4])));
        *reinterpret_cast<ushort8*>(h2 + t * C + c) = o;
      }
    }
  }
}

// ----------------------------------------------------------- convolution
constexpr int QKV_MAX_HIST = 31;     // taps - 1, general kernels
constexpr int QKV_VEC_MAX_TAPS = 9;  // taps the vectorised kernel holds

struct QkvConvArgs {
  int n_q, n_k, n_v;       // channels of each kind, in this order
  int heads, kv_heads, maps, dim;  // query layout [heads, maps, dim]
  int kdim, vdim;          // per key/value head: n_k / kv_heads, n_v / kv_heads
  int block_size, taps;
  float temp_coef;
  int temp_every;
};

__device__ __forceinline__ float query_factor(int64_t pos, float coef,
                                              int every) {
  if (every <= 0) return 1.f;
  return 1.f + coef * logf((float)((pos + 1) / every) + 1.f);
}

// channel c of a query row [head, map, dim] -> [kv head, map, head of the
// group, dim]
__device__ __forceinline__ int query_dest(int c, const QkvConvArgs& a) {
  const int d = c % a.dim;
  const int m = (c / a.dim) % a.maps;
  const int h = c / (a.dim * a.maps);
  const int r = a.heads / a.kv_heads;
  return (((h / r) * a.maps + m) * r + h % r) * a.dim + d;
}

// One block per row, threads over channels.
template <typename AT>
__global__ __launch_bounds__(256) void conv_qkv_cache_kernel(
    AT* __restrict__ qo, const AT* __restrict__ p, int64_t ldp,
    const float* __restrict__ w, const float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ seq_lens,
    const int* __restrict__ slots, const int* __restrict__ token_seq,
    const int64_t* __restrict__ positions, AT* __restrict__ k_cache,
    AT* __restrict__ v_cache, const int64_t* __restrict__ slot_mapping,
    QkvConvArgs a) {
  const int t = blockIdx.x;
  const int C = a.n_q + a.n_k + a.n_v;
  const SeqRow r = seq_row(t, token_seq, cu, seq_lens, slots);
  const int i = t - r.first_row;
  const bool has_state = r.start > 0 && r.slot >= 0 && a.taps > 1;
  const float* hist =
      state ? state + (int64_t)(r.slot < 0 ? 0 : r.slot) * (a.taps - 1) * C
            : nullptr;
  const float qf = query_factor(positions[t], a.temp_coef, a.temp_every);
  const int64_t slot = slot_mapping[t];
  const int64_t blk = slot / a.block_size, off = slot % a.block_size;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += gridDim.y * 256) {
    float acc = 0.f;
    for (int j = 0; j < a.taps; ++j) {
      const int src = i - (a.taps - 1 - j);
      float xv;
      if (src >= 0)
        xv = Act<AT>::ld(p + (int64_t)(r.first_row + src) * ldp + c);
      else
        xv = has_state ? hist[(int64_t)(src + a.taps - 1) * C + c] : 0.f;
      acc += w[(int64_t)c * a.taps + j] * xv;
    }
    if (c < a.n_q) {
      Act<AT>::st(qo + (int64_t)t * a.n_q + query_dest(c, a), acc * qf);
    } else if (slot >= 0) {
      if (c < a.n_q + a.n_k) {
        const int ck = c - a.n_q;
        const int g = ck / a.kdim, d = ck % a.kdim;
        Act<AT>::st(k_cache + ((blk * a.kv_heads + g) * a.block_size + off) *
                                  a.kdim + d, acc);
      } else {
        const int cv = c - a.n_q - a.n_k;
        const int g = cv / a.vdim, d = cv % a.vdim;
        Act<AT>::st(v_cache + ((blk * a.kv_heads + g) * a.block_size + off) *
                                  a.vdim + d, acc);
      }
    }
  }
}

// bf16 rows, 8 channels per thread (a piece never crosses a head, a map or
// the q | k | v borders: dim, kdim, vdim, n_q, n_k all multiples of 8) and
// rpt consecutive rows per block (QKV_RPT in long steps, fewer in short
// ones so that the launch still fills the chip) with the thread's taps in
// registers; w_t [taps, C] is a transposed copy of the taps.
constexpr int QKV_RPT = 8;
constexpr int QKV_MAX_TAPS = QKV_VEC_MAX_TAPS;

__global__ __launch_bounds__(256) void conv_qkv_cache_vec8_kernel(
    bf16* __restrict__ qo, const bf16* __restrict__ p, int64_t ldp,
    const float* __restrict__ w_t, const float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ seq_lens,
    const int* __restrict__ slots, const int* __restrict__ token_seq,
    const int64_t* __restrict__ positions, bf16* __restrict__ k_cache,
    bf16* __restrict__ v_cache, const int64_t* __restrict__ slot_mapping,
    int T, int rpt, QkvConvArgs a) {
  const int C = a.n_q + a.n_k + a.n_v;
  const int c = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (c >= C) return;
  float wv[QKV_MAX_TAPS][8];
#pragma unroll
  for (int j = 0; j < QKV_MAX_TAPS; ++j) {
    if (j < a.taps) {
      const float4v w0 = *reinterpret_cast<const float4v*>(w_t + (int64_t)j * C + c);
      const float4v w1 = *reinterpret_cast<const float4v*>(w_t + (int64_t)j * C + c + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { wv[j][e] = w0[e]; wv[j][4 + e] = w1[e]; }
    }
  }
  // where this thread's piece goes
  int kind, dst0;  // 0: q (index into the regrouped row), 1: k, 2: v
  int g = 0;
  if (c < a.n_q) {
    kind = 0;
    dst0 = query_dest(c, a);
  } else if (c < a.n_q + a.n_k) {
    kind = 1;
    g = (c - a.n_q) / a.kdim;
    dst0 = (c - a.n_q) % a.kdim;
  } else {
    kind = 2;
    g = (c - a.n_q - a.n_k) / a.vdim;
    dst0 = (c - a.n_q - a.n_k) % a.vdim;
  }
  const int t_end = min(T, (int)(blockIdx.x + 1) * rpt);
  for (int t = blockIdx.x * rpt; t < t_end; ++t) {
    const SeqRow r = seq_row(t, token_seq, cu, seq_lens, slots);
    const int i = t - r.first_row;
    const bool has_state = r.start > 0 && r.slot >= 0 && a.taps > 1;
    const float* hist =
        state ? state + (int64_t)(r.slot < 0 ? 0 : r.slot) * (a.taps - 1) * C
              : nullptr;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
#pragma unroll
    for (int j = 0; j < QKV_MAX_TAPS; ++j) {
      if (j < a.taps) {
        const int src = i - (a.taps - 1 - j);
        float xv[8];
        bool have = true;
        if (src >= 0) {
          const ushort8 v = *reinterpret_cast<const ushort8*>(
              p + (int64_t)(r.first_row + src) * ldp + c);
#pragma unroll
          for (int e = 0; e < 8; ++e) xv[e] = bf16_bits_to_float(v[e]);
        } else if (has_state) {
          const float* hp = hist + (int64_t)(src + a.taps - 1) * C + c;
          const float4v h0 = *reinterpret_cast<const float4v*>(hp);
          const float4v h1 = *reinterpret_cast<const float4v*>(hp + 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) { xv[e] = h0[e]; xv[4 + e] = h1[e]; }
        } else {
          have = false;
        }
        if (have) {
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[e] += wv[j][e] * xv[e];
        }
      }
    }
    ushort8 o;
    if (kind == 0) {
      const float qf = query_factor(positions[t], a.temp_coef, a.temp_every);
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = float_to_bf16_bits(acc[e] * qf);
      *reinterpret_cast<ushort8*>(qo + (int64_t)t * a.n_q + dst0) = o;
    } else {
      const int64_t slot = slot_mapping[t];
      if (slot < 0) continue;
      const int64_t blk = slot / a.block_size, off = slot % a.block_size;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = float_to_bf16_bits(acc[e]);
      if (kind == 1)
        *reinterpret_cast<ushort8*>(
            k_cache + ((blk * a.kv_heads + g) * a.block_size + off) * a.kdim +
            dst0) = o;
      else
        *reinterpret_cast<ushort8*>(
            v_cache + ((blk * a.kv_heads + g) * a.block_size + off) * a.vdim +
            dst0) = o;
    }
  }
}

// New history of a sequence = its last taps-1 inputs after this step: rows
// of this step where there are enough, older history shifted up otherwise.
// One thread per (sequence, channel) reads all it needs before it writes.
template <typename AT>
__global__ __launch_bounds__(256) void qkv_history_kernel(
    float* __restrict__ state, const AT* __restrict__ p, int64_t ldp,
    const int* __restrict__ cu, const int* __restrict__ seq_lens,
    const int* __restrict__ slots, int C, int taps) {
  const int s = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  const int a = cu[s], rows = cu[s + 1] - a;
  const int slot = slots[s];
  if (c >= C || rows == 0 || slot < 0) return;
  const int start = seq_lens[s] - rows;
  const int nh = taps - 1;
  float* hist = state + (int64_t)slot * nh * C + c;
  float nv[QKV_MAX_HIST];
#pragma unroll
  for (int i = 0; i < QKV_MAX_HIST; ++i) {
    if (i < nh) {
      const int src = rows - nh + i;  // index into this step's rows
      if (src >= 0)
        nv[i] = Act<AT>::ld(p + (int64_t)(a + src) * ldp + c);
      else
        nv[i] = start > 0 ? hist[(int64_t)(src + nh) * C] : 0.f;
    }
  }
#pragma unroll
  for (int i = 0; i < QKV_MAX_HIST; ++i)
    if (i < nh) hist[(int64_t)i * C] = nv[i];
}

// ------------------------------------------------------ difference heads
// One wave per (row, head): a [T, G, 2, R, V] holds map 0 and map 1 of
// head g * R + i at [t, g, 0, i] and [t, g, 1, i]. Values per lane:
// DIFF_VPT (V <= 64 * DIFF_VPT).
constexpr int DIFF_VPT = 8;

template <typename AT>
__global__ __launch_bounds__(256) void diff_head_norm_gate_kernel(
    AT* __restrict__ out, int64_t ldo, const AT* __restrict__ a,
    const AT* __restrict__ gate, int64_t ldg, float lam, float eps,
    float mult, int T, int H, int G, int V) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int64_t idx = (int64_t)blockIdx.x * 4 + wave;
  if (idx >= (int64_t)T * H) return;
  const int64_t t = idx / H;
  const int h = (int)(idx % H);
  const int R = H / G;
  const int g = h / R, i = h % R;
  const AT* a1 = a + (((t * G + g) * 2 + 0) * R + i) * V;
  const AT* a2 = a + (((t * G + g) * 2 + 1) * R + i) * V;
  float o[DIFF_VPT];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < DIFF_VPT; ++u) {
    const int d = lane + 64 * u;
    if (d < V) {
      o[u] = Act<AT>::ld(a1 + d) - lam * Act<AT>::ld(a2 + d);
      ss += o[u] * o[u];
    }
  }
  ss = wave_reduce_sum(ss);
  const float f = mult / sqrtf(ss / (float)V + eps);
  const AT* gr = gate + t * ldg + (int64_t)h * V;
  AT* orow = out + t * ldo + (int64_t)h * V;
#pragma unroll
  for (int u = 0; u < DIFF_VPT; ++u) {
    const int d = lane + 64 * u;
    if (d < V) Act<AT>::st(orow + d, o[u] * f * sigmoid_f(Act<AT>::ld(gr + d)));
  }
}

// bf16, 8 values per lane: a head is V / 8 neighbouring lanes (a power of
// two, at most 64), so a wave holds 512 / V heads and reduces inside each.
__global__ __launch_bounds__(256) void diff_head_norm_gate_vec8_kernel(
    bf16* __restrict__ out, int64_t ldo, const bf16* __restrict__ a,
    const bf16* __restrict__ gate, int64_t ldg, float lam, float eps,
    float mult, int64_t n_heads, int H, int G, int V) {
  const int L = V / 8;  // lanes per head
  const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) / L;
  const int d = (threadIdx.x % L) * 8;
  const bool live = idx < n_heads;
  const int64_t t = live ? idx / H : 0;
  const int h = live ? (int)(idx % H) : 0;
  const int R = H / G;
  const int g = h / R, i = h % R;
  float o[8];
  float ss = 0.f;
  if (live) {
    const ushort8 u1 = *reinterpret_cast<const ushort8*>(
        a + (((t * G + g) * 2 + 0) * R + i) * V + d);
    const ushort8 u2 = *reinterpret_cast<const ushort8*>(
        a + (((t * G + g) * 2 + 1) * R + i) * V + d);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      o[e] = bf16_bits_to_float(u1[e]) - lam * bf16_bits_to_float(u2[e]);
      ss += o[e] * o[e];
    }
  }
  for (int off = L / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, WAVE_SIZE);
  if (!live) return;
  const float f = mult / sqrtf(ss / (float)V + eps);
  const ushort8 gv =
      *reinterpret_cast<const ushort8*>(gate + t * ldg + (int64_t)h * V + d);
  ushort8 r;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float z = bf16_bits_to_float(gv[e]);
    r[e] = float_to_bf16_bits(o[e] * f / (1.f + __expf(-z)));
  }
  *reinterpret_cast<ushort8*>(out + t * ldo + (int64_t)h * V + d) = r;
}

// ------------------------------------------------------- expert activation
template <typename AT>
__global__ __launch_bounds__(256) void moe_glu_scaled_kernel(
    AT* __restrict__ out, const AT* __restrict__ gu, int64_t ldg,
    const float* __restrict__ scale, int64_t total, int E, int ff, int sff) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int F = E * ff + sff;
  const int64_t t = idx / F;
  const int c = (int)(idx % F);
  const AT* row = gu + t * ldg;
  float g, u;
  if (c < E * ff) {
    const int e = c / ff, i = c % ff;
    const float s = scale[t * E + e];
    if (s == 0.f) {  // an expert the row does not use: exactly nothing
      Act<AT>::st(out + idx, 0.f);
      return;
    }
    g = s * Act<AT>::ld(row + (int64_t)e * 2 * ff + i);
    u = s * Act<AT>::ld(row + (int64_t)e * 2 * ff + ff + i);
  } else {
    const int i = c - E * ff;
    g = Act<AT>::ld(row + (int64_t)E * 2 * ff + i);
    u = Act<AT>::ld(row + (int64_t)E * 2 * ff + sff + i);
  }
  Act<AT>::st(out + idx, silu_f(g) * u);
}

// bf16, 8 columns per thread (ff and sff multiples of 8)
__global__ __launch_bounds__(256) void moe_glu_scaled_vec8_kernel(
    bf16* __restrict__ out, const bf16* __restrict__ gu, int64_t ldg,
    const float* __restrict__ scale, int64_t total8, int E, int ff, int sff) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total8) return;
  const int F = E * ff + sff;
  const int F8 = F / 8;
  const int64_t t = idx / F8;
  const int c = (int)(idx % F8) * 8;
  const bf16* row = gu + t * ldg;
  float s = 1.f;
  const bf16 *gp, *up;
  if (c < E * ff) {
    const int e = c / ff, i = c % ff;
    s = scale[t * E + e];
    gp = row + (int64_t)e * 2 * ff + i;
    up = gp + ff;
  } else {
    const int i = c - E * ff;
    gp = row + (int64_t)E * 2 * ff + i;
    up = gp + sff;
  }
  ushort8 o;
  if (s == 0.f) {
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = 0;
  } else {
    const ushort8 gv = *reinterpret_cast<const ushort8*>(gp);
    const ushort8 uv = *reinterpret_cast<const ushort8*>(up);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float g = s * bf16_bits_to_float(gv[e]);
      const float u = s * bf16_bits_to_float(uv[e]);
      o[e] = float_to_bf16_bits(g / (1.f + __expf(-g)) * u);
    }
  }
  *reinterpret_cast<ushort8*>(out + t * F + c) = o;
}

}  // namespace arks

using namespace arks;

extern "C" void arks_seq_residual_pair_norm(
    void* x, void* h1, void* h2, const void* y1, const void* s1,
    const void* y2, const void* s2, const void* w1, const void* w2, float eps,
    int64_t T, int C, int act_f32, hipStream_t stream) {
  if (T == 0) return;
  if (!act_f32 && C % 8 == 0 && C <= 256 * 8 * PAIR_NORM_IT) {
    hipLaunchKernelGGL(residual_pair_norm_vec8_kernel, dim3((unsigned)T),
                       dim3(256), 0, stream, (float*)x, (bf16*)h1, (bf16*)h2,
                       (const bf16*)y1, (const float*)s1, (const bf16*)y2,
                       (const float*)s2, (const float*)w1, (const float*)w2,
                       eps, C);
    return;
  }
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (residual_pair_norm_kernel<AT>), dim3((unsigned)T), dim3(256), 0, stream,
      (float*)x, (AT*)h1, (AT*)h2, (const AT*)y1, (const float*)s1,
      (const AT*)y2, (const float*)s2, (const float*)w1, (const float*)w2, eps,
      C));
}

extern "C" int arks_seq_conv_qkv_cache(
    void* qo, const void* p, int64_t ldp, const void* w, const void* w_t,
    void* state, const void* cu, const void* seq_lens, const void* slots,
    const void* token_seq, const void* positions, void* k_cache,
    void* v_cache, const void* slot_mapping, int T, int S, int n_q, int n_k,
    int n_v, int heads, int kv_heads, int maps, int block_size, int taps,
    float temp_coef, int temp_every, int act_f32, hipStream_t stream) {
  if (taps - 1 > QKV_MAX_HIST || taps < 1) return 1;
  if (T == 0) return 0;
  QkvConvArgs a;
  a.n_q = n_q; a.n_k = n_k; a.n_v = n_v;
  a.heads = heads; a.kv_heads = kv_heads; a.maps = maps;
  a.dim = n_q / (heads * maps);
  a.kdim = n_k / kv_heads; a.vdim = n_v / kv_heads;
  a.block_size = block_size; a.taps = taps;
  a.temp_coef = temp_coef; a.temp_every = temp_every;
  const int C = n_q + n_k + n_v;
  const int cb = (C + 255) / 256;
  const bool vec8 = !act_f32 && w_t && taps <= QKV_VEC_MAX_TAPS &&
                    ldp % 8 == 0 &&
                    ((uintptr_t)p % 16) == 0 && a.dim % 8 == 0 &&
                    a.kdim % 8 == 0 && a.vdim % 8 == 0;
  // rows per block: as many as leave about 1024 blocks
  const int cb8 = (C / 8 + 255) / 256;
  int rpt = (int)(((int64_t)T * cb8) / 1024);
  rpt = rpt < 1 ? 1 : (rpt > QKV_RPT ? QKV_RPT : rpt);
  SEQ_DISPATCH_ACT(act_f32, {
    if (vec8)
      hipLaunchKernelGGL(conv_qkv_cache_vec8_kernel,
                         dim3((T + rpt - 1) / rpt, cb8),
                         dim3(256), 0, stream, (bf16*)qo, (const bf16*)p, ldp,
                         (const float*)w_t, (const float*)state,
                         (const int*)cu, (const int*)seq_lens,
                         (const int*)slots, (const int*)token_seq,
                         (const int64_t*)positions, (bf16*)k_cache,
                         (bf16*)v_cache, (const int64_t*)slot_mapping, T, rpt,
                         a);
    else
      hipLaunchKernelGGL((conv_qkv_cache_kernel<AT>), dim3(T, cb), dim3(256),
                         0, stream, (AT*)qo, (const AT*)p, ldp,
                         (const float*)w, (const float*)state, (const int*)cu,
                         (const int*)seq_lens, (const int*)slots,
                         (const int*)token_seq, (const int64_t*)positions,
                         (AT*)k_cache, (AT*)v_cache,
                         (const int64_t*)slot_mapping, a);
    if (taps > 1)
      hipLaunchKernelGGL((qkv_history_kernel<AT>), dim3(S, cb), dim3(256), 0,
                         stream, (float*)state, (const AT*)p, ldp,
                         (const int*)cu, (const int*)seq_lens,
                         (const int*)slots, C, taps);
  });
  return 0;
}

extern "C" int arks_seq_diff_head_norm_gate(
    void* out, int64_t ldo, const void* a, const void* gate, int64_t ldg,
    float lam, float eps, float mult, int T, int H, int G, int V, int act_f32,
    hipStream_t stream) {
  if (V > 64 * DIFF_VPT) return 1;
  if (T == 0) return 0;
  const int64_t n = (int64_t)T * H;
  const int L = V / 8;
  if (!act_f32 && V % 8 == 0 && L <= 64 && (L & (L - 1)) == 0 &&
      ldo % 8 == 0 && ldg % 8 == 0 && ((uintptr_t)out & 15) == 0 &&
      ((uintptr_t)gate & 15) == 0 && ((uintptr_t)a & 15) == 0) {
    const int64_t threads = n * L;
    hipLaunchKernelGGL(diff_head_norm_gate_vec8_kernel,
                       dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                       stream, (bf16*)out, ldo, (const bf16*)a,
                       (const bf16*)gate, ldg, lam, eps, mult, n, H, G, V);
    return 0;
  }
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (diff_head_norm_gate_kernel<AT>), dim3((unsigned)((n + 3) / 4)),
      dim3(256), 0, stream, (AT*)out, ldo, (const AT*)a, (const AT*)gate, ldg,
      lam, eps, mult, T, H, G, V));
  return 0;
}

extern "C" void arks_seq_moe_glu_scaled(void* out, const void* gu, int64_t ldg,
                                        const void* scale, int64_t T, int E,
                                        int ff, int sff, int act_f32,
                                        hipStream_t stream) {
  if (T == 0) return;
  const int64_t total = T * ((int64_t)E * ff + sff);
  if (!act_f32 && ff % 8 == 0 && sff % 8 == 0 && ldg % 8 == 0 &&
      ((uintptr_t)gu % 16) == 0) {
    const int64_t total8 = total / 8;
    hipLaunchKernelGGL(moe_glu_scaled_vec8_kernel,
                       dim3((unsigned)((total8 + 255) / 256)), dim3(256), 0,
                       stream, (bf16*)out, (const bf16*)gu, ldg,
                       (const float*)scale, total8, E, ff, sff);
    return;
  }
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (moe_glu_scaled_kernel<AT>), dim3((unsigned)((total + 255) / 256)),
      dim3(256), 0, stream, (AT*)out, (const AT*)gu, ldg, (const float*)scale,
      total, E, ff, sff));
}
