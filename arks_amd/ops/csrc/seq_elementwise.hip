// Row-wise kernels around the fp32 residual stream of the layer-list
// decoders: token shift, gated output norm + residual add, final norm,
// gated RMS norm, tanh-GELU, and the attention front end (per-head q/k RMS
// norm, rotary, position-turned values, paged cache write).
#include "seq_common.h"

namespace arks {

// xs[t] = x[t] + (x[t-1] - x[t]) * w, x[-1] = the sequence's stored last
// row (or 0 at position 0). The block of a sequence's FIRST row is the only
// reader of the stored row, and the one that replaces it with the last row
// of this step — same thread, read before write, so no ordering between
// blocks is needed.
template <typename AT>
__global__ __launch_bounds__(256) void token_shift_kernel(
    AT* __restrict__ xs, AT* __restrict__ xa, const float* __restrict__ x,
    const float* __restrict__ w, float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ seq_lens,
    const int* __restrict__ slots, const int* __restrict__ token_seq, int W) {
  const int t = blockIdx.x;
  const SeqRow r = seq_row(t, token_seq, cu, seq_lens, slots);
  const bool first = (t == r.first_row);
  const bool has_state = r.start > 0 && r.slot >= 0;
  const float* xr = x + (int64_t)t * W;
  const float* xp = x + (int64_t)(t - 1) * W;
  const float* xl = x + (int64_t)(r.first_row + r.rows - 1) * W;
  float* st = state + (int64_t)(r.slot < 0 ? 0 : r.slot) * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float xv = xr[i];
    const float prev = first ? (has_state ? st[i] : 0.f) : xp[i];
    Act<AT>::st(xs + (int64_t)t * W + i, xv + (prev - xv) * w[i]);
    if (xa) Act<AT>::st(xa + (int64_t)t * W + i, xv);
    if (first && r.slot >= 0) st[i] = xl[i];
  }
}

// x += rmsnorm(y * sigmoid(g + gb)) * w ; optional cast copy of the new x.
template <typename AT>
__global__ __launch_bounds__(256) void gated_norm_residual_kernel(
    float* __restrict__ x, AT* __restrict__ xa, const AT* __restrict__ y,
    const AT* __restrict__ g, int64_t ldg, const float* __restrict__ gb,
    const float* __restrict__ w, float eps, int W) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  const AT* yr = y + (int64_t)t * W;
  const AT* gr = g ? g + (int64_t)t * ldg : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    float z = Act<AT>::ld(yr + i);
    if (gr) z *= sigmoid_f(Act<AT>::ld(gr + i) + gb[i]);
    ss += z * z;
  }
  ss = block_reduce_sum<256>(ss, scratch);
  const float rstd = 1.f / sqrtf(ss / (float)W + eps);
  float* xr = x + (int64_t)t * W;
  for (int i = threadIdx.x; i < W; i += 256) {
    float z = Act<AT>::ld(yr + i);
    if (gr) z *= sigmoid_f(Act<AT>::ld(gr + i) + gb[i]);
    const float nx = xr[i] + z * rstd * w[i];
    xr[i] = nx;
    if (xa) Act<AT>::st(xa + (int64_t)t * W + i, nx);
  }
}

// bf16 rows, 8 elements per thread and iteration, the gated values kept in
// registers between the two passes (W <= 8 * 256 * GNR_VPT).
constexpr int GNR_VPT = 4;

__global__ __launch_bounds__(256) void gated_norm_residual_vec8_kernel(
    float* __restrict__ x, bf16* __restrict__ xa, const bf16* __restrict__ y,
    const bf16* __restrict__ g, int64_t ldg, const float* __restrict__ gb,
    const float* __restrict__ w, float eps, int W) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  const bf16* yr = y + (int64_t)t * W;
  const bf16* gr = g ? g + (int64_t)t * ldg : nullptr;
  float z[GNR_VPT][8];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < GNR_VPT; ++k) {
    const int i = (k * 256 + threadIdx.x) * 8;
    if (i < W) {
      const ushort8 yv = *reinterpret_cast<const ushort8*>(yr + i);
#pragma unroll
      for (int e = 0; e < 8; ++e) z[k][e] = bf16_bits_to_float(yv[e]);
      if (gr) {
        const ushort8 gv = *reinterpret_cast<const ushort8*>(gr + i);
        const float4v b0 = *reinterpret_cast<const float4v*>(gb + i);
        const float4v b1 = *reinterpret_cast<const float4v*>(gb + i + 4);
#pragma unroll
        for (int e = 0; e < 8; ++e)
          z[k][e] *= sigmoid_f(bf16_bits_to_float(gv[e]) + (e < 4 ? b0[e] : b1[e - 4]));
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += z[k][e] * z[k][e];
    }
  }
  ss = block_reduce_sum<256>(ss, scratch);
  const float rstd = 1.f / sqrtf(ss / (float)W + eps);
  float* xr = x + (int64_t)t * W;
#pragma unroll
  for (int k = 0; k < GNR_VPT; ++k) {
    const int i = (k * 256 + threadIdx.x) * 8;
    if (i < W) {
      float4v x0 = *reinterpret_cast<const float4v*>(xr + i);
      float4v x1 = *reinterpret_cast<const float4v*>(xr + i + 4);
      const float4v w0 = *reinterpret_cast<const float4v*>(w + i);
      const float4v w1 = *reinterpret_cast<const float4v*>(w + i + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        x0[e] += z[k][e] * rstd * w0[e];
        x1[e] += z[k][4 + e] * rstd * w1[e];
      }
      *reinterpret_cast<float4v*>(xr + i) = x0;
      *reinterpret_cast<float4v*>(xr + i + 4) = x1;
      if (xa) {
        ushort8 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          o[e] = float_to_bf16_bits(x0[e]);
          o[4 + e] = float_to_bf16_bits(x1[e]);
        }
        *reinterpret_cast<ushort8*>(xa + (int64_t)t * W + i) = o;
      }
    }
  }
}

// token shift, bf16 outputs, 8 elements per thread (W % 8 == 0)
__global__ __launch_bounds__(256) void token_shift_vec8_kernel(
    bf16* __restrict__ xs, bf16* __restrict__ xa, const float* __restrict__ x,
    const float* __restrict__ w, float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ seq_lens,
    const int* __restrict__ slots, const int* __restrict__ token_seq, int W) {
  const int t = blockIdx.x;
  const SeqRow r = seq_row(t, token_seq, cu, seq_lens, slots);
  const bool first = (t == r.first_row);
  const bool has_state = r.start > 0 && r.slot >= 0;
  const float* xr = x + (int64_t)t * W;
  const float* xp = first ? (state + (int64_t)(r.slot < 0 ? 0 : r.slot) * W)
                          : x + (int64_t)(t - 1) * W;
  const bool zero_prev = first && !has_state;
  const float* xl = x + (int64_t)(r.first_row + r.rows - 1) * W;
  for (int i = threadIdx.x * 8; i < W; i += 256 * 8) {
    ushort8 os, oa;
#pragma unroll
    for (int hlf = 0; hlf < 2; ++hlf) {
      const int j = i + 4 * hlf;
      const float4v xv = *reinterpret_cast<const float4v*>(xr + j);
      float4v pv = {0.f, 0.f, 0.f, 0.f};
      if (!zero_prev) pv = *reinterpret_cast<const float4v*>(xp + j);
      const float4v wv = *reinterpret_cast<const float4v*>(w + j);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        os[4 * hlf + e] = float_to_bf16_bits(xv[e] + (pv[e] - xv[e]) * wv[e]);
        oa[4 * hlf + e] = float_to_bf16_bits(xv[e]);
      }
      if (first && r.slot >= 0)
        *reinterpret_cast<float4v*>(state + (int64_t)r.slot * W + j) =
            *reinterpret_cast<const float4v*>(xl + j);
    }
    *reinterpret_cast<ushort8*>(xs + (int64_t)t * W + i) = os;
    *reinterpret_cast<ushort8*>(xa + (int64_t)t * W + i) = oa;
  }
}

// out = rmsnorm(x) * w [* sigmoid(gate)], x fp32.
template <typename AT>
__global__ __launch_bounds__(256) void rms_norm_f32_kernel(
    AT* __restrict__ out, const float* __restrict__ x,
    const float* __restrict__ w, const AT* __restrict__ gate, int64_t ldg,
    float eps, int W) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  const float* xr = x + (int64_t)t * W;
  // the first 16 * 256 elements of the row stay in registers between the
  // two passes; longer rows re-read their tail
  constexpr int KEEP = 16;
  float xv[KEEP];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < KEEP; ++u) {
    const int i = threadIdx.x + 256 * u;
    xv[u] = i < W ? xr[i] : 0.f;
    ss += xv[u] * xv[u];
  }
  for (int i = threadIdx.x + 256 * KEEP; i < W; i += 256) ss += xr[i] * xr[i];
  ss = block_reduce_sum<256>(ss, scratch);
  const float rstd = 1.f / sqrtf(ss / (float)W + eps);
#pragma unroll
  for (int u = 0; u < KEEP; ++u) {
    const int i = threadIdx.x + 256 * u;
    if (i < W) {
      float v = xv[u] * rstd * w[i];
      if (gate) v *= sigmoid_f(Act<AT>::ld(gate + (int64_t)t * ldg + i));
      Act<AT>::st(out + (int64_t)t * W + i, v);
    }
  }
  for (int i = threadIdx.x + 256 * KEEP; i < W; i += 256) {
    float v = xr[i] * rstd * w[i];
    if (gate) v *= sigmoid_f(Act<AT>::ld(gate + (int64_t)t * ldg + i));
    Act<AT>::st(out + (int64_t)t * W + i, v);
  }
}

template <typename AT>
__global__ __launch_bounds__(256) void gelu_tanh_kernel(
    AT* __restrict__ out, const AT* __restrict__ x, int64_t ldx, int64_t rows,
    int n) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= rows * n) return;
  const int64_t r = idx / n;
  const int c = (int)(idx - r * n);
  const float z = Act<AT>::ld(x + r * ldx + c);
  const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
  Act<AT>::st(out + idx, 0.5f * z * (1.f + tanhf(u)));
}

// bf16, 8 elements per thread; tanh(u) = 1 - 2 / (1 + e^(2u)) with the
// hardware exponential (saturates cleanly at both ends)
__global__ __launch_bounds__(256) void gelu_tanh_vec8_kernel(
    bf16* __restrict__ out, const bf16* __restrict__ x, int64_t ldx,
    int64_t rows, int n8) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= rows * n8) return;
  const int64_t r = idx / n8;
  const int c = (int)(idx - r * n8) * 8;
  const ushort8 v = *reinterpret_cast<const ushort8*>(x + r * ldx + c);
  ushort8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float z = bf16_bits_to_float(v[e]);
    const float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
    const float th = 1.f - 2.f / (1.f + __expf(2.f * u));
    o[e] = float_to_bf16_bits(0.5f * z * (1.f + th));
  }
  *reinterpret_cast<ushort8*>(out + r * (int64_t)n8 * 8 + c) = o;
}

// One block per row: the row's rotary angles (they depend on the position
// and the pair only) are evaluated once into LDS, then the block's waves
// walk the head slots — [0,H) query heads, [H,H+G) key heads, [H+G,H+2G)
// value heads. q/k: RMS norm over the head (weight or none) then rotary on
// the first 2*n_rot dims, cos and sin times rot_mag, then (norm_after) the
// head divided by its root mean square once more, without a weight; v:
// turned by the row's position over all its dims (n_vrot pairs; 0 = stored
// plain). Pairs are (2i,2i+1) when interleaved, (i, i+n) otherwise. k and v
// go to their page.
constexpr int ROPE_MAX_PAIRS = 256;

template <typename AT>
__global__ __launch_bounds__(256) void qk_norm_rope_cache_kernel(
    AT* __restrict__ qo, const AT* __restrict__ q, const AT* __restrict__ k,
    const AT* __restrict__ v, int64_t ldq, int64_t ldk, int64_t ldv,
    const float* __restrict__ qw, const float* __restrict__ kw, float eps,
    const int64_t* __restrict__ positions, const float* __restrict__ freq_qk,
    int n_rot, const float* __restrict__ freq_v, int n_vrot,
    AT* __restrict__ k_cache, AT* __restrict__ v_cache,
    const int64_t* __restrict__ slot_mapping, int H, int G, int D, int V,
    int block_size, int interleaved, float rot_mag, int norm_after) {
  __shared__ float cs_qk[ROPE_MAX_PAIRS][2];
  __shared__ float cs_v[ROPE_MAX_PAIRS][2];
  const int t = blockIdx.x;
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < n_rot; i += 256) {
    float sn, cs;
    sincosf(pos * freq_qk[i], &sn, &cs);
    cs_qk[i][0] = cs * rot_mag;
    cs_qk[i][1] = sn * rot_mag;
  }
  for (int i = threadIdx.x; i < n_vrot; i += 256)
    sincosf(pos * freq_v[i], &cs_v[i][1], &cs_v[i][0]);
  __syncthreads();
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int64_t slot = slot_mapping[t];
  for (int hs = wave; hs < H + 2 * G; hs += 4) {
    const AT* src;
    AT* dst;
    const float* nw = nullptr;
    const float(*cs)[2];
    int n, npairs;
    if (hs < H) {
      src = q + (int64_t)t * ldq + (int64_t)hs * D;
      dst = qo + ((int64_t)t * H + hs) * D;
      n = D; npairs = n_rot; cs = cs_qk; nw = qw;
    } else {
      if (slot < 0) continue;
      const int64_t blk = slot / block_size, off = slot % block_size;
      if (hs < H + G) {
        const int g = hs - H;
        src = k + (int64_t)t * ldk + (int64_t)g * D;
        dst = k_cache + ((blk * G + g) * block_size + off) * D;
        n = D; npairs = n_rot; cs = cs_qk; nw = kw;
      } else {
        const int g = hs - H - G;
        src = v + (int64_t)t * ldv + (int64_t)g * V;
        dst = v_cache + ((blk * G + g) * block_size + off) * V;
        n = V; npairs = n_vrot; cs = cs_v;
      }
    }
    const bool normed = nw != nullptr;
    const bool after = norm_after && hs < H + G;
    // the head is read once: this lane's pairs stay in registers between
    // the sum of squares and the rotation (npairs <= 64 * 4)
    float pa[ROPE_MAX_PAIRS / 64], pb[ROPE_MAX_PAIRS / 64];
    float ss = 0.f;
#pragma unroll
    for (int u = 0; u < ROPE_MAX_PAIRS / 64; ++u) {
      const int i = lane + 64 * u;
      if (i < npairs) {
        pa[u] = Act<AT>::ld(src + (interleaved ? 2 * i : i));
        pb[u] = Act<AT>::ld(src + (interleaved ? 2 * i + 1 : i + npairs));
        ss += pa[u] * pa[u] + pb[u] * pb[u];
      }
    }
    float rstd = 1.f;
    if (normed) {
      for (int i = 2 * npairs + lane; i < n; i += 64) {
        const float a = Act<AT>::ld(src + i);
        ss += a * a;
      }
      ss = wave_reduce_sum(ss);
      rstd = 1.f / sqrtf(ss / (float)n + eps);
    }
    // the turned pairs replace the plain ones in the registers
    float ss2 = 0.f;
#pragma unroll
    for (int u = 0; u < ROPE_MAX_PAIRS / 64; ++u) {
      const int i = lane + 64 * u;
      if (i < npairs) {
        const int d0 = interleaved ? 2 * i : i;
        const int d1 = interleaved ? 2 * i + 1 : i + npairs;
        float a = pa[u] * rstd, b = pb[u] * rstd;
        if (normed) { a *= nw[d0]; b *= nw[d1]; }
        const float c = cs[i][0], sn = cs[i][1];
        pa[u] = a * c - b * sn;
        pb[u] = b * c + a * sn;
        ss2 += pa[u] * pa[u] + pb[u] * pb[u];
      }
    }
    float rstd2 = 1.f;
    if (after) {
      for (int i = 2 * npairs + lane; i < n; i += 64) {
        float a = Act<AT>::ld(src + i) * rstd;
        if (normed) a *= nw[i];
        ss2 += a * a;
      }
      ss2 = wave_reduce_sum(ss2);
      rstd2 = 1.f / sqrtf(ss2 / (float)n + eps);
    }
#pragma unroll
    for (int u = 0; u < ROPE_MAX_PAIRS / 64; ++u) {
      const int i = lane + 64 * u;
      if (i < npairs) {
        const int d0 = interleaved ? 2 * i : i;
        const int d1 = interleaved ? 2 * i + 1 : i + npairs;
        Act<AT>::st(dst + d0, pa[u] * rstd2);
        Act<AT>::st(dst + d1, pb[u] * rstd2);
      }
    }
    for (int i = 2 * npairs + lane; i < n; i += 64) {
      float a = Act<AT>::ld(src + i) * rstd;
      if (normed) a *= nw[i];
      Act<AT>::st(dst + i, a * rstd2);
    }
  }
}

// bf16 rows, half-split pairs, values stored plain, D / 8 lanes per head
// slot (a power of two, at most 64; V <= D), 8 dims per lane with 16-byte
// accesses: the same work as qk_norm_rope_cache_kernel, one block per row,
// the row's cos / sin (times rot_mag) once in LDS. A pair's two dims sit
// n_rot apart, i.e. n_rot / 8 lanes apart (n_rot % 8 == 0): the partner's
// values come by shuffle. Sums of squares are reduced inside a head's lanes.
__global__ __launch_bounds__(256) void qk_norm_rope_cache_vec8_kernel(
    bf16* __restrict__ qo, const bf16* __restrict__ q,
    const bf16* __restrict__ k, const bf16* __restrict__ v, int64_t ldq,
    int64_t ldk, int64_t ldv, const float* __restrict__ qw,
    const float* __restrict__ kw, float eps,
    const int64_t* __restrict__ positions, const float* __restrict__ freq_qk,
    int n_rot, bf16* __restrict__ k_cache, bf16* __restrict__ v_cache,
    const int64_t* __restrict__ slot_mapping, int H, int G, int D, int V,
    int block_size, float rot_mag, int norm_after) {
  __shared__ float cs_qk[ROPE_MAX_PAIRS][2];
  const int t = blockIdx.x;
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < n_rot; i += 256) {
    float sn, cs;
    sincosf(pos * freq_qk[i], &sn, &cs);
    cs_qk[i][0] = cs * rot_mag;
    cs_qk[i][1] = sn * rot_mag;
  }
  __syncthreads();
  const int L = D / 8;
  const int sub = threadIdx.x % L;          // lane inside the head
  const int d0 = sub * 8;
  const int per_pass = 256 / L;
  const int lane = threadIdx.x % WAVE_SIZE;
  const int hop = n_rot / 8;                // lanes between a pair's dims
  const int64_t slot = slot_mapping[t];
  const int n_slots = H + 2 * G;
  for (int hs0 = 0; hs0 < n_slots; hs0 += per_pass) {
    const int hs = hs0 + threadIdx.x / L;
    const bool live = hs < n_slots;
    const bf16* src = nullptr;
    bf16* dst = nullptr;
    const float* nw = nullptr;
    bool is_v = false;
    if (live) {
      if (hs < H) {
        src = q + (int64_t)t * ldq + (int64_t)hs * D;
        dst = qo + ((int64_t)t * H + hs) * D;
        nw = qw;
      } else if (slot >= 0) {
        const int64_t blk = slot / block_size, off = slot % block_size;
        if (hs < H + G) {
          const int g = hs - H;
          src = k + (int64_t)t * ldk + (int64_t)g * D;
          dst = k_cache + ((blk * G + g) * block_size + off) * D;
          nw = kw;
        } else {
          const int g = hs - H - G;
          is_v = true;
          if (d0 < V) {
            src = v + (int64_t)t * ldv + (int64_t)g * V;
            dst = v_cache + ((blk * G + g) * block_size + off) * V;
          }
        }
      }
    }
    float x[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = 0.f;
    if (src) {
      const ushort8 u = *reinterpret_cast<const ushort8*>(src + d0);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = bf16_bits_to_float(u[e]);
    }
    if (is_v) {  // values pass as they are (every lane still joins the shuffles)
      if (src) {
        const ushort8 u = *reinterpret_cast<const ushort8*>(src + d0);
        *reinterpret_cast<ushort8*>(dst + d0) = u;
      }
      src = nullptr;
    }
    if (qw != nullptr) {  // norm with a weight in front of the turn
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
      for (int off = L / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, WAVE_SIZE);
      const float rstd = 1.f / sqrtf(ss / (float)D + eps);
      if (nw) {
#pragma unroll
        for (int e = 0; e < 8; ++e) x[e] *= rstd * nw[d0 + e];
      }
    }
    if (n_rot > 0) {
      const bool first = d0 < n_rot, second = !first && d0 < 2 * n_rot;
      const int partner = first ? lane + hop : lane - hop;
      float y[8];
#pragma unroll
      for (int e = 0; e < 8; ++e)
        y[e] = __shfl(x[e], (first || second) ? partner : lane, WAVE_SIZE);
      if (first || second) {
        const int i0 = first ? d0 : d0 - n_rot;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float c = cs_qk[i0 + e][0], sn = cs_qk[i0 + e][1];
          x[e] = first ? x[e] * c - y[e] * sn : x[e] * c + y[e] * sn;
        }
      }
    }
    if (norm_after) {
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
      for (int off = L / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, WAVE_SIZE);
      const float rstd = 1.f / sqrtf(ss / (float)D + eps);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] *= rstd;
    }
    if (src) {
      ushort8 o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = float_to_bf16_bits(x[e]);
      *reinterpret_cast<ushort8*>(dst + d0) = o;
    }
  }
}

// Turn every head row of out [T, H, V] back by its row's position: pair m
// by -pos * freq[m] (the cache holds values turned forward by their own
// positions, so the weighted sum comes out in the query's frame). One block
// per row, the angles evaluated once for all heads.
template <typename AT>
__global__ __launch_bounds__(256) void unrotate_rows_kernel(
    AT* __restrict__ out, const int64_t* __restrict__ positions,
    const float* __restrict__ freq, int H, int V, int interleaved) {
  __shared__ float cs[ROPE_MAX_PAIRS][2];
  const int t = blockIdx.x;
  const float pos = (float)positions[t];
  const int npairs = V / 2;
  for (int i = threadIdx.x; i < npairs; i += 256)
    sincosf(-pos * freq[i], &cs[i][1], &cs[i][0]);
  __syncthreads();
  for (int e = threadIdx.x; e < H * npairs; e += 256) {
    const int h = e / npairs, i = e - h * npairs;
    AT* row = out + ((int64_t)t * H + h) * V;
    const int d0 = interleaved ? 2 * i : i;
    const int d1 = interleaved ? 2 * i + 1 : i + npairs;
    const float a = Act<AT>::ld(row + d0), b = Act<AT>::ld(row + d1);
    Act<AT>::st(row + d0, a * cs[i][0] - b * cs[i][1]);
    Act<AT>::st(row + d1, b * cs[i][0] + a * cs[i][1]);
  }
}

}  // namespace arks

using namespace arks;

extern "C" int arks_seq_unrotate_rows(void* out, const void* positions,
                                      const void* freq, int T, int H, int V,
                                      int interleaved, int act_f32,
                                      hipStream_t stream) {
  if (V / 2 > ROPE_MAX_PAIRS) return 1;
  if (T == 0) return 0;
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (unrotate_rows_kernel<AT>), dim3(T), dim3(256), 0, stream, (AT*)out,
      (const int64_t*)positions, (const float*)freq, H, V, interleaved));
  return 0;
}

extern "C" void arks_seq_token_shift(void* xs, void* xa, const void* x,
                                     const void* w, void* state, const void* cu,
                                     const void* seq_lens, const void* slots,
                                     const void* token_seq, int T, int W,
                                     int act_f32, hipStream_t stream) {
  if (T == 0) return;
  if (!act_f32 && xa && W % 8 == 0) {
    hipLaunchKernelGGL(token_shift_vec8_kernel, dim3(T), dim3(256), 0, stream,
                       (bf16*)xs, (bf16*)xa, (const float*)x, (const float*)w,
                       (float*)state, (const int*)cu, (const int*)seq_lens,
                       (const int*)slots, (const int*)token_seq, W);
    return;
  }
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (token_shift_kernel<AT>), dim3(T), dim3(256), 0, stream, (AT*)xs,
      (AT*)xa, (const float*)x, (const float*)w, (float*)state, (const int*)cu,
      (const int*)seq_lens, (const int*)slots, (const int*)token_seq, W));
}

extern "C" void arks_seq_gated_norm_residual(void* x, void* xa, const void* y,
                                             const void* g, int64_t ldg,
                                             const void* gb, const void* w,
                                             float eps, int T, int W,
                                             int act_f32, hipStream_t stream) {
  if (T == 0) return;
  if (!act_f32 && W % 8 == 0 && W <= 8 * 256 * GNR_VPT && ldg % 8 == 0 &&
      ((uintptr_t)g % 16) == 0) {
    hipLaunchKernelGGL(gated_norm_residual_vec8_kernel, dim3(T), dim3(256), 0,
                       stream, (float*)x, (bf16*)xa, (const bf16*)y,
                       (const bf16*)g, ldg, (const float*)gb, (const float*)w,
                       eps, W);
    return;
  }
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (gated_norm_residual_kernel<AT>), dim3(T), dim3(256), 0, stream,
      (float*)x, (AT*)xa, (const AT*)y, (const AT*)g, ldg, (const float*)gb,
      (const float*)w, eps, W));
}

extern "C" void arks_seq_rms_norm_f32(void* out, const void* x, const void* w,
                                      const void* gate, int64_t ldg, float eps,
                                      int T, int W, int act_f32,
                                      hipStream_t stream) {
  if (T == 0) return;
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (rms_norm_f32_kernel<AT>), dim3(T), dim3(256), 0, stream, (AT*)out,
      (const float*)x, (const float*)w, (const AT*)gate, ldg, eps, W));
}

extern "C" void arks_seq_gelu_tanh(void* out, const void* x, int64_t ldx,
                                   int64_t rows, int n, int act_f32,
                                   hipStream_t stream) {
  const int64_t total = rows * n;
  if (total == 0) return;
  if (!act_f32 && n % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0) {
    hipLaunchKernelGGL(gelu_tanh_vec8_kernel,
                       dim3((unsigned)((total / 8 + 255) / 256)), dim3(256), 0,
                       stream, (bf16*)out, (const bf16*)x, ldx, rows, n / 8);
    return;
  }
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (gelu_tanh_kernel<AT>), dim3((unsigned)((total + 255) / 256)), dim3(256),
      0, stream, (AT*)out, (const AT*)x, ldx, rows, n));
}

extern "C" int arks_seq_qk_norm_rope_cache(
    void* qo, const void* q, const void* k, const void* v, int64_t ldq,
    int64_t ldk, int64_t ldv, const void* qw, const void* kw, float eps,
    const void* positions, const void* freq_qk, int n_rot, const void* freq_v,
    int n_vrot, void* k_cache, void* v_cache, const void* slot_mapping, int T,
    int H, int G, int D, int V, int block_size, int interleaved, int act_f32,
    float rot_mag, int norm_after, hipStream_t stream) {
  if (n_rot > ROPE_MAX_PAIRS || n_vrot > ROPE_MAX_PAIRS) return 1;
  if (T == 0) return 0;
  const int L = D / 8;
  if (!act_f32 && !interleaved && n_vrot == 0 && D % 8 == 0 && V % 8 == 0 &&
      V <= D && L <= 64 && (L & (L - 1)) == 0 && n_rot % 8 == 0 &&
      ldq % 8 == 0 && ldk % 8 == 0 && ldv % 8 == 0 &&
      (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)qo |
        (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0) {
    hipLaunchKernelGGL(
        qk_norm_rope_cache_vec8_kernel, dim3(T), dim3(256), 0, stream,
        (bf16*)qo, (const bf16*)q, (const bf16*)k, (const bf16*)v, ldq, ldk,
        ldv, (const float*)qw, (const float*)kw, eps,
        (const int64_t*)positions, (const float*)freq_qk, n_rot,
        (bf16*)k_cache, (bf16*)v_cache, (const int64_t*)slot_mapping, H, G, D,
        V, block_size, rot_mag, norm_after);
    return 0;
  }
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (qk_norm_rope_cache_kernel<AT>), dim3(T), dim3(256), 0, stream,
      (AT*)qo, (const AT*)q, (const AT*)k, (const AT*)v, ldq, ldk, ldv,
      (const float*)qw, (const float*)kw, eps, (const int64_t*)positions,
      (const float*)freq_qk, n_rot, (const float*)freq_v, n_vrot, (AT*)k_cache,
      (AT*)v_cache, (const int64_t*)slot_mapping, H, G, D, V, block_size,
      interleaved, rot_mag, norm_after));
  return 0;
}
