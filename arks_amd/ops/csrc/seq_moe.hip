// Expert routing and mixing for the layer-list decoders' sparse
// feed-forward (arks_amd/models/feedforward.py GroupedMoE), bf16 or float
// rows.
//
//   moe_route_grouped  scores over all E experts in fp32, their softmax or
//       (sigmoid) each logit's own sigmoid; experts are cut into
//       `groups` contiguous runs of E/groups, a run's score is its highest
//       expert score and only the `keep` highest-scoring runs stay eligible; the `top`
//       largest scores among those, divided by their sum (+1e-20) unless
//       renorm is off. Ties go to the lower index (groups and experts).
//       matrix (optional, [T, E]): the row's weights at the experts it uses,
//       0 elsewhere.
//   moe_mix_rows  out[t] = sum_j w[t][j] * y[row(t, j)], row given, or
//       ids[t][j] * T + t for dense per-expert outputs y [E, T, H].
#include "seq_common.h"

#include <cfloat>

namespace arks {

constexpr int ROUTE_MAX_E = 1024;
constexpr int ROUTE_MAX_K = 32;

// One wave per row.
__global__ __launch_bounds__(64) void moe_route_grouped_kernel(
    float* __restrict__ weights, int* __restrict__ ids,
    const float* __restrict__ logits, int E, int top, int groups, int keep,
    int sigmoid, int renorm, float* __restrict__ matrix) {
  __shared__ float s_s[ROUTE_MAX_E];
  __shared__ float g_s[ROUTE_MAX_E];  // group scores (groups <= E)
  const int t = blockIdx.x, lane = threadIdx.x;
  const float* row = logits + (int64_t)t * E;
  if (sigmoid) {
    for (int e = lane; e < E; e += 64) s_s[e] = sigmoid_f(row[e]);
  } else {
    float m = -FLT_MAX;
    for (int e = lane; e < E; e += 64) m = fmaxf(m, row[e]);
    m = wave_reduce_max(m);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) {
      const float p = expf(row[e] - m);
      s_s[e] = p;
      sum += p;
    }
    sum = wave_reduce_sum(sum);
    __syncthreads();
    const float inv = 1.f / sum;
    for (int e = lane; e < E; e += 64) s_s[e] *= inv;
  }
  if (matrix)
    for (int e = lane; e < E; e += 64) matrix[(int64_t)t * E + e] = 0.f;
  __syncthreads();
  const int per = E / groups;
  for (int gI = lane; gI < groups; gI += 64) {
    float best = -1.f;
    for (int i = 0; i < per; ++i) best = fmaxf(best, s_s[gI * per + i]);
    g_s[gI] = best;
  }
  __syncthreads();
  // the eligible runs: `keep` argmax passes, the others' experts are
  // marked unavailable (score -1)
  if (keep < groups) {
    for (int r = 0; r < keep; ++r) {
      float best = -2.f;
      int bi = groups;
      for (int gI = lane; gI < groups; gI += 64) {
        const float v = g_s[gI];
        if (v > best || (v == best && gI < bi)) { best = v; bi = gI; }
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const float ob = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
      }
      __syncthreads();
      if (lane == 0) g_s[bi] = -3.f;  // chosen
      __syncthreads();
    }
    for (int e = lane; e < E; e += 64)
      if (g_s[e / per] != -3.f) s_s[e] = -1.f;
    __syncthreads();
  }
  float wsum = 0.f;
  float wk[ROUTE_MAX_K];
  int ik[ROUTE_MAX_K];
  for (int r = 0; r < top; ++r) {
    float best = -2.f;
    int bi = E;
    for (int e = lane; e < E; e += 64) {
      const float v = s_s[e];
      if (v > best || (v == best && e < bi)) { best = v; bi = e; }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    wk[r] = best;
    ik[r] = bi;
    wsum += best;
    __syncthreads();
    if (lane == 0) s_s[bi] = -2.f;
    __syncthreads();
  }
  if (lane == 0) {
    const float d = wsum + 1e-20f;
    for (int r = 0; r < top; ++r) {
      const float w = renorm ? wk[r] / d : wk[r];
      weights[(int64_t)t * top + r] = w;
      ids[(int64_t)t * top + r] = ik[r];
      if (matrix) matrix[(int64_t)t * E + ik[r]] = w;
    }
  }
}

template <typename AT>
__global__ __launch_bounds__(256) void moe_mix_rows_kernel(
    AT* __restrict__ out, const AT* __restrict__ y,
    const float* __restrict__ weights, const int* __restrict__ rows, int T,
    int H, int k, int dense, const AT* __restrict__ add) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < H; c += 256) {
    float acc = add ? Act<AT>::ld(add + (int64_t)t * H + c) : 0.f;
    for (int j = 0; j < k; ++j) {
      const int64_t r = dense ? (int64_t)rows[t * k + j] * T + t
                              : (int64_t)rows[t * k + j];
      acc += weights[t * k + j] * Act<AT>::ld(y + r * H + c);
    }
    Act<AT>::st(out + (int64_t)t * H + c, acc);
  }
}

// bf16, 8 channels per thread (H % 8 == 0)
__global__ __launch_bounds__(256) void moe_mix_rows_vec8_kernel(
    bf16* __restrict__ out, const bf16* __restrict__ y,
    const float* __restrict__ weights, const int* __restrict__ rows, int T,
    int H, int k, int dense, const bf16* __restrict__ add) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x * 8; c < H; c += 256 * 8) {
    float acc[8];
    if (add) {
      const ushort8 u = *reinterpret_cast<const ushort8*>(add + (int64_t)t * H + c);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = bf16_bits_to_float(u[e]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    }
    for (int j = 0; j < k; ++j) {
      const int64_t r = dense ? (int64_t)rows[t * k + j] * T + t
                              : (int64_t)rows[t * k + j];
      const float w = weights[t * k + j];
      const ushort8 u = *reinterpret_cast<const ushort8*>(y + r * H + c);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += w * bf16_bits_to_float(u[e]);
    }
    ushort8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = float_to_bf16_bits(acc[e]);
    *reinterpret_cast<ushort8*>(out + (int64_t)t * H + c) = o;
  }
}

}  // namespace arks

using namespace arks;

extern "C" int arks_seq_moe_route_grouped(void* weights, void* ids,
                                          const void* logits, int T, int E,
                                          int top, int groups, int keep,
                                          int sigmoid, int renorm,
                                          void* matrix, hipStream_t stream) {
  if (E > ROUTE_MAX_E || top > ROUTE_MAX_K || groups < 1 || E % groups ||
      keep > groups || top > keep * (E / groups))
    return 1;
  if (T == 0) return 0;
  hipLaunchKernelGGL(moe_route_grouped_kernel, dim3(T), dim3(64), 0, stream,
                     (float*)weights, (int*)ids, (const float*)logits, E, top,
                     groups, keep, sigmoid, renorm, (float*)matrix);
  return 0;
}

extern "C" void arks_seq_moe_mix_rows(void* out, const void* y,
                                      const void* weights, const void* rows,
                                      int T, int H, int k, int dense,
                                      const void* add, int act_f32,
                                      hipStream_t stream) {
  if (T == 0) return;
  if (!act_f32 && H % 8 == 0) {
    hipLaunchKernelGGL(moe_mix_rows_vec8_kernel, dim3(T), dim3(256), 0, stream,
                       (bf16*)out, (const bf16*)y, (const float*)weights,
                       (const int*)rows, T, H, k, dense, (const bf16*)add);
    return;
  }
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (moe_mix_rows_kernel<AT>), dim3(T), dim3(256), 0, stream, (AT*)out,
      (const AT*)y, (const float*)weights, (const int*)rows, T, H, k, dense,
      (const AT*)add));
}
