// Row kernels of the stream arrangement (arks_amd/models/hybrid.py
// StreamBlock): the residual lives in `s` weighted copies xs[s][T][C], fp32.
//
//   stream_mix_norm   applies the previous sublayer's result to the copies
//                     (new[t] = sum_s mix[s][t] old[s] + out[t] (y + bias)),
//                     reads the next sublayer's input u = sum_s in[s] new[s]
//                     and writes its layer norm (weight and bias) — one pass
//                     over the copies per sublayer
//   short_conv_residual  h + causal depthwise conv of h over time, with the
//                     last taps-1 rows of every sequence kept as state
//   head_norm_gate    per-head unit RMS times silu(gate) (retention output)
//   glu_act           [gate | up] rows -> activated rows
#include "seq_common.h"

namespace arks {

constexpr int STREAM_MAX = 8;  // residual copies

// One block per row. u is staged in LDS (C floats) between the passes: mean,
// then the mean squared deviation, then the output.
template <typename AT, int VEC>
__global__ __launch_bounds__(256) void stream_mix_norm_kernel(
    float* __restrict__ xs, float* __restrict__ n_out,
    const AT* __restrict__ y, int64_t ldy, const float* __restrict__ y_bias,
    const float* __restrict__ mix, const float* __restrict__ out_w,
    const float* __restrict__ in_w, const float* __restrict__ norm_w,
    const float* __restrict__ norm_b, float eps, int S, int64_t T, int C) {
  extern __shared__ float u_s[];
  __shared__ float red[8];
  __shared__ float par[STREAM_MAX * STREAM_MAX + 2 * STREAM_MAX];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  float* mix_s = par;
  float* out_s = par + STREAM_MAX * STREAM_MAX;
  float* in_s = out_s + STREAM_MAX;
  if (tid < S * S) mix_s[tid] = y ? mix[tid] : 0.f;
  if (tid < S) {
    out_s[tid] = y ? out_w[tid] : 0.f;
    in_s[tid] = in_w ? in_w[tid] : 0.f;
  }
  __syncthreads();
  float sum = 0.f;
  for (int c = tid * VEC; c < C; c += 256 * VEC) {
    float old[STREAM_MAX][VEC], nw[STREAM_MAX][VEC], yv[VEC];
#pragma unroll
    for (int s = 0; s < STREAM_MAX; ++s) {
      if (s < S) {
        const float* p = xs + ((int64_t)s * T + t) * C + c;
        if (VEC == 4) {
          const float4v v = *reinterpret_cast<const float4v*>(p);
#pragma unroll
          for (int e = 0; e < VEC; ++e) old[s][e] = v[e];
        } else {
          old[s][0] = p[0];
        }
      }
    }
    if (y) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        yv[e] = Act<AT>::ld(y + t * ldy + c + e);
        if (y_bias) yv[e] += y_bias[c + e];
      }
#pragma unroll
      for (int d = 0; d < STREAM_MAX; ++d) {
        if (d < S) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) nw[d][e] = out_s[d] * yv[e];
#pragma unroll
          for (int s = 0; s < STREAM_MAX; ++s)
            if (s < S) {
#pragma unroll
              for (int e = 0; e < VEC; ++e) nw[d][e] += mix_s[s * S + d] * old[s][e];
            }
          float* p = xs + ((int64_t)d * T + t) * C + c;
          if (VEC == 4) {
            float4v v;
#pragma unroll
            for (int e = 0; e < VEC; ++e) v[e] = nw[d][e];
            *reinterpret_cast<float4v*>(p) = v;
          } else {
            p[0] = nw[d][0];
          }
        }
      }
    } else {
#pragma unroll
      for (int d = 0; d < STREAM_MAX; ++d)
        if (d < S) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) nw[d][e] = old[d][e];
        }
    }
    if (in_w) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        float u = 0.f;
#pragma unroll
        for (int d = 0; d < STREAM_MAX; ++d)
          if (d < S) u += in_s[d] * nw[d][e];
        u_s[c + e] = u;
        sum += u;
      }
    }
  }
  if (!in_w) return;
  const float mean = block_reduce_sum<256>(sum, red) / (float)C;
  __syncthreads();
  float sq = 0.f;
  for (int c = tid; c < C; c += 256) {
    const float d = u_s[c] - mean;
    sq += d * d;
  }
  const float var = block_reduce_sum<256>(sq, red) / (float)C;
  const float rstd = 1.f / sqrtf(var + eps);
  for (int c = tid; c < C; c += 256)
    n_out[t * C + c] = (u_s[c] - mean) * rstd * norm_w[c] + norm_b[c];
}

// The same for S <= 4 copies and rows of up to 1024 * NV channels
// (C % 4 == 0): every thread keeps its float4 pieces of u in registers
// between the passes, so the copies are read once and nothing is staged.
template <typename AT, int NV, int S>
__global__ __launch_bounds__(256) void stream_mix_norm_reg_kernel(
    float* __restrict__ xs, float* __restrict__ n_out,
    const AT* __restrict__ y, int64_t ldy, const float* __restrict__ y_bias,
    const float* __restrict__ mix, const float* __restrict__ out_w,
    const float* __restrict__ in_w, const float* __restrict__ norm_w,
    const float* __restrict__ norm_b, float eps, int64_t T, int C) {
  __shared__ float red[8];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  float mixv[S * S], outv[S], inv_[S];
#pragma unroll
  for (int i = 0; i < S * S; ++i) mixv[i] = y ? mix[i] : 0.f;
#pragma unroll
  for (int i = 0; i < S; ++i) {
    outv[i] = y ? out_w[i] : 0.f;
    inv_[i] = in_w ? in_w[i] : 0.f;
  }
  float4v u[NV];
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = (tid + 256 * j) * 4;
    u[j] = {0.f, 0.f, 0.f, 0.f};
    if (c < C) {
      float4v old[S];
#pragma unroll
      for (int s = 0; s < S; ++s)
        old[s] = *reinterpret_cast<const float4v*>(xs + ((int64_t)s * T + t) * C + c);
      if (y) {
        float4v yv;
#pragma unroll
        for (int e = 0; e < 4; ++e) yv[e] = Act<AT>::ld(y + t * ldy + c + e);
        if (y_bias) yv += *reinterpret_cast<const float4v*>(y_bias + c);
#pragma unroll
        for (int d = 0; d < S; ++d) {
          float4v nw = outv[d] * yv;
#pragma unroll
          for (int s = 0; s < S; ++s) nw += mixv[s * S + d] * old[s];
          *reinterpret_cast<float4v*>(xs + ((int64_t)d * T + t) * C + c) = nw;
          u[j] += inv_[d] * nw;
        }
      } else {
#pragma unroll
        for (int d = 0; d < S; ++d) u[j] += inv_[d] * old[d];
      }
      sum += u[j][0] + u[j][1] + u[j][2] + u[j][3];
    }
  }
  if (!in_w) return;
  const float mean = block_reduce_sum<256>(sum, red) / (float)C;
  __syncthreads();
  float sq = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = (tid + 256 * j) * 4;
    if (c < C) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float d = u[j][e] - mean;
        sq += d * d;
      }
    }
  }
  const float var = block_reduce_sum<256>(sq, red) / (float)C;
  const float rstd = 1.f / sqrtf(var + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int c = (tid + 256 * j) * 4;
    if (c < C) {
      const float4v w = *reinterpret_cast<const float4v*>(norm_w + c);
      const float4v b = *reinterpret_cast<const float4v*>(norm_b + c);
      float4v o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (u[j][e] - mean) * rstd * w[e] + b[e];
      *reinterpret_cast<float4v*>(n_out + t * C + c) = o;
    }
  }
}

// One block per (row, 256 channels). Inputs before the step's first row come
// from the sequence's stored history (zeros at position 0); the history is
// replaced by a later launch, so every reader here sees the old one.
template <typename AT>
__global__ __launch_bounds__(256) void short_conv_residual_kernel(
    AT* __restrict__ out, const float* __restrict__ h,
    const float* __restrict__ w, const float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ seq_lens,
    const int* __restrict__ slots, const int* __restrict__ token_seq, int C,
    int taps) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const SeqRow r = seq_row(t, token_seq, cu, seq_lens, slots);
  const int i = t - r.first_row;
  const bool has_state = r.start > 0 && r.slot >= 0;
  const float* hist =
      state ? state + (int64_t)(r.slot < 0 ? 0 : r.slot) * (taps - 1) * C : nullptr;
  float acc = h[(int64_t)t * C + c];
  for (int j = 0; j < taps; ++j) {
    const int src = i - (taps - 1 - j);
    float xv;
    if (src >= 0)
      xv = h[(int64_t)(r.first_row + src) * C + c];
    else
      xv = has_state ? hist[(int64_t)(src + taps - 1) * C + c] : 0.f;
    acc += w[(int64_t)c * taps + j] * xv;
  }
  Act<AT>::st(out + (int64_t)t * C + c, acc);
}

// 4 channels per thread and rpb consecutive rows per block (16 for long
// steps, fewer for short ones so the grid still fills the chip): the thread
// walks its rows with the last taps-1 inputs in registers, so every input
// is read once per block (plus the block's first rows' history).
constexpr int SC_MAX_TAPS = 8;

template <typename AT>
__global__ __launch_bounds__(256) void short_conv_residual_vec_kernel(
    AT* __restrict__ out, const float* __restrict__ h,
    const float* __restrict__ w, const float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ seq_lens,
    const int* __restrict__ slots, const int* __restrict__ token_seq, int T,
    int C, int taps, int rpb) {
  const int c = (blockIdx.y * 256 + threadIdx.x) * 4;
  if (c >= C) return;
  float4v wv[SC_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < SC_MAX_TAPS; ++j)
    if (j < taps) {
#pragma unroll
      for (int e = 0; e < 4; ++e) wv[j][e] = w[(int64_t)(c + e) * taps + j];
    }
  const int t0 = blockIdx.x * rpb;
  const int t1 = min(T, t0 + rpb);
  float4v prev[SC_MAX_TAPS];  // prev[j]: the input taps-1-j rows back
  int cur_seq = -1;
  for (int t = t0; t < t1; ++t) {
    const int seq = token_seq[t];
    if (seq != cur_seq) {
      // (re)load the history of this row: earlier rows of the step, the
      // sequence's stored inputs, or zeros before its start
      cur_seq = seq;
      const SeqRow r = seq_row(t, token_seq, cu, seq_lens, slots);
      const int i = t - r.first_row;
      const bool has_state = r.start > 0 && r.slot >= 0;
      const float* hist =
          state ? state + (int64_t)(r.slot < 0 ? 0 : r.slot) * (taps - 1) * C : nullptr;
#pragma unroll
      for (int j = 0; j < SC_MAX_TAPS; ++j)
        if (j < taps - 1) {
          const int src = i - (taps - 1 - j);
          if (src >= 0)
            prev[j] = *reinterpret_cast<const float4v*>(
                h + (int64_t)(r.first_row + src) * C + c);
          else if (has_state)
            prev[j] = *reinterpret_cast<const float4v*>(
                hist + (int64_t)(src + taps - 1) * C + c);
          else
            prev[j] = {0.f, 0.f, 0.f, 0.f};
        }
    }
    const float4v x = *reinterpret_cast<const float4v*>(h + (int64_t)t * C + c);
    float4v acc = x;
#pragma unroll
    for (int j = 0; j < SC_MAX_TAPS; ++j)
      if (j < taps - 1) acc += wv[j] * prev[j];
#pragma unroll
    for (int j = 0; j < SC_MAX_TAPS; ++j)
      if (j == taps - 1) acc += wv[j] * x;
#pragma unroll
    for (int e = 0; e < 4; ++e) Act<AT>::st(out + (int64_t)t * C + c + e, acc[e]);
#pragma unroll
    for (int j = 0; j < SC_MAX_TAPS - 1; ++j) {
      if (j < taps - 2) prev[j] = prev[j + 1];
      else if (j == taps - 2) prev[j] = x;
    }
  }
}

constexpr int SC_MAX_HIST = 15;

// New history = the last taps-1 inputs after this step. One thread per
// (sequence, channel) reads all it needs before it writes.
__global__ __launch_bounds__(256) void short_conv_state_kernel(
    float* __restrict__ state, const float* __restrict__ h,
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
  float nv[SC_MAX_HIST];
#pragma unroll
  for (int i = 0; i < SC_MAX_HIST; ++i) {
    if (i < nh) {
      const int src = rows - nh + i;  // index into this step's rows
      if (src >= 0)
        nv[i] = h[(int64_t)(a + src) * C + c];
      else  // older: the history's entry src + nh, zeros before position 0
        nv[i] = (start + src >= 0 && start > 0) ? hist[(int64_t)(src + nh) * C] : 0.f;
    }
  }
#pragma unroll
  for (int i = 0; i < SC_MAX_HIST; ++i)
    if (i < nh) hist[(int64_t)i * C] = nv[i];
}

// One wave per (row, head): o / rms(o) * silu(g) * scale.
template <typename AT>
__global__ __launch_bounds__(64) void head_norm_gate_kernel(
    AT* __restrict__ out, int64_t ldo, const float* __restrict__ o,
    const AT* __restrict__ gate, int64_t ldg, float eps, int V,
    float out_scale) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + (t * gridDim.y + h) * V;
  float sq = 0.f;
  for (int d = lane; d < V; d += 64) sq += orow[d] * orow[d];
  sq = wave_reduce_sum(sq);
  const float r = out_scale / sqrtf(sq / (float)V + eps);
  for (int d = lane; d < V; d += 64) {
    const float g = Act<AT>::ld(gate + t * ldg + (int64_t)h * V + d);
    Act<AT>::st(out + t * ldo + (int64_t)h * V + d, orow[d] * r * silu_f(g));
  }
}

// mode 0: silu(g) * u;  mode 1: g = min(g, limit), u = clamp(u, +-limit),
// g * sigmoid(alpha g) * (u + 1);  mode 2: gelu_tanh(g) * u. The output is
// a row-strided view (ldo).
__device__ __forceinline__ float glu_value(float g, float u, int mode,
                                           float limit, float alpha) {
  if (mode == 0) return silu_f(g) * u;
  if (mode == 2) {
    const float z = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    return 0.5f * g * (1.f + tanhf(z)) * u;
  }
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g * sigmoid_f(alpha * g) * (u + 1.f);
}

template <typename AT>
__global__ __launch_bounds__(256) void glu_act_kernel(
    AT* __restrict__ out, int64_t ldo, const AT* __restrict__ gu, int64_t ldg,
    int64_t rows, int F, int mode, float limit, float alpha,
    const float* __restrict__ row_scale) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= rows * F) return;
  const int64_t t = i / F;
  const int c = (int)(i - t * F);
  const float rs = row_scale ? row_scale[t] : 1.f;
  const float g = rs * Act<AT>::ld(gu + t * ldg + c);
  const float u = rs * Act<AT>::ld(gu + t * ldg + F + c);
  Act<AT>::st(out + t * ldo + c, glu_value(g, u, mode, limit, alpha));
}

// bf16, 8 elements per thread (F % 8 == 0, 16-byte aligned rows)
__global__ __launch_bounds__(256) void glu_act_vec8_kernel(
    bf16* __restrict__ out, int64_t ldo, const bf16* __restrict__ gu,
    int64_t ldg, int64_t rows, int F, int mode, float limit, float alpha,
    const float* __restrict__ row_scale) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i >= rows * F) return;
  const int64_t t = i / F;
  const int c = (int)(i - t * F);
  const float rs = row_scale ? row_scale[t] : 1.f;
  const ushort8 gv = *reinterpret_cast<const ushort8*>(gu + t * ldg + c);
  const ushort8 uv = *reinterpret_cast<const ushort8*>(gu + t * ldg + F + c);
  ushort8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    o[e] = float_to_bf16_bits(glu_value(rs * bf16_bits_to_float(gv[e]),
                                        rs * bf16_bits_to_float(uv[e]), mode,
                                        limit, alpha));
  }
  *reinterpret_cast<ushort8*>(out + t * ldo + c) = o;
}

}  // namespace arks

using namespace arks;

extern "C" int arks_seq_stream_mix_norm(
    void* xs, void* n_out, const void* y, int64_t ldy, const void* y_bias,
    const void* mix, const void* out_w, const void* in_w, const void* norm_w,
    const void* norm_b, float eps, int S, int64_t T, int C, int act_f32,
    hipStream_t stream) {
  if (S > STREAM_MAX || (int64_t)C * 4 > 64 * 1024) return 1;
  if (T == 0) return 0;
  const size_t lds = (size_t)C * 4;
  const bool vec = C % 4 == 0 && (y == nullptr || ldy % 4 == 0);
  if (C % 4 == 0 && C <= 8192 && S <= 4) {
#define SMR(NV, SS)                                                            \
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(                                \
      (stream_mix_norm_reg_kernel<AT, NV, SS>), dim3((unsigned)T), dim3(256),  \
      0, stream, (float*)xs, (float*)n_out, (const AT*)y, ldy,                 \
      (const float*)y_bias, (const float*)mix, (const float*)out_w,            \
      (const float*)in_w, (const float*)norm_w, (const float*)norm_b, eps, T,  \
      C))
#define SMS(NV)                \
  do {                         \
    if (S == 1) SMR(NV, 1);    \
    else if (S == 2) SMR(NV, 2); \
    else if (S == 3) SMR(NV, 3); \
    else SMR(NV, 4);           \
  } while (0)
    if (C <= 1024) SMS(1);
    else if (C <= 2048) SMS(2);
    else if (C <= 4096) SMS(4);
    else SMS(8);
#undef SMS
#undef SMR
    return 0;
  }
#define SMN(VEC)                                                              \
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(                               \
      (stream_mix_norm_kernel<AT, VEC>), dim3((unsigned)T), dim3(256), lds,   \
      stream, (float*)xs, (float*)n_out, (const AT*)y, ldy,                   \
      (const float*)y_bias, (const float*)mix, (const float*)out_w,           \
      (const float*)in_w, (const float*)norm_w, (const float*)norm_b, eps, S, \
      T, C))
  if (vec) SMN(4);
  else SMN(1);
#undef SMN
  return 0;
}

extern "C" int arks_seq_short_conv_residual(
    void* out, const void* h, const void* w, void* state, const void* cu,
    const void* seq_lens, const void* slots, const void* token_seq, int T,
    int S, int C, int taps, int act_f32, hipStream_t stream) {
  if (taps - 1 > SC_MAX_HIST) return 1;
  if (T == 0) return 0;
  const int cb = (C + 255) / 256;
  if (C % 4 == 0 && taps <= SC_MAX_TAPS) {
    const int rpb = T >= 8192 ? 16 : (T >= 1024 ? 4 : 1);
    SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
        (short_conv_residual_vec_kernel<AT>),
        dim3((T + rpb - 1) / rpb, (C / 4 + 255) / 256), dim3(256), 0,
        stream, (AT*)out, (const float*)h, (const float*)w,
        (const float*)state, (const int*)cu, (const int*)seq_lens,
        (const int*)slots, (const int*)token_seq, T, C, taps, rpb));
  } else {
    SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
        (short_conv_residual_kernel<AT>), dim3(T, cb), dim3(256), 0, stream,
        (AT*)out, (const float*)h, (const float*)w, (const float*)state,
        (const int*)cu, (const int*)seq_lens, (const int*)slots,
        (const int*)token_seq, C, taps));
  }
  if (taps > 1)
    hipLaunchKernelGGL(short_conv_state_kernel, dim3(S, cb), dim3(256), 0,
                       stream, (float*)state, (const float*)h, (const int*)cu,
                       (const int*)seq_lens, (const int*)slots, C, taps);
  return 0;
}

extern "C" void arks_seq_head_norm_gate(void* out, int64_t ldo, const void* o,
                                        const void* gate, int64_t ldg,
                                        float eps, int T, int H, int V,
                                        float out_scale, int act_f32,
                                        hipStream_t stream) {
  if (T == 0) return;
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (head_norm_gate_kernel<AT>), dim3(T, H), dim3(64), 0, stream, (AT*)out,
      ldo, (const float*)o, (const AT*)gate, ldg, eps, V, out_scale));
}

extern "C" void arks_seq_glu_act(void* out, int64_t ldo, const void* gu,
                                 int64_t ldg, int64_t rows, int F, int mode,
                                 float limit, float alpha,
                                 const void* row_scale, int act_f32,
                                 hipStream_t stream) {
  const int64_t n = rows * F;
  if (n == 0) return;
  if (!act_f32 && F % 8 == 0 && ldg % 8 == 0 && ldo % 8 == 0 &&
      ((uintptr_t)out & 15) == 0 && ((uintptr_t)gu & 15) == 0) {
    hipLaunchKernelGGL(glu_act_vec8_kernel,
                       dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0,
                       stream, (bf16*)out, ldo, (const bf16*)gu, ldg, rows, F,
                       mode, limit, alpha, (const float*)row_scale);
    return;
  }
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (glu_act_kernel<AT>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
      stream, (AT*)out, ldo, (const AT*)gu, ldg, rows, F, mode, limit, alpha,
      (const float*)row_scale));
}
