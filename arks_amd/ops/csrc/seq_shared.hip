// Row kernels of the shared-norm blocks and of latent attention:
//   residual_tanh_norm: x (fp32 residual) += mult * y, then
//       h = tanh(alpha x) * w + b  — a norm without statistics, so nothing
//       is reduced over the row and the kernel is purely elementwise;
//   latent_prepare: RMS norm of the query latent; RMS norm of the key/value
//       latent and rotation of the shared key part, written to the row's
//       place in the paged latent cache;
//   latent_query: [absorbed query | rotated part] per head.
#include "seq_common.h"

namespace arks {

// tanh for rows that are rounded to bf16 afterwards: 1 - 2 / (e^{2z} + 1)
// with the hardware exponential; absolute error ~1e-7.
template <typename AT>
__device__ __forceinline__ float tanh_act(float z);
template <>
__device__ __forceinline__ float tanh_act<float>(float z) { return tanhf(z); }
template <>
__device__ __forceinline__ float tanh_act<bf16>(float z) {
  const float e = __expf(2.f * fminf(fmaxf(z, -15.f), 15.f));
  return 1.f - 2.f / (e + 1.f);
}

// One thread per element. y, h: [T, C] dense; xa: [T, C] with row stride.
template <typename AT>
__global__ __launch_bounds__(256) void residual_tanh_norm_kernel(
    float* __restrict__ x, AT* __restrict__ h, AT* __restrict__ xa,
    int64_t ldxa, const AT* __restrict__ y, float mult,
    const float* __restrict__ alpha, const float* __restrict__ w,
    const float* __restrict__ b, int64_t n, int C) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float v = x[i];
  if (y) {
    v += mult * Act<AT>::ld(y + i);
    x[i] = v;
  }
  const int64_t t = i / C;
  const int c = (int)(i - t * C);
  if (xa) Act<AT>::st(xa + t * ldxa + c, v);
  if (h) Act<AT>::st(h + i, tanh_act<AT>(alpha[0] * v) * w[c] + b[c]);
}

// bf16 rows, 8 elements per thread (C % 8 == 0, 16-byte aligned rows).
__global__ __launch_bounds__(256) void residual_tanh_norm_vec8_kernel(
    float* __restrict__ x, bf16* __restrict__ h, bf16* __restrict__ xa,
    int64_t ldxa, const bf16* __restrict__ y, float mult,
    const float* __restrict__ alpha, const float* __restrict__ w,
    const float* __restrict__ b, int64_t n, int C) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i >= n) return;
  float v[8];
  {
    const float4v a0 = *reinterpret_cast<const float4v*>(x + i);
    const float4v a1 = *reinterpret_cast<const float4v*>(x + i + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { v[e] = a0[e]; v[4 + e] = a1[e]; }
  }
  if (y) {
    const ushort8 yv = *reinterpret_cast<const ushort8*>(y + i);
    float4v o0, o1;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] += mult * bf16_bits_to_float(yv[e]);
#pragma unroll
    for (int e = 0; e < 4; ++e) { o0[e] = v[e]; o1[e] = v[4 + e]; }
    *reinterpret_cast<float4v*>(x + i) = o0;
    *reinterpret_cast<float4v*>(x + i + 4) = o1;
  }
  const int64_t t = i / C;
  const int c = (int)(i - t * C);
  if (xa) {
    ushort8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = float_to_bf16_bits(v[e]);
    *reinterpret_cast<ushort8*>(xa + t * ldxa + c) = o;
  }
  if (h) {
    const float al = alpha[0];
    const float4v w0 = *reinterpret_cast<const float4v*>(w + c);
    const float4v w1 = *reinterpret_cast<const float4v*>(w + c + 4);
    const float4v b0 = *reinterpret_cast<const float4v*>(b + c);
    const float4v b1 = *reinterpret_cast<const float4v*>(b + c + 4);
    ushort8 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      o[e] = float_to_bf16_bits(tanh_act<bf16>(al * v[e]) * w0[e] + b0[e]);
      o[4 + e] =
          float_to_bf16_bits(tanh_act<bf16>(al * v[4 + e]) * w1[e] + b1[e]);
    }
    *reinterpret_cast<ushort8*>(h + i) = o;
  }
}

// One block per row. cq [T, Rq] (row stride ldq) -> cqn [T, Rq] dense;
// ckv [T, Rk + 2P] (row stride ldk) -> its cache row.
template <typename AT>
__global__ __launch_bounds__(256) void latent_prepare_kernel(
    AT* __restrict__ cqn, const AT* __restrict__ cq, int64_t ldq,
    const AT* __restrict__ ckv, int64_t ldk, const float* __restrict__ qw,
    const float* __restrict__ kw, float eps,
    const int64_t* __restrict__ positions, const float* __restrict__ freq,
    AT* __restrict__ cache, const int64_t* __restrict__ slot_mapping, int Rq,
    int Rk, int P) {
  __shared__ float scratch[4];
  __shared__ float scratch2[4];
  const int t = blockIdx.x;
  const AT* qr = cq + (int64_t)t * ldq;
  float ss = 0.f;
  for (int i = threadIdx.x; i < Rq; i += 256) {
    const float a = Act<AT>::ld(qr + i);
    ss += a * a;
  }
  ss = block_reduce_sum<256>(ss, scratch);
  const float rq = 1.f / sqrtf(ss / (float)Rq + eps);
  for (int i = threadIdx.x; i < Rq; i += 256)
    Act<AT>::st(cqn + (int64_t)t * Rq + i, Act<AT>::ld(qr + i) * rq * qw[i]);
  const int64_t slot = slot_mapping[t];
  if (slot < 0) return;  // uniform over the block
  const AT* kr = ckv + (int64_t)t * ldk;
  AT* dst = cache + slot * (int64_t)(Rk + 2 * P);
  float s2 = 0.f;
  for (int i = threadIdx.x; i < Rk; i += 256) {
    const float a = Act<AT>::ld(kr + i);
    s2 += a * a;
  }
  s2 = block_reduce_sum<256>(s2, scratch2);
  const float rk = 1.f / sqrtf(s2 / (float)Rk + eps);
  for (int i = threadIdx.x; i < Rk; i += 256)
    Act<AT>::st(dst + i, Act<AT>::ld(kr + i) * rk * kw[i]);
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < P; i += 256) {
    float sn, cs;
    sincosf(pos * freq[i], &sn, &cs);
    const float a = Act<AT>::ld(kr + Rk + 2 * i);
    const float b = Act<AT>::ld(kr + Rk + 2 * i + 1);
    Act<AT>::st(dst + Rk + 2 * i, a * cs - b * sn);
    Act<AT>::st(dst + Rk + 2 * i + 1, b * cs + a * sn);
  }
}

// out [T, H, Rk + 2P] = [q_abs[h, t, :] | rotated q[t, h, D:]]; one block
// per row, waves over heads. q_abs null: the first part is q[t, h, :D].
template <typename AT>
__global__ __launch_bounds__(256) void latent_query_kernel(
    AT* __restrict__ out, const AT* __restrict__ q,
    const AT* __restrict__ q_abs, const int64_t* __restrict__ positions,
    const float* __restrict__ freq, int T, int H, int D, int Rk, int P) {
  const int t = blockIdx.x;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const float pos = (float)positions[t];
  for (int hh = wave; hh < H; hh += 4) {
    AT* dst = out + ((int64_t)t * H + hh) * (Rk + 2 * P);
    // without q_abs the plain part is q's own (Rk == D)
    const AT* src = q_abs ? q_abs + ((int64_t)hh * T + t) * Rk
                          : q + ((int64_t)t * H + hh) * (D + 2 * P);
    for (int i = lane; i < Rk; i += 64) dst[i] = src[i];
    const AT* qr = q + ((int64_t)t * H + hh) * (D + 2 * P) + D;
    for (int i = lane; i < P; i += 64) {
      float sn, cs;
      sincosf(pos * freq[i], &sn, &cs);
      const float a = Act<AT>::ld(qr + 2 * i);
      const float b = Act<AT>::ld(qr + 2 * i + 1);
      Act<AT>::st(dst + Rk + 2 * i, a * cs - b * sn);
      Act<AT>::st(dst + Rk + 2 * i + 1, b * cs + a * sn);
    }
  }
}

}  // namespace arks

using namespace arks;

extern "C" void arks_seq_residual_tanh_norm(
    void* x, void* h, void* xa, int64_t ldxa, const void* y, float mult,
    const void* alpha, const void* w, const void* b, int64_t T, int C,
    int act_f32, hipStream_t stream) {
  const int64_t n = T * C;
  if (n == 0) return;
  const bool aligned = (((uintptr_t)x | (uintptr_t)h | (uintptr_t)xa |
                         (uintptr_t)y | (uintptr_t)w | (uintptr_t)b) & 15) == 0;
  if (!act_f32 && C % 8 == 0 && ldxa % 8 == 0 && aligned) {
    hipLaunchKernelGGL(residual_tanh_norm_vec8_kernel,
                       dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0,
                       stream, (float*)x, (bf16*)h, (bf16*)xa, ldxa,
                       (const bf16*)y, mult, (const float*)alpha,
                       (const float*)w, (const float*)b, n, C);
    return;
  }
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (residual_tanh_norm_kernel<AT>), dim3((unsigned)((n + 255) / 256)),
      dim3(256), 0, stream, (float*)x, (AT*)h, (AT*)xa, ldxa, (const AT*)y,
      mult, (const float*)alpha, (const float*)w, (const float*)b, n, C));
}

extern "C" void arks_seq_latent_prepare(
    void* cqn, const void* cq, int64_t ldq, const void* ckv, int64_t ldk,
    const void* qw, const void* kw, float eps, const void* positions,
    const void* freq, void* cache, const void* slot_mapping, int T, int Rq,
    int Rk, int P, int act_f32, hipStream_t stream) {
  if (T == 0) return;
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (latent_prepare_kernel<AT>), dim3(T), dim3(256), 0, stream, (AT*)cqn,
      (const AT*)cq, ldq, (const AT*)ckv, ldk, (const float*)qw,
      (const float*)kw, eps, (const int64_t*)positions, (const float*)freq,
      (AT*)cache, (const int64_t*)slot_mapping, Rq, Rk, P));
}

extern "C" void arks_seq_latent_query(void* out, const void* q,
                                      const void* q_abs, const void* positions,
                                      const void* freq, int T, int H, int D,
                                      int Rk, int P, int act_f32,
                                      hipStream_t stream) {
  if (T == 0) return;
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (latent_query_kernel<AT>), dim3(T), dim3(256), 0, stream, (AT*)out,
      (const AT*)q, (const AT*)q_abs, (const int64_t*)positions,
      (const float*)freq, T, H, D, Rk, P));
}
