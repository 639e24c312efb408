// Mamba2 mixer kernels: the scalar-decay state-space recurrence
//   S_h <- exp(-rate_h dt_h) S_h + dt_h B_g x_h^T      (S_h: N x V, fp32)
//   y_h = S_h^T C_g + D_h x_h,      dt = softplus(dt_raw + dt_bias)
// over rows [x | B | C] that already went through the short convolution
// (seq_mamba.hip causal_conv_silu), and the gated group norm behind it.
// Head h reads group g = h / (P / G) of B and C.
//
// Scan: one wave per (sequence or chunk, head, 64 value columns); lane v
// keeps column S[:, v] in registers, so y needs no reduction across lanes.
// B and C of MB2_ROWS rows at a time are staged in LDS (every lane reads
// all of them). With `out` null only the end state and the summed step
// sizes are produced (pass 1 of the chunk-parallel prefill); the combine
// kernel then turns every chunk's end-from-zero state into its start state
// and leaves the sequence's final state in its slot.
#include "seq_common.h"

namespace arks {

constexpr int MB2_ROWS = 8;

template <typename AT, int NREG>
__global__ __launch_bounds__(64) void mamba2_scan_kernel(
    float* __restrict__ out, const AT* __restrict__ xbc, int64_t ldx,
    const AT* __restrict__ dt_raw, int64_t ldd,
    const float* __restrict__ dt_bias, const float* __restrict__ rate,
    const float* __restrict__ Dp, float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ seq_lens,
    const int* __restrict__ slots, float* __restrict__ dsum, int P, int V,
    int N, int G) {
  __shared__ float bc_s[MB2_ROWS][2 * NREG];
  __shared__ float dt_s[MB2_ROWS];
  const int s = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int v = blockIdx.z * 64 + lane;
  const bool live = v < V;
  const int first = cu[s], rows = cu[s + 1] - first;
  if (rows == 0) return;
  const int start = seq_lens[s] - rows;
  const int slot = slots[s];
  const int g = h / (P / G);
  const float r = rate[h], bias = dt_bias[h], dskip = Dp[h];
  float st[NREG];
  float* sp = state + (((int64_t)(slot < 0 ? 0 : slot) * P + h) * N) * V + v;
  const bool resume = start > 0 && slot >= 0 && live;
#pragma unroll
  for (int n = 0; n < NREG; ++n)
    st[n] = (resume && n < N) ? sp[(int64_t)n * V] : 0.f;
  const int64_t boff = (int64_t)P * V + (int64_t)g * N;
  const int64_t coff = boff + (int64_t)G * N;
  float dt_total = 0.f;
  for (int r0 = 0; r0 < rows; r0 += MB2_ROWS) {
    const int nr = min(MB2_ROWS, rows - r0);
    __syncthreads();  // the previous rows' readers are done
    for (int i = lane; i < nr * 2 * N; i += 64) {
      const int rr = i / (2 * N), c = i % (2 * N);
      const AT* row = xbc + (int64_t)(first + r0 + rr) * ldx;
      bc_s[rr][c < N ? c : NREG + c - N] =
          Act<AT>::ld(row + (c < N ? boff + c : coff + c - N));
    }
    if (lane < nr)
      dt_s[lane] = softplus_f(
          Act<AT>::ld(dt_raw + (int64_t)(first + r0 + lane) * ldd + h) + bias);
    __syncthreads();
    for (int rr = 0; rr < nr; ++rr) {
      const int t = first + r0 + rr;
      const float dt = dt_s[rr];
      const float a = expf(-r * dt);
      dt_total += dt;
      const float xv =
          live ? Act<AT>::ld(xbc + (int64_t)t * ldx + (int64_t)h * V + v) : 0.f;
      const float dx = dt * xv;
      float y = 0.f;
#pragma unroll
      for (int n = 0; n < NREG; ++n) {
        if (n < N) {
          st[n] = a * st[n] + bc_s[rr][n] * dx;
          y += st[n] * bc_s[rr][NREG + n];
        }
      }
      if (out && live) out[(int64_t)t * P * V + (int64_t)h * V + v] = y + dskip * xv;
    }
  }
  if (slot >= 0 && live) {
#pragma unroll
    for (int n = 0; n < NREG; ++n)
      if (n < N) sp[(int64_t)n * V] = st[n];
  }
  if (dsum && slot >= 0 && lane == 0 && blockIdx.z == 0)
    dsum[(int64_t)slot * P + h] = dt_total;
}

// part [chunks, P, N, V]: end states from zero in, start states out; the
// sequence's final state goes to its slot of `state`.
__global__ __launch_bounds__(256) void mamba2_combine_kernel(
    float* __restrict__ part, const float* __restrict__ dsum,
    const float* __restrict__ rate, float* __restrict__ state,
    const int* __restrict__ chunk_off, const int* __restrict__ cu,
    const int* __restrict__ seq_lens, const int* __restrict__ slots, int P,
    int NV) {
  const int s = blockIdx.y;
  const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (e >= (int64_t)P * NV) return;
  const int h = (int)(e / NV);
  const int rows = cu[s + 1] - cu[s];
  if (rows == 0) return;
  const int start = seq_lens[s] - rows;
  const int slot = slots[s];
  const float r = rate[h];
  float carry =
      (start > 0 && slot >= 0) ? state[(int64_t)slot * P * NV + e] : 0.f;
  for (int k = chunk_off[s]; k < chunk_off[s + 1]; ++k) {
    float* p = part + (int64_t)k * P * NV + e;
    const float local = *p;
    *p = carry;
    carry = expf(-r * dsum[(int64_t)k * P + h]) * carry + local;
  }
  if (slot >= 0) state[(int64_t)slot * P * NV + e] = carry;
}

// out = unit_rms_per_group(y * silu(z)) * w * out_scale; one block per
// (row, group), the gated values of up to 8 * 256 channels stay in
// registers between the two passes.
template <typename AT>
__global__ __launch_bounds__(256) void gate_group_norm_kernel(
    AT* __restrict__ out, int64_t ldo, const float* __restrict__ y,
    const AT* __restrict__ z, int64_t ldz, const float* __restrict__ w,
    float eps, int C, int groups, float out_scale) {
  __shared__ float scratch[4];
  const int t = blockIdx.x, grp = blockIdx.y;
  const int n = C / groups, c0 = grp * n;
  constexpr int KEEP = 8;
  float gv[KEEP];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < KEEP; ++u) {
    const int i = threadIdx.x + 256 * u;
    gv[u] = 0.f;
    if (i < n) {
      gv[u] = y[(int64_t)t * C + c0 + i] *
              silu_f(Act<AT>::ld(z + (int64_t)t * ldz + c0 + i));
      ss += gv[u] * gv[u];
    }
  }
  for (int i = threadIdx.x + 256 * KEEP; i < n; i += 256) {
    const float a = y[(int64_t)t * C + c0 + i] *
                    silu_f(Act<AT>::ld(z + (int64_t)t * ldz + c0 + i));
    ss += a * a;
  }
  ss = block_reduce_sum<256>(ss, scratch);
  const float rstd = out_scale / sqrtf(ss / (float)n + eps);
#pragma unroll
  for (int u = 0; u < KEEP; ++u) {
    const int i = threadIdx.x + 256 * u;
    if (i < n)
      Act<AT>::st(out + (int64_t)t * ldo + c0 + i, gv[u] * rstd * w[c0 + i]);
  }
  for (int i = threadIdx.x + 256 * KEEP; i < n; i += 256) {
    const float a = y[(int64_t)t * C + c0 + i] *
                    silu_f(Act<AT>::ld(z + (int64_t)t * ldz + c0 + i));
    Act<AT>::st(out + (int64_t)t * ldo + c0 + i, a * rstd * w[c0 + i]);
  }
}

}  // namespace arks

using namespace arks;

// Returns 1 when the state size is beyond the kernel's register budget.
extern "C" int arks_seq_mamba2_scan(
    void* out, const void* xbc, int64_t ldx, const void* dt_raw, int64_t ldd,
    const void* dt_bias, const void* rate, const void* Dp, void* state,
    const void* cu, const void* seq_lens, const void* slots, void* dsum, int S,
    int P, int V, int N, int G, int act_f32, hipStream_t stream) {
  if (N > 256 || N < 1 || P % G) return 1;
  if (S == 0) return 0;
  const dim3 grid(S, P, (V + 63) / 64);
#define MB2_LAUNCH(NR)                                                        \
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(                               \
      (mamba2_scan_kernel<AT, NR>), grid, dim3(64), 0, stream, (float*)out,   \
      (const AT*)xbc, ldx, (const AT*)dt_raw, ldd, (const float*)dt_bias,     \
      (const float*)rate, (const float*)Dp, (float*)state, (const int*)cu,    \
      (const int*)seq_lens, (const int*)slots, (float*)dsum, P, V, N, G))
  if (N <= 16) MB2_LAUNCH(16);
  else if (N <= 64) MB2_LAUNCH(64);
  else if (N <= 128) MB2_LAUNCH(128);
  else MB2_LAUNCH(256);
#undef MB2_LAUNCH
  return 0;
}

extern "C" void arks_seq_mamba2_combine(
    void* part, const void* dsum, const void* rate, void* state,
    const void* chunk_off, const void* cu, const void* seq_lens,
    const void* slots, int S, int P, int NV, hipStream_t stream) {
  const int64_t n = (int64_t)P * NV;
  if (S == 0 || n == 0) return;
  hipLaunchKernelGGL(mamba2_combine_kernel,
                     dim3((unsigned)((n + 255) / 256), S), dim3(256), 0, stream,
                     (float*)part, (const float*)dsum, (const float*)rate,
                     (float*)state, (const int*)chunk_off, (const int*)cu,
                     (const int*)seq_lens, (const int*)slots, P, NV);
}

extern "C" void arks_seq_gate_group_norm(void* out, int64_t ldo, const void* y,
                                         const void* z, int64_t ldz,
                                         const void* w, float eps, int T, int C,
                                         int groups, float out_scale,
                                         int act_f32, hipStream_t stream) {
  if (T == 0) return;
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (gate_group_norm_kernel<AT>), dim3(T, groups), dim3(256), 0, stream,
      (AT*)out, ldo, (const float*)y, (const AT*)z, ldz, (const float*)w, eps,
      C, groups, out_scale));
}
