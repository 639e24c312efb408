// Mamba2 mixer kernels: the scalar-decay state-space recurrence
//   S_h <- exp(-rate_h dt_h) S_h + dt_h B_g x_h^T      (S_h: N x V, fp32)
//   y_h = S_h^T C_g + D_h x_h,      dt = softplus(dt_raw + dt_bias)
// over rows [x | B | C] that already went through the short convolution
// (seq_mamba.hip causal_conv_silu), and the gated group norm behind it.
// Head h reads group g = h / (P / G) of B and C.
//
// Scan: lane v keeps (a part of) column S[:, v] in registers, so y needs no
// reduction across lanes. B and C of MB2_ROWS rows at a time are staged in
// LDS (every lane reads all of them). With `out` null only the end state and the summed step
// sizes are produced (pass 1 of the chunk-parallel prefill); the combine
// kernel then turns every chunk's end-from-zero state into its start state
// and leaves the sequence's final state in its slot.
#include "seq_common.h"

namespace arks {

constexpr int MB2_ROWS = 16;

// One workgroup = SPLIT waves per (sequence or chunk, HP heads of one group,
// 64 value columns): wave w keeps state rows [w * NR, (w + 1) * NR) of
// column v of each of its HP heads in lane v's registers; the waves'
// partial outputs of a block of rows meet in LDS. Heads of one group read
// the same B and C, so HP > 1 divides the LDS reads per multiply-add (it
// also halves the waves per SIMD, and measured slower: the launcher uses
// HP = 1). FULL: N == NR * SPLIT, no bound checks on the rows.
template <typename AT, int NR, int SPLIT, int HP, bool FULL>
__global__ __launch_bounds__(64 * SPLIT) void mamba2_scan_kernel(
    float* __restrict__ out, const AT* __restrict__ xbc, int64_t ldx,
    const AT* __restrict__ dt_raw, int64_t ldd,
    const float* __restrict__ dt_bias, const float* __restrict__ rate,
    const float* __restrict__ Dp, float* __restrict__ state,
    const int* __restrict__ cu, const int* __restrict__ seq_lens,
    const int* __restrict__ slots, float* __restrict__ dsum, int P, int V,
    int N, int G) {
  constexpr int NTOT = NR * SPLIT;
  constexpr int THREADS = 64 * SPLIT;
  __shared__ __attribute__((aligned(16))) float bc_s[MB2_ROWS][2 * NTOT];
  __shared__ float dt_s[MB2_ROWS][HP];
  __shared__ float x_s[MB2_ROWS][HP][64];
  __shared__ float y_s[SPLIT > 1 ? SPLIT : 1][MB2_ROWS][HP][64];
  const int s = blockIdx.x, h0 = blockIdx.y * HP;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int v = blockIdx.z * 64 + lane;
  const bool live = v < V;
  const int first = cu[s], rows = cu[s + 1] - first;
  if (rows == 0) return;
  const int start = seq_lens[s] - rows;
  const int slot = slots[s];
  const int g = h0 / (P / G);
  const int n0 = wave * NR;
  float r[HP], dskip[HP], dt_total[HP];
  float st[HP][NR];
  const bool resume = start > 0 && slot >= 0 && live;
  float* sp =
      state + (((int64_t)(slot < 0 ? 0 : slot) * P + h0) * N + n0) * V + v;
#pragma unroll
  for (int hp = 0; hp < HP; ++hp) {
    r[hp] = rate[h0 + hp];
    dskip[hp] = Dp[h0 + hp];
    dt_total[hp] = 0.f;
#pragma unroll
    for (int n = 0; n < NR; ++n)
      st[hp][n] = (resume && n0 + n < N)
                      ? sp[((int64_t)hp * N + n) * V] : 0.f;
  }
  const int64_t boff = (int64_t)P * V + (int64_t)g * N;
  const int64_t coff = boff + (int64_t)G * N;
  for (int r0 = 0; r0 < rows; r0 += MB2_ROWS) {
    const int nr = min(MB2_ROWS, rows - r0);
    __syncthreads();  // the previous rows' readers are done
    // without outputs only B is needed
    const int ncol = out ? 2 * N : N;
    for (int i = threadIdx.x; i < nr * ncol; i += THREADS) {
      const int rr = i / ncol, c = i % ncol;
      const AT* row = xbc + (int64_t)(first + r0 + rr) * ldx;
      bc_s[rr][c < N ? c : NTOT + c - N] =
          Act<AT>::ld(row + (c < N ? boff + c : coff + c - N));
    }
    // this block's x rows too: a load from memory inside the row loop
    // would expose its latency once per row
    for (int i = threadIdx.x; i < nr * HP * 64; i += THREADS) {
      const int rr = i / (HP * 64), hp = (i / 64) % HP, l = i % 64;
      const int vv = blockIdx.z * 64 + l;
      x_s[rr][hp][l] =
          vv < V ? Act<AT>::ld(xbc + (int64_t)(first + r0 + rr) * ldx +
                               (int64_t)(h0 + hp) * V + vv) : 0.f;
    }
    if (threadIdx.x < nr * HP) {
      const int rr = threadIdx.x / HP, hp = threadIdx.x % HP;
      dt_s[rr][hp] = softplus_f(
          Act<AT>::ld(dt_raw + (int64_t)(first + r0 + rr) * ldd + h0 + hp) +
          dt_bias[h0 + hp]);
    }
    __syncthreads();
    for (int rr = 0; rr < nr; ++rr) {
      const int t = first + r0 + rr;
      float a[HP], dx[HP], xv[HP], y[HP];
#pragma unroll
      for (int hp = 0; hp < HP; ++hp) {
        const float dt = dt_s[rr][hp];
        a[hp] = expf(-r[hp] * dt);
        dt_total[hp] += dt;
        xv[hp] = x_s[rr][hp][lane];
        dx[hp] = dt * xv[hp];
        y[hp] = 0.f;
      }
      const float* bs = &bc_s[rr][n0];
      const float* cs = &bc_s[rr][NTOT + n0];
      if (out) {
#pragma unroll
        for (int n = 0; n < NR; ++n) {
          if (FULL || n0 + n < N) {
            const float bn = bs[n], cn = cs[n];
#pragma unroll
            for (int hp = 0; hp < HP; ++hp) {
              st[hp][n] = fmaf(a[hp], st[hp][n], bn * dx[hp]);
              y[hp] = fmaf(st[hp][n], cn, y[hp]);
            }
          }
        }
#pragma unroll
        for (int hp = 0; hp < HP; ++hp) {
          if (SPLIT == 1) {
            if (live)
              out[(int64_t)t * P * V + (int64_t)(h0 + hp) * V + v] =
                  y[hp] + dskip[hp] * xv[hp];
          } else {
            y_s[wave][rr][hp][lane] =
                wave == 0 ? y[hp] + dskip[hp] * xv[hp] : y[hp];
          }
        }
      } else {
#pragma unroll
        for (int n = 0; n < NR; ++n) {
          if (FULL || n0 + n < N) {
            const float bn = bs[n];
#pragma unroll
            for (int hp = 0; hp < HP; ++hp)
              st[hp][n] = fmaf(a[hp], st[hp][n], bn * dx[hp]);
          }
        }
      }
    }
    if (SPLIT > 1 && out) {
      __syncthreads();
      for (int i = wave; i < nr * HP; i += SPLIT) {
        const int rr = i / HP, hp = i % HP;
        float y = 0.f;
#pragma unroll
        for (int w = 0; w < SPLIT; ++w) y += y_s[w][rr][hp][lane];
        if (live)
          out[(int64_t)(first + r0 + rr) * P * V + (int64_t)(h0 + hp) * V + v] = y;
      }
    }
  }
  if (slot >= 0 && live) {
#pragma unroll
    for (int hp = 0; hp < HP; ++hp)
#pragma unroll
      for (int n = 0; n < NR; ++n)
        if (n0 + n < N) sp[((int64_t)hp * N + n) * V] = st[hp][n];
  }
  if (dsum && slot >= 0 && threadIdx.x == 0 && blockIdx.z == 0) {
#pragma unroll
    for (int hp = 0; hp < HP; ++hp)
      dsum[(int64_t)slot * P + h0 + hp] = dt_total[hp];
  }
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

// bf16 rows, 4 channels per thread (group size % 4 == 0, aligned rows): the
// gated values of up to 2048 channels of the group stay in registers.
__global__ __launch_bounds__(256) void gate_group_norm_vec4_kernel(
    bf16* __restrict__ out, int64_t ldo, const float* __restrict__ y,
    const bf16* __restrict__ z, int64_t ldz, const float* __restrict__ w,
    float eps, int C, int groups, float out_scale) {
  __shared__ float scratch[4];
  const int t = blockIdx.x, grp = blockIdx.y;
  const int n = C / groups, c0 = grp * n;
  constexpr int KEEP = 2;
  float gv[KEEP][4];
  float ss = 0.f;
  auto gated = [&](int i, float (&g)[4]) {
    const float4v yv =
        *reinterpret_cast<const float4v*>(y + (int64_t)t * C + c0 + i);
    const ushort4v zv =
        *reinterpret_cast<const ushort4v*>(z + (int64_t)t * ldz + c0 + i);
#pragma unroll
    for (int e = 0; e < 4; ++e) g[e] = yv[e] * silu_f(bf16_bits_to_float(zv[e]));
  };
#pragma unroll
  for (int u = 0; u < KEEP; ++u) {
    const int i = (threadIdx.x + 256 * u) * 4;
#pragma unroll
    for (int e = 0; e < 4; ++e) gv[u][e] = 0.f;
    if (i < n) {
      gated(i, gv[u]);
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += gv[u][e] * gv[u][e];
    }
  }
  for (int i = (threadIdx.x + 256 * KEEP) * 4; i < n; i += 1024) {
    float g[4];
    gated(i, g);
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += g[e] * g[e];
  }
  ss = block_reduce_sum<256>(ss, scratch);
  const float rstd = out_scale / sqrtf(ss / (float)n + eps);
  auto put = [&](int i, const float (&g)[4]) {
    const float4v wv = *reinterpret_cast<const float4v*>(w + c0 + i);
    ushort4v o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = float_to_bf16_bits(g[e] * rstd * wv[e]);
    *reinterpret_cast<ushort4v*>(out + (int64_t)t * ldo + c0 + i) = o;
  };
#pragma unroll
  for (int u = 0; u < KEEP; ++u) {
    const int i = (threadIdx.x + 256 * u) * 4;
    if (i < n) put(i, gv[u]);
  }
  for (int i = (threadIdx.x + 256 * KEEP) * 4; i < n; i += 1024) {
    float g[4];
    gated(i, g);
    put(i, g);
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
  // heads per lane: heads of one group share B and C
  // measured on gfx950 (16384 rows, 128 heads x 64, state 128): one head
  // per lane with 32 state rows a lane runs both passes in 4.3 ms; two
  // heads per lane 5.5 ms, 64 rows a lane 5.8 ms (fewer waves per SIMD)
  const int hp = 1;
  const dim3 grid(S, P / hp, (V + 63) / 64);
#define MB2_ARGS                                                              \
  (float*)out, (const AT*)xbc, ldx, (const AT*)dt_raw, ldd,                   \
      (const float*)dt_bias, (const float*)rate, (const float*)Dp,            \
      (float*)state, (const int*)cu, (const int*)seq_lens, (const int*)slots, \
      (float*)dsum, P, V, N, G
#define MB2_LAUNCH3(NR, SPLIT, HP, FULL)                                      \
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(                               \
      (mamba2_scan_kernel<AT, NR, SPLIT, HP, FULL>), grid, dim3(64 * SPLIT),  \
      0, stream, MB2_ARGS))
#define MB2_LAUNCH(NR, SPLIT)                                                 \
  do {                                                                        \
    if (N == NR * SPLIT) MB2_LAUNCH3(NR, SPLIT, 1, true);                     \
    else MB2_LAUNCH3(NR, SPLIT, 1, false);                                    \
  } while (0)
  if (N <= 16) MB2_LAUNCH(16, 1);
  else if (N <= 64) MB2_LAUNCH(32, 2);
  else if (N <= 128) MB2_LAUNCH(32, 4);
  else MB2_LAUNCH(64, 4);
#undef MB2_LAUNCH
#undef MB2_LAUNCH3
#undef MB2_ARGS
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
  const int n = C / groups;
  if (!act_f32 && n % 4 == 0 && ldz % 4 == 0 && ldo % 4 == 0 && C % 4 == 0 &&
      ((uintptr_t)y & 15) == 0 && ((uintptr_t)w & 15) == 0 &&
      ((uintptr_t)z & 7) == 0 && ((uintptr_t)out & 7) == 0) {
    hipLaunchKernelGGL(gate_group_norm_vec4_kernel, dim3(T, groups), dim3(256),
                       0, stream, (bf16*)out, ldo, (const float*)y,
                       (const bf16*)z, ldz, (const float*)w, eps, C, groups,
                       out_scale);
    return;
  }
  SEQ_DISPATCH_ACT(act_f32, hipLaunchKernelGGL(
      (gate_group_norm_kernel<AT>), dim3(T, groups), dim3(256), 0, stream,
      (AT*)out, ldo, (const float*)y, (const AT*)z, ldz, (const float*)w, eps,
      C, groups, out_scale));
}
