// Masked softmax attention over paged keys on the matrix cores (bf16 rows
// and pages of 16 tokens, gfx950): the fast path of
// ops.attention_sink_paged for capped scores, sliding windows that keep the
// first keys, per-head sinks, and caches whose value is a leading part of
// the key's row (seq_attention.hip holds the general kernel and the exact
// definition). Built on the tiling of seq_window_mfma.hip: keys pass
// through LDS 32 at a time (K rows XOR-swizzled where the row length
// allows, V as a transposed-read image), both products run on
// v_mfma_f32_16x16x32_bf16, the softmax is online and fp32.
//
// What is new here:
//   * a tile's 64 score columns are (position, head) pairs: HPT heads of
//     one key/value head's group side by side for 64 / HPT consecutive
//     positions. With many query heads on one key/value head (latent
//     attention has ONE) the keys are staged once for all of them; with one
//     head per group the tile is 64 positions of that head;
//   * masks per (column, key): key j for the column at position i iff
//     j <= i and (i - j < window or j < keep_first); a tile walks the key
//     tiles that hold kept keys, then those from its oldest row's window on;
//   * scores may be capped, s <- c tanh(s / c), and the running softmax may
//     start from a sink (max sink[h], sum 1);
//   * key and value rows have strides of their own (ldk, ldv);
//   * no host work list: a workgroup finds its (sequence, first position)
//     by walking cu_seqlens, or — steps of single rows — from token_seq;
//   * a cache row may hold several keys side by side that share its value
//     (MaskArgs::maps): each is a key group of its own with its own heads.
#include "seq_common.h"

#include <cfloat>

namespace arks {

typedef __attribute__((ext_vector_type(8))) __bf16 mk_bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 mk_bf16x4;
typedef __attribute__((ext_vector_type(4))) float mk_f32x4;

constexpr int MK_QTILE = 64;
constexpr int MK_KTILE = 32;
constexpr int MK_PAGE = 16;
constexpr int MK_PPAD = 40;

__device__ __forceinline__ float mk_cap(float s, float cap, float inv_cap) {
  // cap * tanh(s / cap), tanh(z) = 1 - 2 / (e^{2z} + 1)
  const float z = fminf(fmaxf(s * inv_cap, -15.f), 15.f);
  return cap * (1.f - 2.f / (__expf(2.f * z) + 1.f));
}

struct MaskArgs {
  float scale, softcap, out_scale;
  int window, keep_first;  // window: INT_MAX / 2 when there is none
  // key maps per cache row: a row holds `maps` keys of D dims side by side
  // that share the row's value; the kernels' G counts (key/value head, map)
  // groups, group g reads key g % maps of the rows of head g / maps
  int maps;
};

template <int D, int V>  // V: the value columns one workgroup holds
struct MaskedTileLds {
  static constexpr int K_BYTES = MK_KTILE * D * 2;
  static constexpr int VT_BYTES = (V / 16) * 8 * 96 * 2;
  static constexpr int P_BYTES = 4 * 16 * MK_PPAD * 2;
  static constexpr int BYTES = K_BYTES + VT_BYTES + P_BYTES;
};

// SHR: the value is the leading part of the key's row (one cache, equal
// strides), so a tile's rows are loaded once.
// VS > 1: the value columns are cut into VS parts, one workgroup each (all
// of them compute the scores): long value rows then need fewer registers
// and less LDS per workgroup, so several fit a CU and hide each other's
// load latency.
template <int D, int VFULL, bool SINGLE, bool SHR, int VS>
__global__ __launch_bounds__(
    256, VS > 1 ? 2 : (D + VFULL <= 256 ? 3 : (D + VFULL <= 384 ? 2 : 1)))
void attn_masked_tile_kernel(
    bf16* __restrict__ out, int64_t ldo, const bf16* __restrict__ q,
    const bf16* __restrict__ k_cache, int64_t ldk,
    const bf16* __restrict__ v_cache, int64_t ldv,
    const int* __restrict__ block_tables, const int* __restrict__ kv_lens,
    const int* __restrict__ cu, const int* __restrict__ token_seq,
    const float* __restrict__ sink_w, int num_seqs, MaskArgs a, int G, int H,
    int hpt_shift, int max_blocks, float* __restrict__ ws) {
  constexpr int V = VFULL / VS;  // this workgroup's value columns
  constexpr int STEPS = D / 32;
  constexpr int CHUNKS = V / 16;
  constexpr int SWZ = (D % 64 == 0) ? 1 : 0;
  const int voff = (blockIdx.x % VS) * V;
  // gridDim.z > 1: workgroup z takes every gridDim.z-th key tile and leaves
  // (output sums, max, sum) per column in ws for the combine kernel
  const int ks = gridDim.z, kz = blockIdx.z;
  using Lds = MaskedTileLds<D, V>;
  extern __shared__ __attribute__((aligned(16))) char mk_smem[];
  bf16* k_lds = reinterpret_cast<bf16*>(mk_smem);                 // [32][D]
  bf16* vt_img = reinterpret_cast<bf16*>(mk_smem + Lds::K_BYTES);  // [V/16][8][96]
  bf16* p_lds = reinterpret_cast<bf16*>(mk_smem + Lds::K_BYTES + Lds::VT_BYTES);

  const int HPT = 1 << hpt_shift;        // heads per tile
  const int PPT = MK_QTILE >> hpt_shift;  // positions per tile
  int seq_idx = -1, p0 = 0;
  if (SINGLE) {
    seq_idx = token_seq[blockIdx.y];
    p0 = blockIdx.y - cu[seq_idx];
  } else {
    // the last tiles of a sequence see the most keys: they start first, so
    // the launch ends on short tiles
    int left = gridDim.y - 1 - blockIdx.y;
    for (int s = 0; s < num_seqs; ++s) {
      const int n = (cu[s + 1] - cu[s] + PPT - 1) / PPT;
      if (left < n) {
        seq_idx = s;
        p0 = left * PPT;
        break;
      }
      left -= n;
    }
  }
  if (seq_idx < 0) return;
  const int GQ = H / G;
  const int hblocks = GQ >> hpt_shift;  // head blocks per key/value head
  const int kvh = (blockIdx.x / VS) / hblocks;
  const int h0 = kvh * GQ + ((blockIdx.x / VS) % hblocks) * HPT;
  const int GR = G / a.maps, kvr = kvh / a.maps;  // heads of rows, this one
  const bf16* __restrict__ k_rows = k_cache + (kvh % a.maps) * D;
  const int q_start = cu[seq_idx];
  const int q_len = cu[seq_idx + 1] - q_start;
  const int kv_len = kv_lens[seq_idx];
  const int kv_off = kv_len - q_len;
  const int n_pos = SINGLE ? 1 : min(PPT, q_len - p0);
  const int* __restrict__ bt = block_tables + (int64_t)seq_idx * max_blocks;

  const int tid = threadIdx.x;
  const int wave = tid / WAVE_SIZE, lane = tid % WAVE_SIZE;
  const int lq = lane % 16, la = lane / 16;

  // this lane's score column
  const int col = wave * 16 + lq;
  const int my_p = col >> hpt_shift;
  const bool col_valid = my_p < n_pos;
  const int h = h0 + (col & (HPT - 1));
  const int my_pos = kv_off + p0 + (col_valid ? my_p : 0);
  const bool wave_active = wave * 16 < n_pos * HPT;
  mk_bf16x8 qfrag[STEPS];
  {
    const int64_t qbase =
        ((int64_t)(q_start + p0 + (col_valid ? my_p : 0)) * H + h) * D;
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      ushort8 u = *reinterpret_cast<const ushort8*>(q + qbase + st * 32 + 8 * la);
      qfrag[st] = *reinterpret_cast<mk_bf16x8*>(&u);
    }
  }
  const float inv_cap = a.softcap > 0.f ? 1.f / a.softcap : 0.f;
  const bool sunk = sink_w != nullptr && kz == 0;
  float m_run = sunk ? sink_w[h] : -FLT_MAX;
  float l_run = sunk ? 1.f : 0.f;
  mk_f32x4 oacc[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) oacc[c] = {0.f, 0.f, 0.f, 0.f};

  const int first_pos = kv_off + p0, last_pos = first_pos + n_pos - 1;
  const int kmax = last_pos + 1;
  const int tok_tiles = (kmax + MK_KTILE - 1) / MK_KTILE;
  const int keep_tiles =
      (min(a.keep_first, kmax) + MK_KTILE - 1) / MK_KTILE;
  const int tok_j0 =
      max(keep_tiles, max(0, first_pos - a.window + 1) / MK_KTILE);
  const int n_iter = keep_tiles + max(0, tok_tiles - tok_j0);

  // A tile's rows travel global -> registers -> LDS. The loads of the next
  // tile are issued right after this tile's rows reach LDS, so they fly
  // while the tile is computed: with one or two workgroups on a CU nothing
  // else would hide their latency. The tile's two pages are looked up once.
  constexpr int KIT = (MK_KTILE * (D / 8) + 255) / 256;
  constexpr int VIT = SHR ? 1 : (MK_KTILE * (V / 8) + 255) / 256;
  ushort8 kld[KIT], vld[VIT];
  auto tile_base = [&](int it) {
    return (it < keep_tiles ? it : tok_j0 + it - keep_tiles) * MK_KTILE;
  };
  auto load_tile = [&](int it) {
    const int key_base = tile_base(it);
    const int pg0 = bt[key_base / MK_PAGE];
    const int pg1 =
        key_base + MK_PAGE < kmax ? bt[key_base / MK_PAGE + 1] : 0;
#pragma unroll
    for (int j = 0; j < KIT; ++j) {
      const int i = tid + 256 * j;
      const int key = i / (D / 8);
      const int col8 = (i % (D / 8)) * 8;
      const int kg = key_base + key;
      ushort8 kv{};
      if (i < MK_KTILE * (D / 8) && kg < kmax) {
        const int64_t row =
            ((int64_t)(key < MK_PAGE ? pg0 : pg1) * GR + kvr) * MK_PAGE +
            kg % MK_PAGE;
        kv = *reinterpret_cast<const ushort8*>(k_rows + row * ldk + col8);
      }
      kld[j] = kv;
    }
    if (!SHR) {
#pragma unroll
      for (int j = 0; j < VIT; ++j) {
        const int i = tid + 256 * j;
        const int key = i / (V / 8);
        const int col8 = (i % (V / 8)) * 8;
        const int kg = key_base + key;
        ushort8 vv{};
        if (i < MK_KTILE * (V / 8) && kg < kmax) {
          const int64_t row =
              ((int64_t)(key < MK_PAGE ? pg0 : pg1) * GR + kvr) * MK_PAGE +
              kg % MK_PAGE;
          vv = *reinterpret_cast<const ushort8*>(v_cache + row * ldv + voff +
                                                 col8);
        }
        vld[j] = vv;
      }
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int j = 0; j < KIT; ++j) {
      const int i = tid + 256 * j;
      const int key = i / (D / 8);
      const int col8 = (i % (D / 8)) * 8;
      if (i < MK_KTILE * (D / 8)) {
        const int swz = (col8 * 2) ^ (SWZ * ((key & 7) << 4));
        *reinterpret_cast<ushort8*>(
            reinterpret_cast<char*>(k_lds + key * D) + swz) = kld[j];
        // the value is the leading part of the key's row: no second load
        if (SHR && col8 >= voff && col8 < voff + V) {
          const int vc = col8 - voff;
          *reinterpret_cast<ushort8*>(
              &vt_img[((vc >> 4) * 8 + (key >> 2)) * 96 + (key & 3) * 16 +
                      (vc & 15)]) = kld[j];
        }
      }
    }
    if (!SHR) {
#pragma unroll
      for (int j = 0; j < VIT; ++j) {
        const int i = tid + 256 * j;
        const int key = i / (V / 8);
        const int col8 = (i % (V / 8)) * 8;
        if (i < MK_KTILE * (V / 8))
          *reinterpret_cast<ushort8*>(
              &vt_img[((col8 >> 4) * 8 + (key >> 2)) * 96 + (key & 3) * 16 +
                      (col8 & 15)]) = vld[j];
      }
    }
  };
  if (kz < n_iter) load_tile(kz);

  for (int it = kz; it < n_iter; it += ks) {
    const int key_base = tile_base(it);
    store_tile();
    __syncthreads();
    if (it + ks < n_iter) load_tile(it + ks);

    if (wave_active) {
      mk_f32x4 sc[2];
      sc[0] = {0.f, 0.f, 0.f, 0.f};
      sc[1] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
        const int key = sub * 16 + lq;
#pragma unroll
        for (int st = 0; st < STEPS; ++st) {
          const int col_byte = (st * 32 + 8 * la) * 2;
          const int swz = col_byte ^ (SWZ * ((key & 7) << 4));
          ushort8 u = *reinterpret_cast<const ushort8*>(
              reinterpret_cast<const char*>(k_lds + key * D) + swz);
          sc[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              *reinterpret_cast<mk_bf16x8*>(&u), qfrag[st], sc[sub], 0, 0, 0);
        }
      }
      float p[8];
      bool msk[8];
      float tile_max = -FLT_MAX;
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int kg = key_base + sub * 16 + 4 * la + r;
          const int i = sub * 4 + r;
          msk[i] = col_valid && kg <= my_pos &&
                   (kg > my_pos - a.window || kg < a.keep_first);
          float s = sc[sub][r] * a.scale;
          if (a.softcap > 0.f) s = mk_cap(s, a.softcap, inv_cap);
          p[i] = msk[i] ? s : -FLT_MAX;
          tile_max = fmaxf(tile_max, p[i]);
        }
      }
      tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, WAVE_SIZE));
      tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, WAVE_SIZE));
      const float m_new = fmaxf(m_run, tile_max);
      float alpha = 1.f, psum = 0.f;
      if (m_new > -FLT_MAX) {
        alpha = __expf(m_run - m_new);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          p[i] = msk[i] ? __expf(p[i] - m_new) : 0.f;
          psum += p[i];
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) p[i] = 0.f;
      }
      psum += __shfl_xor(psum, 16, WAVE_SIZE);
      psum += __shfl_xor(psum, 32, WAVE_SIZE);
      l_run = l_run * alpha + psum;
      m_run = m_new;

      float row_alpha[4];
#pragma unroll
      for (int r = 0; r < 4; ++r)
        row_alpha[r] = __shfl(alpha, 4 * la + r, WAVE_SIZE);
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
        for (int r = 0; r < 4; ++r) oacc[c][r] *= row_alpha[r];
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
        ushort4v pk;
#pragma unroll
        for (int r = 0; r < 4; ++r) pk[r] = float_to_bf16_bits(p[sub * 4 + r]);
        *reinterpret_cast<ushort4v*>(
            &p_lds[(wave * 16 + lq) * MK_PPAD + sub * 16 + 4 * la]) = pk;
      }
    }
    __syncthreads();

    if (wave_active) {
      ushort8 pa = *reinterpret_cast<const ushort8*>(
          &p_lds[(wave * 16 + lq) * MK_PPAD + 8 * la]);
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c) {
        mk_bf16x4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
            (__attribute__((address_space(3))) mk_bf16x4*)(
                reinterpret_cast<char*>(&vt_img[(c * 8 + 2 * la) * 96]) + lq * 8));
        mk_bf16x4 v2 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
            (__attribute__((address_space(3))) mk_bf16x4*)(
                reinterpret_cast<char*>(&vt_img[(c * 8 + 2 * la + 1) * 96]) +
                lq * 8));
        mk_bf16x8 vb;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          vb[e] = v1[e];
          vb[e + 4] = v2[e];
        }
        oacc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            *reinterpret_cast<mk_bf16x8*>(&pa), vb, oacc[c], 0, 0, 0);
      }
    }
    __syncthreads();
  }

  if (ks > 1) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int c2 = wave * 16 + 4 * la + r;
      const int pp = c2 >> hpt_shift;
      const float mr = __shfl(m_run, 4 * la + r, WAVE_SIZE);
      const float lr = __shfl(l_run, 4 * la + r, WAVE_SIZE);
      if (pp >= n_pos) continue;
      float* wp = ws + (((int64_t)(q_start + p0 + pp) * H + h0 +
                         (c2 & (HPT - 1))) * ks + kz) * (VFULL + 2);
#pragma unroll
      for (int c = 0; c < CHUNKS; ++c) wp[voff + c * 16 + lq] = oacc[c][r];
      if (lq == 0 && voff == 0) {
        wp[VFULL] = mr;
        wp[VFULL + 1] = lr;
      }
    }
    return;
  }
  float row_inv[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float lr = __shfl(l_run, 4 * la + r, WAVE_SIZE);
    row_inv[r] = lr > 0.f ? a.out_scale / lr : 0.f;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int c2 = wave * 16 + 4 * la + r;  // column of the tile
    const int pp = c2 >> hpt_shift;
    if (pp >= n_pos) continue;
    const int64_t obase = (int64_t)(q_start + p0 + pp) * ldo +
                          (int64_t)(h0 + (c2 & (HPT - 1))) * VFULL + voff;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
      out[obase + c * 16 + lq] = float_to_bf16_bits(oacc[c][r] * row_inv[r]);
  }
}

// Merge the key-split partials of one (row, head): ws [T, H, ks, V + 2].
__global__ __launch_bounds__(64) void attn_masked_combine_kernel(
    bf16* __restrict__ out, int64_t ldo, const float* __restrict__ ws, int H,
    int V, int ks, float out_scale) {
  const int t = blockIdx.x, h = blockIdx.y;
  const float* wp = ws + ((int64_t)t * H + h) * ks * (V + 2);
  float m = -FLT_MAX;
  for (int z = 0; z < ks; ++z) m = fmaxf(m, wp[z * (V + 2) + V]);
  float l = 0.f;
  for (int z = 0; z < ks; ++z)
    l += wp[z * (V + 2) + V + 1] * __expf(wp[z * (V + 2) + V] - m);
  const float inv = l > 0.f ? out_scale / l : 0.f;
  for (int d = threadIdx.x; d < V; d += 64) {
    float acc = 0.f;
    for (int z = 0; z < ks; ++z)
      acc += wp[z * (V + 2) + d] * __expf(wp[z * (V + 2) + V] - m);
    out[(int64_t)t * ldo + (int64_t)h * V + d] = float_to_bf16_bits(acc * inv);
  }
}

// Single rows, groups of up to 16 query heads: one workgroup per (row,
// key/value head) whose four waves each take every fourth visible 32-key
// tile with no barrier between tiles — K from the pages straight into the
// MFMA A operand, V through a per-wave transposed-read image, P through a
// per-wave tile — and merge their (max, sum, output) partials through LDS.
// The sink, counted once, starts wave 0's running softmax.
template <int D, int V>
__global__ __launch_bounds__(256, 2) void attn_masked_dec_kernel(
    bf16* __restrict__ out, int64_t ldo, const bf16* __restrict__ q,
    const bf16* __restrict__ k_cache, int64_t ldk,
    const bf16* __restrict__ v_cache, int64_t ldv,
    const int* __restrict__ block_tables, const int* __restrict__ kv_lens,
    const int* __restrict__ cu, const int* __restrict__ token_seq,
    const float* __restrict__ sink_w, MaskArgs a, int G, int H,
    int max_blocks) {
  constexpr int STEPS = D / 32;
  constexpr int CHUNKS = V / 16;
  constexpr int E = V / 16;  // value dims per thread in the merge
  const int t = blockIdx.y, kvh = blockIdx.x;
  const int GQ = H / G;
  const int GR = G / a.maps, kvr = kvh / a.maps;
  const bf16* __restrict__ k_rows = k_cache + (kvh % a.maps) * D;
  const int seq = token_seq[t];
  const int q_start = cu[seq];
  const int pos = kv_lens[seq] - (cu[seq + 1] - q_start) + (t - q_start);
  const int* __restrict__ bt = block_tables + (int64_t)seq * max_blocks;
  const int tid = threadIdx.x;
  const int wave = tid / WAVE_SIZE, lane = tid % WAVE_SIZE;
  const int lq = lane % 16, la = lane / 16;

  constexpr int VT_BYTES = (V / 16) * 8 * 96 * 2;
  constexpr int P_BYTES = 16 * MK_PPAD * 2;
  constexpr int MERGE_BYTES = 16 * (V + 2) * 4;
  constexpr int WAVE_BYTES0 =
      VT_BYTES + P_BYTES > MERGE_BYTES ? VT_BYTES + P_BYTES : MERGE_BYTES;
  constexpr int WAVE_BYTES = (WAVE_BYTES0 + 15) & ~15;
  __shared__ __attribute__((aligned(16))) char smem[4][WAVE_BYTES];
  bf16* vt_lds = reinterpret_cast<bf16*>(smem[wave]);
  bf16* p_lds = reinterpret_cast<bf16*>(smem[wave] + VT_BYTES);
  float* merge_lds = reinterpret_cast<float*>(smem[wave]);

  const bool head_valid = lq < GQ;
  mk_bf16x8 qfrag[STEPS];
  {
    const bf16* qp =
        q + ((int64_t)t * H + kvh * GQ + (head_valid ? lq : 0)) * D;
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      ushort8 u{};
      if (head_valid) u = *reinterpret_cast<const ushort8*>(qp + st * 32 + 8 * la);
      qfrag[st] = *reinterpret_cast<mk_bf16x8*>(&u);
    }
  }
  const float inv_cap = a.softcap > 0.f ? 1.f / a.softcap : 0.f;
  const bool sunk = sink_w != nullptr && wave == 0 && head_valid;
  float m_run = sunk ? sink_w[kvh * GQ + lq] : -FLT_MAX;
  float l_run = sunk ? 1.f : 0.f;
  mk_f32x4 oacc[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) oacc[c] = {0.f, 0.f, 0.f, 0.f};

  const int kmax = pos + 1;
  const int tok_tiles = (kmax + MK_KTILE - 1) / MK_KTILE;
  const int keep_tiles = (min(a.keep_first, kmax) + MK_KTILE - 1) / MK_KTILE;
  const int tok_j0 = max(keep_tiles, max(0, pos - a.window + 1) / MK_KTILE);
  const int n_iter = keep_tiles + max(0, tok_tiles - tok_j0);
  // A tile is two pages. Their ids are looked up two tiles ahead of use
  // and handed to the loads as values: a lookup inside the load would be a
  // dependent chain (id, then rows) that one tile of compute cannot hide.
  auto tile_base = [&](int it) {
    return (it < keep_tiles ? it : tok_j0 + it - keep_tiles) * MK_KTILE;
  };
  auto tile_pages = [&](int it, int& p0, int& p1) {
    const int key_base = tile_base(it);
    p0 = (it < n_iter && key_base < kmax) ? bt[key_base / MK_PAGE] : 0;
    p1 = (it < n_iter && key_base + MK_PAGE < kmax)
             ? bt[key_base / MK_PAGE + 1] : 0;
  };
  constexpr int NV = MK_KTILE * V / 8 / WAVE_SIZE;

  auto load_tile = [&](int it, int p0, int p1, ushort8 (&kr)[2][STEPS],
                       ushort8 (&vr)[NV]) {
    const int key_base = tile_base(it);
    auto row_of = [&](int key) -> int64_t {  // key within the tile
      return ((int64_t)(key < MK_PAGE ? p0 : p1) * GR + kvr) * MK_PAGE +
             key % MK_PAGE;
    };
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = lane + WAVE_SIZE * j;
      const int key = i / (V / 8);
      const int col8 = (i % (V / 8)) * 8;
      ushort8 v{};
      if (key_base + key < kmax)
        v = *reinterpret_cast<const ushort8*>(v_cache + row_of(key) * ldv +
                                              col8);
      vr[j] = v;
    }
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int key = sub * 16 + lq;
      const bool have = key_base + key < kmax;
      const bf16* krow = k_rows + (have ? row_of(key) : 0) * ldk + 8 * la;
#pragma unroll
      for (int st = 0; st < STEPS; ++st) {
        ushort8 u{};
        if (have) u = *reinterpret_cast<const ushort8*>(krow + st * 32);
        kr[sub][st] = u;
      }
    }
  };
  ushort8 kreg[2][STEPS], vv[NV];
  int cp0, cp1, np0, np1;
  tile_pages(wave, cp0, cp1);
  tile_pages(wave + 4, np0, np1);
  if (wave < n_iter) load_tile(wave, cp0, cp1, kreg, vv);

  for (int it = wave; it < n_iter; it += 4) {
    const int key_base = tile_base(it);
    int nnp0, nnp1;
    tile_pages(it + 8, nnp0, nnp1);
    ushort8 knext[2][STEPS], vnext[NV];
    if (it + 4 < n_iter) load_tile(it + 4, np0, np1, knext, vnext);
    np0 = nnp0;
    np1 = nnp1;
    mk_f32x4 sc[2];
    sc[0] = {0.f, 0.f, 0.f, 0.f};
    sc[1] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
#pragma unroll
      for (int st = 0; st < STEPS; ++st)
        sc[sub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            *reinterpret_cast<mk_bf16x8*>(&kreg[sub][st]), qfrag[st], sc[sub],
            0, 0, 0);
    float p[8];
    float tile_max = -FLT_MAX;
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int kg = key_base + sub * 16 + 4 * la + r;
        const int i = sub * 4 + r;
        const bool vis =
            kg <= pos && (kg > pos - a.window || kg < a.keep_first);
        float s = sc[sub][r] * a.scale;
        if (a.softcap > 0.f) s = mk_cap(s, a.softcap, inv_cap);
        p[i] = vis ? s : -FLT_MAX;
        tile_max = fmaxf(tile_max, p[i]);
      }
    }
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, WAVE_SIZE));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, WAVE_SIZE));
    const float m_new = fmaxf(m_run, tile_max);
    float alpha = 1.f, psum = 0.f;
    if (m_new > -FLT_MAX) {
      alpha = __expf(m_run - m_new);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        p[i] = (p[i] > -FLT_MAX) ? __expf(p[i] - m_new) : 0.f;
        psum += p[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) p[i] = 0.f;
    }
    psum += __shfl_xor(psum, 16, WAVE_SIZE);
    psum += __shfl_xor(psum, 32, WAVE_SIZE);
    l_run = l_run * alpha + psum;
    m_run = m_new;
    float row_alpha[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) row_alpha[r] = __shfl(alpha, 4 * la + r, WAVE_SIZE);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) oacc[c][r] *= row_alpha[r];
    // LDS runs in order within a wave: these stores land after the
    // previous tile's reads
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = lane + WAVE_SIZE * j;
      const int key = i / (V / 8);
      const int col8 = (i % (V / 8)) * 8;
      *reinterpret_cast<ushort8*>(
          &vt_lds[((col8 >> 4) * 8 + (key >> 2)) * 96 + (key & 3) * 16 +
                  (col8 & 15)]) = vv[j];
    }
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      ushort4v pk;
#pragma unroll
      for (int r = 0; r < 4; ++r) pk[r] = float_to_bf16_bits(p[sub * 4 + r]);
      *reinterpret_cast<ushort4v*>(&p_lds[lq * MK_PPAD + sub * 16 + 4 * la]) = pk;
    }
    // producer -> consumer between lanes of this wave: the LDS counter only
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    ushort8 pa = *reinterpret_cast<const ushort8*>(&p_lds[lq * MK_PPAD + 8 * la]);
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
      mk_bf16x4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
          (__attribute__((address_space(3))) mk_bf16x4*)(
              reinterpret_cast<char*>(&vt_lds[(c * 8 + 2 * la) * 96]) + lq * 8));
      mk_bf16x4 v2 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
          (__attribute__((address_space(3))) mk_bf16x4*)(
              reinterpret_cast<char*>(&vt_lds[(c * 8 + 2 * la + 1) * 96]) + lq * 8));
      mk_bf16x8 vb;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        vb[e] = v1[e];
        vb[e + 4] = v2[e];
      }
      oacc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
          *reinterpret_cast<mk_bf16x8*>(&pa), vb, oacc[c], 0, 0, 0);
    }
    if (it + 4 < n_iter) {
#pragma unroll
      for (int sub = 0; sub < 2; ++sub)
#pragma unroll
        for (int st = 0; st < STEPS; ++st) kreg[sub][st] = knext[sub][st];
#pragma unroll
      for (int j = 0; j < NV; ++j) vv[j] = vnext[j];
    }
  }

  __syncthreads();  // every wave is done with its tiles before the union flips
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c)
#pragma unroll
    for (int r = 0; r < 4; ++r)
      merge_lds[(4 * la + r) * (V + 2) + c * 16 + lq] = oacc[c][r];
  if (la == 0) {
    merge_lds[lq * (V + 2) + V] = m_run;
    merge_lds[lq * (V + 2) + V + 1] = l_run;
  }
  __syncthreads();
  // 256 threads = 16 heads x 16 slices of the value dims
  const int g = tid / 16, lane16 = tid % 16;
  if (g >= GQ) return;
  float mf = -FLT_MAX, lf = 0.f, af[E];
#pragma unroll
  for (int e = 0; e < E; ++e) af[e] = 0.f;
  for (int w = 0; w < 4; ++w) {
    const float* wl = reinterpret_cast<const float*>(smem[w]);
    const float mw = wl[g * (V + 2) + V];
    const float lw = wl[g * (V + 2) + V + 1];
    const float mn = fmaxf(mf, mw);
    const float a1 = __expf(mf - mn), a2 = __expf(mw - mn);
    lf = lf * a1 + lw * a2;
#pragma unroll
    for (int e = 0; e < E; ++e)
      af[e] = af[e] * a1 + wl[g * (V + 2) + lane16 * E + e] * a2;
    mf = mn;
  }
  const float inv = lf > 0.f ? a.out_scale / lf : 0.f;
  bf16* op = out + (int64_t)t * ldo + (int64_t)(kvh * GQ + g) * V + lane16 * E;
#pragma unroll
  for (int e = 0; e < E; ++e) op[e] = float_to_bf16_bits(af[e] * inv);
}

template <int D, int V, bool SINGLE, bool SHR, int VS>
int launch_masked_tile(dim3 grid, hipStream_t stream, bf16* out, int64_t ldo,
                       const bf16* q, const bf16* k_cache, int64_t ldk,
                       const bf16* v_cache, int64_t ldv, const int* bt,
                       const int* kv_lens, const int* cu, const int* token_seq,
                       const float* sink_w, int num_seqs, MaskArgs a, int G,
                       int H, int hpt_shift, int max_blocks, float* ws) {
  constexpr int BYTES = MaskedTileLds<D, V / VS>::BYTES;
  grid.x *= VS;
  static bool raised = false;
  if (BYTES > 48 * 1024 && !raised) {
    if (hipFuncSetAttribute(
            reinterpret_cast<const void*>(
                &attn_masked_tile_kernel<D, V, SINGLE, SHR, VS>),
            hipFuncAttributeMaxDynamicSharedMemorySize, BYTES) != hipSuccess)
      return 1;
    raised = true;
  }
  hipLaunchKernelGGL((attn_masked_tile_kernel<D, V, SINGLE, SHR, VS>), grid,
                     dim3(256),
                     BYTES, stream, out, ldo, q, k_cache, ldk, v_cache, ldv, bt,
                     kv_lens, cu, token_seq, sink_w, num_seqs, a, G, H,
                     hpt_shift, max_blocks, ws);
  if (grid.z > 1)
    hipLaunchKernelGGL(attn_masked_combine_kernel, dim3(grid.y, H), dim3(64),
                       0, stream, out, ldo, ws, H, V, (int)grid.z,
                       a.out_scale);
  return 0;
}

// heads per tile: the largest power of two, at most 64, that divides the
// group of query heads on one key/value head
static int masked_hpt_shift(int GQ) {
  int shift = 0;
  while (shift < 6 && GQ % (2 << shift) == 0) ++shift;
  return shift;
}

}  // namespace arks

using namespace arks;

// Steps of single rows through the tile kernel (groups above 16 heads):
// into how many workgroups a row's key tiles are split so that the launch
// fills the chip (1: no split, no workspace).
extern "C" int arks_seq_attn_masked_ksplit(int T, int H, int G,
                                           int max_blocks) {
  const int GQ = H / G;
  if (GQ <= 16) return 1;
  const int base = G * (GQ >> masked_hpt_shift(GQ)) * T;
  const int tiles = (max_blocks * MK_PAGE + MK_KTILE - 1) / MK_KTILE;
  int ks = (512 + base - 1) / base;
  if (ks > 16) ks = 16;
  if (ks > tiles / 2) ks = tiles / 2;
  return ks < 1 ? 1 : ks;
}

// Returns 1 when no kernel is built for these sizes (the caller then runs
// the general kernel).
extern "C" int arks_seq_attn_masked_mfma(
    void* out, int64_t ldo, const void* q, const void* k_cache, int64_t ldk,
    const void* v_cache, int64_t ldv, const void* block_tables,
    const void* seq_lens, const void* cu, const void* token_seq, float scale,
    const void* sink_w, float softcap, int window, int keep_first,
    float out_scale, int T, int H, int G, int D, int V, int bs, int max_blocks,
    int num_seqs, int single_rows, void* ws, int ksplit, int maps,
    hipStream_t stream) {
  // G: key groups, maps of them per key/value head of the cache
  if (maps < 1 || G % maps || (maps > 1 && v_cache == k_cache)) return 1;
  if (bs != MK_PAGE || H % G || ldk % 8 || ldv % 8 || ldo % 8 ||
      ((uintptr_t)q & 15) || ((uintptr_t)k_cache & 15) ||
      ((uintptr_t)v_cache & 15) || ((uintptr_t)out & 15))
    return 1;
  if (T == 0) return 0;
  const int GQ = H / G;
  MaskArgs a;
  a.scale = scale;
  a.softcap = softcap;
  a.out_scale = out_scale;
  a.window = window > 0 ? window : (1 << 30);
  a.keep_first = window > 0 ? keep_first : 0;
  a.maps = maps;
  const bool shared_rows = v_cache == k_cache && ldv == ldk;
  const int hpt_shift = masked_hpt_shift(GQ);
  const int ppt = MK_QTILE >> hpt_shift;
  const dim3 grid_tile(G * (GQ >> hpt_shift),
                       single_rows ? T : (T + ppt - 1) / ppt + num_seqs,
                       single_rows && ws && ksplit > 1 ? ksplit : 1);
#define MK_ARGS                                                               \
  (bf16*)out, ldo, (const bf16*)q, (const bf16*)k_cache, ldk,                 \
      (const bf16*)v_cache, ldv, (const int*)block_tables,                    \
      (const int*)seq_lens, (const int*)cu, (const int*)token_seq,            \
      (const float*)sink_w
#define MK_TILE(DD, VV, SHR, VS)                                              \
  if (D == DD && V == VV && shared_rows == SHR) {                             \
    if (single_rows)                                                          \
      return launch_masked_tile<DD, VV, true, SHR, VS>(                       \
          grid_tile, stream, MK_ARGS, num_seqs, a, G, H, hpt_shift,           \
          max_blocks, (float*)ws);                                            \
    return launch_masked_tile<DD, VV, false, SHR, VS>(                        \
        grid_tile, stream, MK_ARGS, num_seqs, a, G, H, hpt_shift, max_blocks, \
        nullptr);                                                             \
  }
#define MK_DEC(DD, VV)                                                        \
  if (D == DD && V == VV && single_rows && GQ <= 16) {                        \
    hipLaunchKernelGGL((attn_masked_dec_kernel<DD, VV>), dim3(G, T),          \
                       dim3(256), 0, stream, MK_ARGS, a, G, H, max_blocks);   \
    return 0;                                                                 \
  }
  MK_DEC(64, 64)
  MK_DEC(128, 128)
  MK_DEC(128, 64)
  MK_DEC(96, 96)
  MK_DEC(96, 64)
  MK_TILE(64, 64, false, 1)
  MK_TILE(128, 128, false, 1)
  MK_TILE(128, 64, false, 1)
  MK_TILE(96, 96, false, 1)
  MK_TILE(96, 64, false, 1)
  MK_TILE(64, 32, false, 1)
  MK_TILE(192, 128, false, 1)
  MK_TILE(96, 64, true, 1)
  MK_TILE(320, 256, true, 2)
  MK_TILE(576, 512, true, 4)
#undef MK_TILE
#undef MK_DEC
#undef MK_ARGS
  return 1;
}
