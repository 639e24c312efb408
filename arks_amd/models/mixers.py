"""Sequence mixers for layer-list decoders, each with its constants as
constructor parameters so that more than one design can use it:

- SinkRotaryAttention: grouped-query softmax attention over the paged KV
  cache with optional per-head q/k RMS norm, partial rotary (interleaved or
  half-split pairs), a value-less sink key of score 0 in every softmax, and
  values that are stored turned by their own position and turned back at
  the query's position after the weighted sum.
- LightningMixer: linear attention with one scalar decay per head and a
  [dim x vdim] fp32 state per head and sequence, gated RMS-normed output.
- Mamba1Mixer: short causal depthwise convolution + selective scan with an
  [inner x state] fp32 state per sequence.
- WindowPoolAttention: grouped-query softmax attention without positions in
  the scores, over a sliding window of recent keys plus one pooled (mean)
  key/value per block of older positions; biases on every projection.
- RetentionMixer: the lightning recurrence on plain rows (nothing
  activated) with partial rotary on q and k, scaled keys, a per-head unit
  RMS of the output and a silu gate.
- ParallelMixer: two of the above fed the same input, as ONE
  in-projection GEMM and ONE out-projection GEMM over the concatenated
  (pre-scaled) head outputs.
- SinkRotaryAttention also takes tanh-capped scores (softcap) and a sliding
  window that keeps the first keys of the sequence visible (window,
  keep_first); without own projections it is a split mixer too.
- LatentAttention: queries and keys/values through low-rank latents; the
  cache holds one normed latent and one rotated key part per token, shared
  by all heads, and the per-head up-projections are applied to the query
  and to the attention result instead of to every cached token; a learned
  per-head sink in the softmax.
- Mamba2Mixer: short causal convolution over [x | B | C], one scalar decay
  per head and token, an [state x vdim] fp32 state per head and sequence,
  silu gate, RMS norm in equal groups of channels.
- SinkRotaryAttention also takes rotary frequencies scaled over a ramp of
  wavelengths (rot_scaling), a unit RMS of q and k AFTER the rotation
  (unit_norm_after) and values that are the keys as projected
  (value_is_key: no value projection).
- DiffAttention: two softmax maps per head over the same values, combined
  as a1 - lambda a2 and brought to unit RMS per head; short causal
  convolutions behind the q, k and v projections (their last inputs are
  per-sequence state), a query factor that grows with the logarithm of the
  position, a sigmoid output gate; optionally on the pages of an earlier
  layer's keys and values.

WindowPoolAttention, RetentionMixer, LatentAttention and Mamba2Mixer are
"split" mixers: they name the rows of their
in-projection (in_spans) and the columns of their out-projection
(out_cols) and do everything between in core(), so that a parent can fuse
the projections of several of them; alone, SplitMixer.forward runs the
same three steps with projections of their own.

Every mixer maps the (already token-shifted) rows [T, width] of one engine
step to [T, width]; rows of several sequences are packed, prompt portions
beside single decoded tokens, and ForwardBatch says where each sequence's
rows, pages and state slot are. Projections run as library GEMMs in the
model's dtype; everything that enters a softmax, a norm or a recurrence is
fp32 inside the kernels (arks_amd/ops/csrc/seq_*.hip).

Per-layer cache: each mixer names the tensors it needs in cache_layout():
"paged" ones get a leading [num_blocks] axis and are addressed through the
block tables, "slot" ones a leading [num_slots] axis addressed by
ForwardBatch.state_slots.
"""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..engine.forward_batch import ForwardBatch


def linear(x: torch.Tensor, w: torch.Tensor, b=None) -> torch.Tensor:
    """x @ w^T (+ b) as a library GEMM (the decode-shaped bf16 cases go to
    the split-K kernel when the main extension is built)."""
    if x.dtype == torch.bfloat16:
        return ops.linear_bf16(x, w, b)
    return F.linear(x, w, b)


_MM_OUT_DTYPE = {}  # device type -> torch.mm(..., out_dtype=) available


def linear_f32(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x @ w^T with fp32 OUTPUT from rows of the model's dtype (bf16 inputs,
    fp32 accumulate, no rounding of the result)."""
    if x.dtype == torch.float32:
        return F.linear(x, w)
    if _MM_OUT_DTYPE.get(x.device.type, True):
        try:
            return torch.mm(x, w.t(), out_dtype=torch.float32)
        except (TypeError, RuntimeError):
            _MM_OUT_DTYPE[x.device.type] = False
    return F.linear(x, w).float()


def step_chunks(batch: ForwardBatch, device, chunk: int = 0):
    """Chunk metadata of this step for the chunk-parallel recurrent prefill
    (None for steps whose rows per sequence all fit one chunk, and inside
    captured decode graphs). chunk: rows per chunk (default ops.SCAN_CHUNK)."""
    chunk = chunk or ops.SCAN_CHUNK
    if (device.type != "cuda" or batch.seq_lens_list is None
            or batch.max_q_len <= chunk):
        return None
    key = ("scan_chunks", chunk)
    if key not in batch.tile_cache:
        batch.tile_cache[key] = ops.scan_chunks(
            batch.seq_lens_list, device, chunk)
    return batch.tile_cache[key]


def _param(*shape, dtype):
    return nn.Parameter(torch.zeros(shape, dtype=dtype), requires_grad=False)


def rotary_inv_freq(base: float, ndims: int) -> torch.Tensor:
    """f_i = base^(-2i/ndims), i < ndims/2, rounded once from float64."""
    i = torch.arange(ndims // 2, dtype=torch.float64)
    return torch.pow(torch.tensor(float(base), dtype=torch.float64),
                     -2.0 * i / ndims).float()


def ramp_scaled_inv_freq(base: float, ndims: int, scaling: dict | None):
    """(frequencies, factor on cos and sin). scaling {factor, original, fast,
    slow}: pair i completes original * f_i / 2 pi turns over the original
    length; with n(t) = ndims ln(original / (2 pi t)) / (2 ln base) the pair
    index that completes t turns, pairs below lo = floor(n(fast)) keep f_i,
    pairs above hi = ceil(n(slow)) get f_i / factor, and those between are
    blended linearly; cos and sin are multiplied by 0.1 ln(factor) + 1.
    Everything in float64, rounded once."""
    import math

    i = torch.arange(ndims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64),
                  -2.0 * i / ndims)
    if not scaling:
        return f.float(), 1.0
    factor = float(scaling["factor"])

    def pair_of(turns):
        return (ndims * math.log(float(scaling["original"])
                                 / (2.0 * math.pi * float(turns)))
                / (2.0 * math.log(float(base))))

    lo = max(math.floor(pair_of(scaling["fast"])), 0)
    hi = min(math.ceil(pair_of(scaling["slow"])), ndims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    f = f / factor * ramp + f * (1.0 - ramp)
    return f.float(), 0.1 * math.log(factor) + 1.0


_DECODE_TILES: dict = {}


class SinkRotaryAttention(nn.Module):
    def __init__(self, width: int, heads: int, kv_heads: int, dim: int,
                 vdim: int, scale: float, rot_base: float, rot_dims: int,
                 eps: float, dtype, qk_norm: bool = True, sink: bool = True,
                 rotate_values: bool = True, interleaved: bool = True,
                 softcap: float = 0.0, window: int = 0, keep_first: int = 0,
                 own_projections: bool = True, rot_scaling: dict | None = None,
                 unit_norm_after: bool = False, value_is_key: bool = False):
        super().__init__()
        assert heads % kv_heads == 0 and rot_dims % 2 == 0 and rot_dims <= dim
        assert not rotate_values or vdim % 2 == 0
        assert not value_is_key or (vdim == dim and not rotate_values)
        self.unit_norm_after, self.value_is_key = unit_norm_after, value_is_key
        self.H, self.G, self.D, self.V = heads, kv_heads, dim, vdim
        self.scale, self.eps = float(scale), eps
        self.sink, self.interleaved = sink, interleaved
        # scores c tanh(s / c); row i sees key j <= i iff i - j < window or
        # j < keep_first (0: plain causal)
        self.softcap, self.window = float(softcap), int(window)
        self.keep_first = int(keep_first)
        self.masked = self.softcap > 0 or self.window > 0
        assert not (self.masked and rotate_values)
        self.out_cols = heads * vdim
        if own_projections:
            self.qkv = _param(
                heads * dim + kv_heads * (dim + (0 if value_is_key else vdim)),
                width, dtype=dtype)
            self.o = _param(width, heads * vdim, dtype=dtype)
        self.q_norm = _param(dim, dtype=torch.float32) if qk_norm else None
        self.k_norm = _param(dim, dtype=torch.float32) if qk_norm else None
        freqs, self.rot_mag = ramp_scaled_inv_freq(rot_base, rot_dims,
                                                   rot_scaling)
        self.register_buffer("inv_freq_qk", freqs, persistent=False)
        self.register_buffer(
            "inv_freq_v",
            rotary_inv_freq(rot_base, vdim) if rotate_values else None,
            persistent=False)

    def in_spans(self) -> list:
        spans = [("q", self.H * self.D, False), ("k", self.G * self.D, False)]
        if not self.value_is_key:
            spans.append(("v", self.G * self.V, False))
        return spans

    def extra_weights(self) -> dict:
        if self.q_norm is None:
            return {}
        return {"q.norm": (self.q_norm, 0), "k.norm": (self.k_norm, 0)}

    def weight_map(self) -> dict:
        H, G, D, V = self.H, self.G, self.D, self.V
        m = {"q": (self.qkv, 0), "k": (self.qkv, H * D), "o": (self.o, 0)}
        if not self.value_is_key:
            m["v"] = (self.qkv, H * D + G * D)
        m.update(self.extra_weights())
        return m

    def _split(self, p):
        """q, k, v views of the in-projection's rows; the value is the key
        as projected where the design has no value projection."""
        H, G, D, V = self.H, self.G, self.D, self.V
        q = p[:, :H * D].unflatten(-1, (H, D))
        k = p[:, H * D:(H + G) * D].unflatten(-1, (G, D))
        if self.value_is_key:
            return q, k, k
        return q, k, p[:, (H + G) * D:(H + G) * D + G * V].unflatten(-1, (G, V))

    def _prepare(self, q, k, v, batch: ForwardBatch, cache: dict):
        return ops.qk_norm_rope_cache(
            q, k, v, self.q_norm, self.k_norm, self.eps, batch.positions,
            self.inv_freq_qk, self.inv_freq_v, cache["k"], cache["v"],
            batch.slot_mapping, self.interleaved, self.rot_mag,
            self.unit_norm_after)

    def cache_layout(self, block_size: int, dtype) -> dict:
        return {"k": ("paged", (self.G, block_size, self.D), dtype),
                "v": ("paged", (self.G, block_size, self.V), dtype)}

    def _tiles(self, batch: ForwardBatch, q):
        """Work lists of the MFMA kernels: host-built once per step and head
        layout (batch.tile_cache), shared by every layer of that layout.
        None where the general kernel runs (CPU, float32, other sizes).
        A captured decode graph has no host lengths, but its work list is
        static — one 64-row tile per sequence — and is kept for the life of
        the process, since the graph holds its address."""
        if not q.is_cuda or q.dtype != torch.bfloat16 or self.D != self.V:
            return None
        if batch.kv_lens_list is None:
            if batch.max_q_len != 1:
                return None
            B = batch.seq_lens.shape[0]
            key = (B, self.H, self.G, self.D, q.device.index)
            if key not in _DECODE_TILES:
                _DECODE_TILES[key] = ops.sink_attention_tiles(
                    [1] * B, [1] * B, self.H, self.G, self.D, q.device)
            return _DECODE_TILES[key]
        key = (self.H, self.G, self.D)
        if key not in batch.tile_cache:
            batch.tile_cache[key] = ops.sink_attention_tiles(
                batch.seq_lens_list, batch.kv_lens_list, self.H, self.G,
                self.D, q.device)
        return batch.tile_cache[key]

    def core(self, p, batch: ForwardBatch, cache: dict, out, out_scale) -> None:
        """p: rows of the in-projection [q | k | v]; writes the head outputs,
        times out_scale, into out [T, H * V] (rows may be strided)."""
        H, G, D, V = self.H, self.G, self.D, self.V
        q, k, v = self._split(p)
        q = self._prepare(q, k, v, batch, cache)
        if self.masked:
            ops.attention_sink_paged(
                q, cache["k"], cache["v"], batch.block_tables, batch.seq_lens,
                batch.cu_seqlens, batch.token_seq, self.scale, self.sink,
                None, self.interleaved, batch.max_q_len, batch.positions,
                softcap=self.softcap, window=self.window,
                keep_first=self.keep_first, out=out.unflatten(-1, (H, V)),
                out_scale=out_scale)
            return
        res = ops.attention_sink_paged(
            q, cache["k"], cache["v"], batch.block_tables, batch.seq_lens,
            batch.cu_seqlens, batch.token_seq, self.scale, self.sink,
            self.inv_freq_v, self.interleaved, batch.max_q_len,
            batch.positions, self._tiles(batch, q))
        if out_scale != 1.0:
            res = res * out_scale
        out.copy_(res.view(p.shape[0], H * V))

    def forward(self, xs, batch: ForwardBatch, cache: dict) -> torch.Tensor:
        T = xs.shape[0]
        H, G, D, V = self.H, self.G, self.D, self.V
        qkv = linear(xs, self.qkv)
        if self.masked:
            out = torch.empty((T, H * V), dtype=xs.dtype, device=xs.device)
            self.core(qkv, batch, cache, out, 1.0)
            return linear(out, self.o)
        q, k, v = self._split(qkv)
        q = self._prepare(q, k, v, batch, cache)
        out = ops.attention_sink_paged(
            q, cache["k"], cache["v"], batch.block_tables, batch.seq_lens,
            batch.cu_seqlens, batch.token_seq, self.scale, self.sink,
            self.inv_freq_v, self.interleaved, batch.max_q_len,
            batch.positions, self._tiles(batch, q))
        return linear(out.view(T, H * V), self.o)


class LightningMixer(nn.Module):
    def __init__(self, width: int, heads: int, dim: int, vdim: int,
                 decay, eps: float, dtype):
        super().__init__()
        assert len(decay) == heads
        self.H, self.D, self.V, self.eps = heads, dim, vdim, eps
        self.qkvg = _param(2 * heads * dim + 2 * heads * vdim, width, dtype=dtype)
        self.o = _param(width, heads * vdim, dtype=dtype)
        self.norm = _param(heads * vdim, dtype=torch.float32)
        self.register_buffer("decay", torch.tensor(
            [float(d) for d in decay], dtype=torch.float64).float(),
            persistent=False)

    def weight_map(self) -> dict:
        HD, HV = self.H * self.D, self.H * self.V
        return {"q": (self.qkvg, 0), "k": (self.qkvg, HD),
                "v": (self.qkvg, 2 * HD), "g": (self.qkvg, 2 * HD + HV),
                "o": (self.o, 0), "norm": (self.norm, 0)}

    def cache_layout(self, block_size: int, dtype) -> dict:
        return {"S": ("slot", (self.H, self.D, self.V), torch.float32)}

    def forward(self, xs, batch: ForwardBatch, cache: dict) -> torch.Tensor:
        T = xs.shape[0]
        H, D, V = self.H, self.D, self.V
        p = linear(xs, self.qkvg)
        q = p[:, :H * D].unflatten(-1, (H, D))
        k = p[:, H * D:2 * H * D].unflatten(-1, (H, D))
        v = p[:, 2 * H * D:2 * H * D + H * V].unflatten(-1, (H, V))
        g = p[:, 2 * H * D + H * V:]
        o = ops.lightning_scan(q, k, v, self.decay, cache["S"],
                               batch.cu_seqlens, batch.seq_lens,
                               batch.state_slots, batch.max_q_len,
                               step_chunks(batch, xs.device))
        y = ops.gated_rmsnorm(o.view(T, H * V), self.norm, g, self.eps, xs.dtype)
        return linear(y, self.o)


class Mamba1Mixer(nn.Module):
    def __init__(self, width: int, inner: int, state: int, dt_rank: int,
                 conv: int, dtype):
        super().__init__()
        self.C, self.N, self.R, self.taps = inner, state, dt_rank, conv
        self.w_in = _param(2 * inner, width, dtype=dtype)
        self.w_x = _param(dt_rank + 2 * state, inner, dtype=dtype)
        self.o = _param(width, inner, dtype=dtype)
        f32 = torch.float32
        self.conv_w = _param(inner, conv, dtype=f32)
        self.conv_b = _param(inner, dtype=f32)
        self.dt_w = _param(inner, dt_rank, dtype=f32)
        self.dt_b = _param(inner, dtype=f32)
        self.A_log = _param(inner, state, dtype=f32)
        self.D = _param(inner, dtype=f32)
        self.register_buffer("A", torch.zeros(inner, state, dtype=f32),
                             persistent=False)
        # dt's projection as a GEMM operand (the kernels can also project
        # in place from the fp32 dt_w: tiny ranks, CPU reference)
        self.register_buffer("dt_w_mm", torch.zeros(inner, dt_rank, dtype=dtype),
                             persistent=False)
        self.register_buffer("conv_w_t", torch.zeros(conv, inner, dtype=f32),
                             persistent=False)

    def weight_map(self) -> dict:
        return {"in": (self.w_in, 0), "x": (self.w_x, 0), "o": (self.o, 0),
                "conv": (self.conv_w, 0), "conv.b": (self.conv_b, 0),
                "dt": (self.dt_w, 0), "dt.b": (self.dt_b, 0),
                "A_log": (self.A_log, 0), "D": (self.D, 0)}

    def finish_loading(self) -> None:
        self.A.copy_(-torch.exp(self.A_log.data.float()))
        self.dt_w_mm.copy_(self.dt_w.data)
        self.conv_w_t.copy_(self.conv_w.data.t())

    def cache_layout(self, block_size: int, dtype) -> dict:
        out = {"ssm": ("slot", (self.C, self.N), torch.float32)}
        if self.taps > 1:
            out["conv"] = ("slot", (self.taps - 1, self.C), torch.float32)
        return out

    def forward(self, xs, batch: ForwardBatch, cache: dict) -> torch.Tensor:
        C = self.C
        xz = linear(xs, self.w_in)
        u = ops.causal_conv_silu(
            xz[:, :C], self.conv_w, self.conv_b, cache.get("conv"),
            batch.cu_seqlens, batch.seq_lens, batch.state_slots,
            batch.token_seq, self.conv_w_t)
        dbc = linear(u, self.w_x)
        dt_pre = None
        if xs.is_cuda and self.R >= 8:
            dt_pre = linear_f32(dbc[:, :self.R], self.dt_w_mm)
        y = ops.selective_scan(
            u, dbc, xz[:, C:], self.dt_w, self.dt_b, self.A, self.D,
            cache["ssm"], batch.cu_seqlens, batch.seq_lens, batch.state_slots,
            batch.max_q_len, dt_pre, step_chunks(batch, xs.device))
        return linear(y, self.o)


class SplitMixer(nn.Module):
    """A mixer in three parts: rows of an in-projection (in_spans: name,
    rows, has_bias), core() from those rows to the columns of an
    out-projection (out_cols, out_bias). With own_projections the module
    holds both projections itself; without, a parent (ParallelMixer) holds
    fused ones and calls core() on its slice."""

    out_has_bias = False

    def in_spans(self) -> list:
        raise NotImplementedError

    def _make_projections(self, width: int, dtype) -> None:
        spans = self.in_spans()
        rows = sum(n for _, n, _ in spans)
        self.w_in = _param(rows, width, dtype=dtype)
        self.b_in = (_param(rows, dtype=dtype)
                     if any(b for _, _, b in spans) else None)
        self.w_out = _param(width, self.out_cols, dtype=dtype)
        self.b_out = _param(width, dtype=dtype) if self.out_has_bias else None

    def weight_map(self) -> dict:
        m, row = {}, 0
        for name, n, has_b in self.in_spans():
            m[name] = (self.w_in, row)
            if has_b:
                m[name + ".b"] = (self.b_in, row)
            row += n
        m["o"] = (self.w_out, 0)
        if self.b_out is not None:
            m["o.b"] = (self.b_out, 0)
        m.update(self.extra_weights())
        return m

    def extra_weights(self) -> dict:
        """Tensors besides the projections the parent may fuse."""
        return {}

    def forward(self, xs, batch: ForwardBatch, cache: dict) -> torch.Tensor:
        p = linear(xs, self.w_in, self.b_in)
        out = torch.empty((xs.shape[0], self.out_cols), dtype=xs.dtype,
                          device=xs.device)
        self.core(p, batch, cache, out, 1.0)
        return linear(out, self.w_out, self.b_out)


class WindowPoolAttention(SplitMixer):
    """Softmax attention, query head h on key/value head h // (H/G), no
    positions in the scores: the row at position i sees keys j with
    0 <= i - j < window and one pooled key/value (the mean over the block,
    taken from what the pages hold) for every block of `pool` positions
    that ends at or before i - window. Paged k/v plus paged pooled kp/vp
    (ops.kv_write_pooled)."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int,
                 vdim: int, scale: float, window: int, pool: int, dtype,
                 bias: bool = True, own_projections: bool = True):
        super().__init__()
        assert heads % kv_heads == 0 and window >= 1 and pool >= 1
        self.H, self.G, self.D, self.V = heads, kv_heads, dim, vdim
        self.scale, self.window, self.pool = float(scale), int(window), int(pool)
        self.bias = self.out_has_bias = bias
        self.out_cols = heads * vdim
        if own_projections:
            self._make_projections(width, dtype)

    def in_spans(self) -> list:
        return [("q", self.H * self.D, self.bias),
                ("k", self.G * self.D, self.bias),
                ("v", self.G * self.V, self.bias)]

    def cache_layout(self, block_size: int, dtype) -> dict:
        spp = ops.pool_slots_per_page(block_size, self.pool)
        return {"k": ("paged", (self.G, block_size, self.D), dtype),
                "v": ("paged", (self.G, block_size, self.V), dtype),
                "kp": ("paged", (self.G, spp, self.D), dtype),
                "vp": ("paged", (self.G, spp, self.V), dtype)}

    def core(self, p, batch: ForwardBatch, cache: dict, out, out_scale) -> None:
        H, G, D, V = self.H, self.G, self.D, self.V
        q = p[:, :H * D].unflatten(-1, (H, D))
        k = p[:, H * D:(H + G) * D].unflatten(-1, (G, D))
        v = p[:, (H + G) * D:(H + G) * D + G * V].unflatten(-1, (G, V))
        ops.kv_write_pooled(k, v, cache["k"], cache["v"], cache["kp"],
                            cache["vp"], batch.slot_mapping, batch.positions,
                            batch.block_tables, batch.token_seq, self.pool)
        ops.attention_window_pool(
            q, cache["k"], cache["v"], cache["kp"], cache["vp"],
            batch.block_tables, batch.seq_lens, batch.cu_seqlens,
            batch.token_seq, self.scale, self.window, self.pool,
            out.unflatten(-1, (H, V)), out_scale, batch.max_q_len)


class RetentionMixer(SplitMixer):
    """S <- decay_h S + k v^T, o = S^T q per head on plain projections: q
    and k turned by their position over their first rot_dims dims
    (half-split pairs unless interleaved), k times k_scale after that; each
    head's o scaled to unit RMS, times silu(gate). fp32 state
    [H, D, V] per sequence; runs the lightning kernels."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay,
                 rot_base: float, rot_dims: int, eps: float, dtype,
                 k_scale: float | None = None, interleaved: bool = False,
                 own_projections: bool = True):
        super().__init__()
        assert len(decay) == heads and rot_dims % 2 == 0 and rot_dims <= dim
        self.H, self.D, self.V, self.eps = heads, dim, vdim, eps
        self.k_scale = float(dim ** -0.5 if k_scale is None else k_scale)
        self.interleaved = interleaved
        self.out_cols = heads * vdim
        self.register_buffer("decay", torch.tensor(
            [float(d) for d in decay], dtype=torch.float64).float(),
            persistent=False)
        self.register_buffer(
            "inv_freq", rotary_inv_freq(rot_base, rot_dims) if rot_dims else None,
            persistent=False)
        if own_projections:
            self._make_projections(width, dtype)

    def in_spans(self) -> list:
        HD, HV = self.H * self.D, self.H * self.V
        return [("q", HD, False), ("k", HD, False), ("v", HV, False),
                ("g", HV, False)]

    def cache_layout(self, block_size: int, dtype) -> dict:
        return {"S": ("slot", (self.H, self.D, self.V), torch.float32)}

    def core(self, p, batch: ForwardBatch, cache: dict, out, out_scale) -> None:
        T = p.shape[0]
        H, D, V = self.H, self.D, self.V
        q = p[:, :H * D].unflatten(-1, (H, D))
        k = p[:, H * D:2 * H * D].unflatten(-1, (H, D))
        v = p[:, 2 * H * D:2 * H * D + H * V].unflatten(-1, (H, V))
        g = p[:, 2 * H * D + H * V:2 * H * D + 2 * H * V]
        o = ops.retention_scan(
            q, k, v, self.decay, cache["S"], batch.cu_seqlens, batch.seq_lens,
            batch.state_slots, batch.positions, self.inv_freq,
            self.interleaved, self.k_scale, batch.max_q_len,
            step_chunks(batch, p.device))
        ops.head_norm_gate(o.view(T, H * V), g, self.eps, H, out, out_scale)


class LatentAttention(SplitMixer):
    """Attention through low-rank latents. Per row: c_q = rmsnorm(W_dq h),
    q = W_uq c_q, laid out per head as [dim plain | rot_dim rotated];
    W_dkv h = [kv_rank | rot_dim]: the first part RMS-normed is the latent c,
    the second, rotated (interleaved pairs), is one key part shared by all
    heads. Keys are [W_uk c | shared part], values W_uv c, causal softmax
    with a learned per-head sink in the denominator.

    Only [c | rotated part] is cached, one row per token ("ckv", one
    key/value head). The up-projections move to the other side of the
    products: q_h' = W_uk,h^T q_h,plain (length kv_rank), so the score is
    q_h' . c + q_h,rot . k_rot and the softmax-weighted sum of latents is
    multiplied by W_uv,h afterwards. The attention kernels therefore see H
    query heads of size kv_rank + rot_dim on ONE key/value head whose value
    is the first kv_rank columns of its key row.

    That form costs kv_rank + rot_dim + kv_rank multiply-adds per (row,
    head, key), against dim + rot_dim + vdim for per-head keys and values,
    and pays for a step of few rows over a long context. A step with a long
    portion (EXPAND_ROWS rows or more of one sequence) therefore takes the
    other form: the latents of every sequence's context are gathered from
    the pages and up-projected once into per-head keys and values for the
    step (temporary pages of the usual layout with a block table of their
    own), and the same attention kernels run on H key/value heads."""

    EXPAND_ROWS = 192

    def __init__(self, width: int, heads: int, dim: int, rot_dim: int,
                 vdim: int, kv_rank: int, q_rank: int, scale: float,
                 rot_base: float, eps: float, dtype,
                 own_projections: bool = True):
        super().__init__()
        assert rot_dim % 2 == 0
        self.H, self.D, self.R, self.V = heads, dim, rot_dim, vdim
        self.rank, self.q_rank = kv_rank, q_rank
        self.scale, self.eps = float(scale), eps
        self.out_cols = heads * vdim
        f32 = torch.float32
        self.dq_norm = _param(q_rank, dtype=f32)
        self.dkv_norm = _param(kv_rank, dtype=f32)
        self.uq = _param(heads * (dim + rot_dim), q_rank, dtype=dtype)
        # per head [dim, kv_rank] and [vdim, kv_rank], heads stacked by rows
        self.uk = _param(heads * dim, kv_rank, dtype=dtype)
        self.uv = _param(heads * vdim, kv_rank, dtype=dtype)
        self.sink = _param(heads, dtype=f32)
        self.register_buffer("inv_freq", rotary_inv_freq(rot_base, rot_dim),
                             persistent=False)
        if own_projections:
            self._make_projections(width, dtype)

    def in_spans(self) -> list:
        return [("dq", self.q_rank, False), ("dkv", self.rank + self.R, False)]

    def extra_weights(self) -> dict:
        return {"dq.norm": (self.dq_norm, 0), "dkv.norm": (self.dkv_norm, 0),
                "uq": (self.uq, 0), "sink": (self.sink, 0),
                "uk": (self.uk, 0), "uv": (self.uv, 0)}

    def cache_layout(self, block_size: int, dtype) -> dict:
        return {"ckv": ("paged", (1, block_size, self.rank + self.R), dtype)}

    def core(self, p, batch: ForwardBatch, cache: dict, out, out_scale) -> None:
        T = p.shape[0]
        H, D, R, V, rank = self.H, self.D, self.R, self.V, self.rank
        ckv = cache["ckv"]
        cq = ops.latent_prepare(
            p[:, :self.q_rank], p[:, self.q_rank:self.q_rank + rank + R],
            self.dq_norm, self.dkv_norm, self.eps, batch.positions,
            self.inv_freq, ckv, batch.slot_mapping)
        q = linear(cq, self.uq).view(T, H, D + R)
        if (batch.max_q_len >= self.EXPAND_ROWS
                and batch.kv_lens_list is not None):
            self._expanded(q, batch, ckv, out, out_scale)
            return
        # [H, T, D] x [H, D, rank]: the key up-projection applied to q
        q_abs = torch.bmm(q[..., :D].transpose(0, 1),
                          self.uk.view(H, D, rank))
        qf = torch.empty((T, H, rank + R), dtype=p.dtype, device=p.device)
        ops.latent_query(q, q_abs, batch.positions, self.inv_freq, qf)
        o_lat = ops.attention_sink_paged(
            qf, ckv, ckv[..., :rank], batch.block_tables, batch.seq_lens,
            batch.cu_seqlens, batch.token_seq, self.scale, False, None, True,
            batch.max_q_len, batch.positions, sink_w=self.sink)
        # [H, T, rank] x [H, rank, V]: the value up-projection
        o = torch.bmm(o_lat.transpose(0, 1),
                      self.uv.view(H, V, rank).transpose(1, 2))
        if out_scale != 1.0:
            o = o * out_scale
        out.unflatten(-1, (H, V)).copy_(o.transpose(0, 1))


    def _expanded(self, q, batch: ForwardBatch, ckv, out, out_scale) -> None:
        T = q.shape[0]
        H, D, R, V, rank = self.H, self.D, self.R, self.V, self.rank
        bs = ckv.shape[2]
        nb = [-(-n // bs) for n in batch.kv_lens_list]
        key = ("latent_pages", bs)
        if key not in batch.tile_cache:
            # the context's pages in sequence order, and the block table
            # of the temporary pages (consecutive), once per step
            dev = q.device
            idx = torch.cat([batch.block_tables[s, :n].long()
                             for s, n in enumerate(nb)])
            table = torch.zeros((len(nb), max(nb)), dtype=torch.int32)
            at = 0
            for s, n in enumerate(nb):
                table[s, :n] = torch.arange(at, at + n, dtype=torch.int32)
                at += n
            batch.tile_cache[key] = (idx, table.to(dev))
        idx, table = batch.tile_cache[key]
        NB = idx.shape[0]
        lat = ckv[idx]  # [NB, 1, bs, rank + R]
        c = lat[..., :rank].reshape(NB * bs, rank)
        kt = torch.empty((NB, H, bs, D + R), dtype=q.dtype, device=q.device)
        kt[..., :D] = linear(c, self.uk).view(NB, bs, H, D).transpose(1, 2)
        kt[..., D:] = lat[..., rank:]
        vt = linear(c, self.uv).view(NB, bs, H, V).transpose(1, 2).contiguous()
        qf = torch.empty((T, H, D + R), dtype=q.dtype, device=q.device)
        ops.latent_query(q, None, batch.positions, self.inv_freq, qf)
        ops.attention_sink_paged(
            qf, kt, vt, table, batch.seq_lens, batch.cu_seqlens,
            batch.token_seq, self.scale, False, None, True, batch.max_q_len,
            batch.positions, sink_w=self.sink, out=out.unflatten(-1, (H, V)),
            out_scale=out_scale)


class Mamba2Mixer(SplitMixer):
    """In-projection rows [z: inner | x: inner | B: G*N | C: G*N | dt: P]
    with inner = P * vdim. [x | B | C] pass a causal depthwise convolution
    (taps per channel, bias) and silu; dt = softplus(dt + dt_bias); head h
    (group h // (P / G)) keeps S_h (N x vdim, fp32):
    S_h <- exp(-exp(A_log_h) dt_h) S_h + dt_h B x_h^T,
    y_h = S_h^T C + D_h x_h. Then y * silu(z), unit RMS in norm_groups equal
    parts of the channels, times the norm weight."""

    def __init__(self, width: int, heads: int, vdim: int, state: int,
                 groups: int, norm_groups: int, conv: int, eps: float, dtype,
                 own_projections: bool = True):
        super().__init__()
        inner = heads * vdim
        assert heads % groups == 0 and inner % norm_groups == 0
        self.P, self.V, self.N, self.G = heads, vdim, state, groups
        self.inner, self.norm_groups = inner, norm_groups
        self.taps, self.eps = conv, eps
        self.ch = inner + 2 * groups * state  # convolved channels
        self.out_cols = inner
        f32 = torch.float32
        self.conv_w = _param(self.ch, conv, dtype=f32)
        self.conv_b = _param(self.ch, dtype=f32)
        self.dt_bias = _param(heads, dtype=f32)
        self.A_log = _param(heads, dtype=f32)
        self.D = _param(heads, dtype=f32)
        self.norm = _param(inner, dtype=f32)
        self.register_buffer("rate", torch.zeros(heads, dtype=f32),
                             persistent=False)
        self.register_buffer("conv_w_t", torch.zeros(conv, self.ch, dtype=f32),
                             persistent=False)
        if own_projections:
            self._make_projections(width, dtype)

    def in_spans(self) -> list:
        return [("in", 2 * self.inner + 2 * self.G * self.N + self.P, False)]

    def extra_weights(self) -> dict:
        return {"conv": (self.conv_w, 0), "conv.b": (self.conv_b, 0),
                "dt_bias": (self.dt_bias, 0), "A_log": (self.A_log, 0),
                "D": (self.D, 0), "norm": (self.norm, 0)}

    def finish_loading(self) -> None:
        self.rate.copy_(torch.exp(self.A_log.data.float()))
        self.conv_w_t.copy_(self.conv_w.data.t())

    def cache_layout(self, block_size: int, dtype) -> dict:
        out = {"ssm": ("slot", (self.P, self.N, self.V), torch.float32)}
        if self.taps > 1:
            out["conv"] = ("slot", (self.taps - 1, self.ch), torch.float32)
        return out

    def core(self, p, batch: ForwardBatch, cache: dict, out, out_scale) -> None:
        inner, ch = self.inner, self.ch
        xbc = ops.causal_conv_silu(
            p[:, inner:inner + ch], self.conv_w, self.conv_b, cache.get("conv"),
            batch.cu_seqlens, batch.seq_lens, batch.state_slots,
            batch.token_seq, self.conv_w_t)
        y = ops.mamba2_scan(
            xbc, p[:, inner + ch:inner + ch + self.P], self.dt_bias, self.rate,
            self.D, cache["ssm"], batch.cu_seqlens, batch.seq_lens,
            batch.state_slots, self.P, self.V, self.N, self.G,
            batch.max_q_len, step_chunks(batch, p.device, ops.MAMBA2_CHUNK))
        ops.gate_group_norm(y, p[:, :inner], self.norm, self.norm_groups,
                            self.eps, out, out_scale)


class DiffAttention(SplitMixer):
    """Softmax attention with two maps per head. In-projection rows
    [q: H*2*D | k: G*2*D | v: G*V | g: H*V], a head's q and a key/value
    head's k laid out [map 1 | map 2]. Per row: q, k and v pass a causal
    depthwise convolution over time (taps per channel, no bias, no
    activation; the last taps-1 projected rows of a sequence are slot
    state); q is multiplied by 1 + temp_coef ln(floor((p + 1) / temp_every)
    + 1) at position p; each map is a causal softmax attention of its own,
    scores q_m . k_m * scale, over the shared values; with
    lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff, one number per layer,
    o = a1 - lambda a2 is divided by its root mean square over the head
    (no weight), multiplied by 1 - diff and by sigmoid(g).

    The pages hold a token's convolved keys with both maps side by side,
    [pages, G, bs, 2*D], and its convolved values [pages, G, bs, V]; the
    attention ops read key m of a row for the query heads of map m
    (ops.attention_sink_paged(maps=2)). shared_kv: the layer has neither k
    nor v rows; core() is handed the pages of the layer it borrows from."""

    MAPS = 2

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int,
                 vdim: int, scale: float, diff: float, conv: int,
                 temp_coef: float, temp_every: int, eps: float, dtype,
                 shared_kv: bool = False, own_projections: bool = True):
        super().__init__()
        assert heads % kv_heads == 0 and conv >= 1
        self.H, self.G, self.D, self.V = heads, kv_heads, dim, vdim
        self.scale, self.diff, self.eps = float(scale), float(diff), eps
        self.taps, self.shared_kv = int(conv), shared_kv
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        M = self.MAPS
        self.n_q = heads * M * dim
        self.n_k = 0 if shared_kv else kv_heads * M * dim
        self.n_v = 0 if shared_kv else kv_heads * vdim
        self.ch = self.n_q + self.n_k + self.n_v  # convolved channels
        self.out_cols = heads * vdim
        f32 = torch.float32
        self.conv_w = _param(self.ch, self.taps, dtype=f32)
        for leaf in ("lq1", "lk1", "lq2", "lk2"):
            setattr(self, leaf, _param(dim, dtype=f32))
        self.lam = float(diff)
        self.register_buffer("conv_w_t", torch.zeros(self.taps, self.ch, dtype=f32),
                             persistent=False)
        if own_projections:
            self._make_projections(width, dtype)

    def in_spans(self) -> list:
        spans = [("q", self.n_q, False)]
        if not self.shared_kv:
            spans += [("k", self.n_k, False), ("v", self.n_v, False)]
        return spans + [("g", self.H * self.V, False)]

    def extra_weights(self) -> dict:
        m = {"q.conv": (self.conv_w, 0)}
        if not self.shared_kv:
            m["k.conv"] = (self.conv_w, self.n_q)
            m["v.conv"] = (self.conv_w, self.n_q + self.n_k)
        for leaf in ("lq1", "lk1", "lq2", "lk2"):
            m[leaf] = (getattr(self, leaf), 0)
        return m

    def finish_loading(self) -> None:
        d = {k: getattr(self, k).data.double() for k in ("lq1", "lk1", "lq2", "lk2")}
        self.lam = float(torch.exp((d["lq1"] * d["lk1"]).sum())
                         - torch.exp((d["lq2"] * d["lk2"]).sum())) + self.diff
        self.conv_w_t.copy_(self.conv_w.data.t())

    def cache_layout(self, block_size: int, dtype) -> dict:
        out = {}
        if not self.shared_kv:
            out["k"] = ("paged", (self.G, block_size, self.MAPS * self.D), dtype)
            out["v"] = ("paged", (self.G, block_size, self.V), dtype)
        if self.taps > 1:
            out["conv"] = ("slot", (self.taps - 1, self.ch), torch.float32)
        return out

    def _prompt_tiles(self, batch: ForwardBatch, q):
        """Work lists of the prefill kernels for a step that holds prompt
        portions (host-built once per step and head layout); None where the
        masked or general kernels run: steps whose longest portion does not
        fill a 256-row tile (the masked tiles are as fast there), captured
        graphs, float32, CPU, head sizes those kernels are not built for."""
        if (not q.is_cuda or q.dtype != torch.bfloat16 or self.D != self.V
                or self.D not in ops.PREFILL_MAP_DIMS or not ops.use_ladder_maps
                or batch.kv_lens_list is None
                or batch.max_q_len < ops.EXTEND2_QTILE):
            return None
        key = ("maps", self.H * self.MAPS, self.D)
        if key not in batch.tile_cache:
            batch.tile_cache[key] = ops.build_extend_tiles(
                batch.seq_lens_list, batch.kv_lens_list, False, q.device,
                num_q_heads=self.H * self.MAPS, flash_decode=False)
        return batch.tile_cache[key]

    def core(self, p, batch: ForwardBatch, cache: dict, out, out_scale) -> None:
        assert out_scale == 1.0
        T = p.shape[0]
        H, G, D, V, M = self.H, self.G, self.D, self.V, self.MAPS
        q = ops.conv_qkv_cache(
            p, self.n_q, self.n_k, self.n_v, self.conv_w, self.conv_w_t,
            cache.get("conv"), batch.cu_seqlens, batch.seq_lens,
            batch.state_slots, batch.token_seq, batch.positions,
            self.temp_coef, self.temp_every, H, G, M, cache["k"], cache["v"],
            batch.slot_mapping)
        q = q.view(T, H * M, D)
        tiles = self._prompt_tiles(batch, q)
        if tiles is not None:
            # steps with prompt portions: the framework's work-sorted
            # prefill kernels (256-row ladder, 64-row) read the two-map rows
            a = ops.attention_extend_paged(
                q, cache["k"], cache["v"], batch.block_tables, batch.seq_lens,
                batch.cu_seqlens, None, self.scale, tiles=tiles,
                native=ops.seq_extension(), maps=M)
        else:
            a = ops.attention_sink_paged(
                q, cache["k"], cache["v"], batch.block_tables, batch.seq_lens,
                batch.cu_seqlens, batch.token_seq, self.scale, False, None,
                False, batch.max_q_len, batch.positions, maps=M)
        ops.diff_head_norm_gate(a, p[:, self.ch:self.ch + H * V], self.lam,
                                self.eps, 1.0 - self.diff, H, G, out)


class ParallelMixer(nn.Module):
    """left_scale * left(h) + right_scale * right(h) for two split mixers:
    one GEMM projects h for both, each core() writes its head outputs,
    already multiplied by its scale, into its columns of one buffer, and
    one GEMM over [W_o,left | W_o,right] sums the two results. The left
    out-projection's bias (times its scale) is handed to the caller as
    out_bias (fp32), to be added where the result meets the residual."""

    def __init__(self, width: int, left: SplitMixer, right: SplitMixer,
                 left_scale: float, right_scale: float, dtype):
        super().__init__()
        self.left, self.right = left, right
        self.scales = (float(left_scale), float(right_scale))
        self._spans = [("left." + n, r, b) for n, r, b in left.in_spans()] + \
                      [("right." + n, r, b) for n, r, b in right.in_spans()]
        self.rows = (sum(r for _, r, _ in left.in_spans()),
                     sum(r for _, r, _ in right.in_spans()))
        self.cols = (left.out_cols, right.out_cols)
        self.w_in = _param(sum(self.rows), width, dtype=dtype)
        self.b_in = (_param(sum(self.rows), dtype=dtype)
                     if any(b for _, _, b in self._spans) else None)
        self.w_out = _param(width, sum(self.cols), dtype=dtype)
        self.o_b = {side: _param(width, dtype=torch.float32)
                    for side, m in (("left", left), ("right", right))
                    if m.out_has_bias}
        for side, p in self.o_b.items():
            self.register_parameter("o_b_" + side, p)
        self.out_bias = (_param(width, dtype=torch.float32)
                         if self.o_b else None)

    def weight_map(self) -> dict:
        m, row = {}, 0
        for name, n, has_b in self._spans:
            m[name] = (self.w_in, row)
            if has_b:
                m[name + ".b"] = (self.b_in, row)
            row += n
        width = self.w_out.shape[0]
        m["left.o"] = (self.w_out, 0, 0, (width, self.cols[0]))
        m["right.o"] = (self.w_out, 0, self.cols[0], (width, self.cols[1]))
        for side in self.o_b:
            m[side + ".o.b"] = (getattr(self, "o_b_" + side), 0)
        return m

    def finish_loading(self) -> None:
        if self.out_bias is not None:
            total = torch.zeros_like(self.out_bias.data)
            for side, scale in zip(("left", "right"), self.scales):
                if side in self.o_b:
                    total += scale * getattr(self, "o_b_" + side).data
            self.out_bias.data.copy_(total)

    def cache_layout(self, block_size: int, dtype) -> dict:
        out = {"left." + k: v
               for k, v in self.left.cache_layout(block_size, dtype).items()}
        out.update({"right." + k: v for k, v in
                    self.right.cache_layout(block_size, dtype).items()})
        return out

    def forward(self, xs, batch: ForwardBatch, cache: dict) -> torch.Tensor:
        p = linear(xs, self.w_in, self.b_in)
        out = torch.empty((xs.shape[0], sum(self.cols)), dtype=xs.dtype,
                          device=xs.device)
        lc = {k[5:]: v for k, v in cache.items() if k.startswith("left.")}
        rc = {k[6:]: v for k, v in cache.items() if k.startswith("right.")}
        self.left.core(p[:, :self.rows[0]], batch, lc, out[:, :self.cols[0]],
                       self.scales[0])
        self.right.core(p[:, self.rows[0]:], batch, rc, out[:, self.cols[0]:],
                        self.scales[1])
        return linear(out, self.w_out)


def build_mixer(kind: str, m: dict, width: int, eps: float, dtype,
                arch: str = "", own_projections: bool = True) -> nn.Module:
    if arch == "Legalix":
        if kind == "attention":
            return SinkRotaryAttention(
                width, m["heads"], m["kv_heads"], m["dim"], m["vdim"],
                m["scale"], m["rot"]["base"], m["rot"]["dims"], eps, dtype,
                qk_norm=False, sink=False, rotate_values=False,
                interleaved=False, softcap=m.get("softcap") or 0.0,
                window=(m.get("mask") or {}).get("size") or 0,
                keep_first=(m.get("mask") or {}).get("keep_first") or 0,
                own_projections=own_projections)
        if kind == "latent_attention":
            return LatentAttention(
                width, m["heads"], m["dim"], m["rot_dim"], m["vdim"],
                m["kv_rank"], m["q_rank"], m["scale"], m["rot"]["base"], eps,
                dtype, own_projections=own_projections)
        if kind == "mamba2":
            return Mamba2Mixer(
                width, m["heads"], m["vdim"], m["state"], m["groups"],
                m["norm_groups"], m["conv"], eps, dtype,
                own_projections=own_projections)
        raise ValueError(f"unknown mixer type {kind!r}")
    if arch == "Rivolix":
        if kind == "attention":
            temp = m.get("q_temp") or {}
            return DiffAttention(
                width, m["heads"], m["kv_heads"], m["dim"], m["vdim"],
                m["scale"], m["diff"], m["conv"], temp.get("coef", 0.0),
                temp.get("every", 0), eps, dtype,
                shared_kv=m.get("kv_from") is not None,
                own_projections=own_projections)
        if kind == "attention_2":
            if m["vdim"] != m["dim"]:
                raise ValueError("attention_2: the values are the keys, "
                                 "so vdim must equal dim")
            rot = m.get("rot") or {"base": 10000.0, "dims": 0}
            return SinkRotaryAttention(
                width, m["heads"], m["kv_heads"], m["dim"], m["vdim"],
                m["scale"], rot["base"], rot["dims"], eps, dtype,
                qk_norm=False, sink=False, rotate_values=False,
                interleaved=False, own_projections=own_projections,
                rot_scaling=rot.get("scaling"), unit_norm_after=True,
                value_is_key=True)
        raise ValueError(f"unknown mixer type {kind!r}")
    if kind == "attention":
        return SinkRotaryAttention(
            width, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"],
            m["rot"]["base"], m["rot"]["dims"], eps, dtype)
    if kind == "lightning":
        return LightningMixer(width, m["heads"], m["dim"], m["vdim"],
                              m["decay"], eps, dtype)
    if kind == "mamba1":
        return Mamba1Mixer(width, m["inner"], m["state"], m["dt_rank"],
                           m["conv"], dtype)
    if kind == "parallel":
        L, R = m["left"], m["right"]
        left = WindowPoolAttention(
            width, L["heads"], L["kv_heads"], L["dim"], L["vdim"], L["scale"],
            L["mask"]["size"], L["mask"]["pool"], dtype,
            own_projections=False)
        right = RetentionMixer(
            width, R["heads"], R["dim"], R["vdim"], R["decay"],
            R["rot"]["base"], R["rot"]["dims"], eps, dtype,
            own_projections=False)
        return ParallelMixer(width, left, right, m["left_scale"],
                             m["right_scale"], dtype)
    raise ValueError(f"unknown mixer type {kind!r}")
