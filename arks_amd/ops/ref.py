"""Reference implementations of every arks_amd custom op, in plain PyTorch.

These are the numerics oracle for the HIP kernels (tests compare the gfx950
kernels against these run in fp32) and the compute path for CPU-only unit
tests of the engine/scheduler/model layers. They are NOT a runtime fallback:
on a GPU box the HIP extension is required and ops fail loudly without it
(see arks_amd/ops/__init__.py).

Conventions shared with the kernels:
- KV cache layout: [num_blocks, num_kv_heads, block_size, head_dim]
- block_tables: int32 [num_seqs, max_blocks_per_seq]
- slot_mapping: int64 flat slot index = block_id * block_size + offset
"""

from __future__ import annotations

import math

import torch


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """RMSNorm over the last dim. Accumulates in fp32 like the kernel."""
    dtype = x.dtype
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    out = xf * torch.rsqrt(var + eps) * weight.float()
    return out.to(dtype)


def fused_add_rmsnorm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6
) -> tuple[torch.Tensor, torch.Tensor]:
    """residual += x; out = rmsnorm(residual). Returns (out, new_residual)."""
    new_residual = (residual.float() + x.float()).to(x.dtype)
    return rmsnorm(new_residual, weight, eps), new_residual


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    """SwiGLU activation: input [..., 2*d] as [gate | up] -> silu(gate) * up."""
    d = gate_up.shape[-1] // 2
    gate = gate_up[..., :d].float()
    up = gate_up[..., d:].float()
    return (torch.nn.functional.silu(gate) * up).to(gate_up.dtype)


def _scaled_inv_freq(inv_freq: torch.Tensor, rope_scaling: dict | None,
                     base: float, head_dim: int) -> tuple[torch.Tensor, float]:
    """Apply an HF rope_scaling config; returns (inv_freq, mscale).
    Supports the llama3 ramp, YaRN (NTK-by-parts + attention scaling) and
    plain linear scaling — matching transformers' rope_utils semantics."""
    if not rope_scaling:
        return inv_freq, 1.0
    rtype = rope_scaling.get("rope_type") or rope_scaling.get("type")
    factor = float(rope_scaling.get("factor", 1.0))
    if rtype == "linear":
        return inv_freq / factor, 1.0
    if rtype == "llama3":
        lo = float(rope_scaling.get("low_freq_factor", 1.0))
        hi = float(rope_scaling.get("high_freq_factor", 4.0))
        orig = float(rope_scaling.get("original_max_position_embeddings", 8192))
        wavelen = 2 * math.pi / inv_freq
        scaled = torch.where(wavelen > orig / lo, inv_freq / factor, inv_freq)
        smooth = (orig / wavelen - lo) / (hi - lo)
        mid = (1 - smooth) * inv_freq / factor + smooth * inv_freq
        is_mid = (wavelen <= orig / lo) & (wavelen >= orig / hi)
        return torch.where(is_mid, mid, scaled), 1.0
    if rtype == "yarn":
        orig = float(rope_scaling.get("original_max_position_embeddings", 4096))
        beta_fast = float(rope_scaling.get("beta_fast", 32.0))
        beta_slow = float(rope_scaling.get("beta_slow", 1.0))

        def corr_dim(num_rot: float) -> float:
            return (head_dim * math.log(orig / (num_rot * 2 * math.pi))) / (
                2 * math.log(base))

        low = max(math.floor(corr_dim(beta_fast)), 0)
        high = min(math.ceil(corr_dim(beta_slow)), head_dim // 2 - 1)
        ramp = torch.clamp(
            (torch.arange(head_dim // 2, dtype=torch.float64,
                          device=inv_freq.device) - low) / max(high - low, 1),
            0, 1,
        )
        # ramp==0 (high-freq dims) -> extrapolate (keep original);
        # ramp==1 (long wavelengths) -> interpolate (divide by factor)
        out = (inv_freq / factor) * ramp + inv_freq * (1 - ramp)
        mscale = float(rope_scaling.get("attention_factor") or
                       (0.1 * math.log(factor) + 1.0))
        return out, mscale
    return inv_freq, 1.0


def rope_cos_sin_cache(
    head_dim: int,
    max_positions: int,
    base: float = 10000.0,
    dtype: torch.dtype = torch.float32,
    device=None,
    rope_scaling: dict | None = None,
) -> torch.Tensor:
    """Precomputed [max_positions, head_dim] cache: first half cos, second half sin
    (per rotary pair), matching HF neox-style RoPE (incl. llama3 / yarn /
    linear rope_scaling)."""
    inv_freq = 1.0 / (
        base ** (torch.arange(0, head_dim, 2, dtype=torch.float64, device=device) / head_dim)
    )
    inv_freq, mscale = _scaled_inv_freq(inv_freq, rope_scaling, base, head_dim)
    t = torch.arange(max_positions, dtype=torch.float64, device=device)
    freqs = torch.outer(t, inv_freq)  # [P, head_dim/2]
    cache = torch.cat([freqs.cos() * mscale, freqs.sin() * mscale], dim=-1)
    return cache.to(dtype)


def rope_apply(
    positions: torch.Tensor,  # [num_tokens] int
    q: torch.Tensor,  # [num_tokens, num_q_heads * head_dim]
    k: torch.Tensor,  # [num_tokens, num_kv_heads * head_dim]
    cos_sin: torch.Tensor,  # [max_pos, head_dim]
    head_dim: int,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Neox-style (rotate-half) RoPE applied out-of-place to q and k."""

    def _rot(x: torch.Tensor) -> torch.Tensor:
        n = x.shape[0]
        xf = x.float().view(n, -1, head_dim)
        half = head_dim // 2
        cs = cos_sin.float()[positions]  # [n, head_dim]
        cos = cs[:, :half].unsqueeze(1)  # [n, 1, half]
        sin = cs[:, half:].unsqueeze(1)
        x1 = xf[..., :half]
        x2 = xf[..., half:]
        o1 = x1 * cos - x2 * sin
        o2 = x2 * cos + x1 * sin
        return torch.cat([o1, o2], dim=-1).view(n, -1).to(x.dtype)

    return _rot(q), _rot(k)


def reshape_and_cache(
    k: torch.Tensor,  # [num_tokens, num_kv_heads, head_dim]
    v: torch.Tensor,
    k_cache: torch.Tensor,  # [num_blocks, num_kv_heads, block_size, head_dim]
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,  # [num_tokens] int64
) -> None:
    block_size = k_cache.shape[2]
    block_ids = slot_mapping // block_size
    offsets = slot_mapping % block_size
    k_cache[block_ids, :, offsets] = k.to(k_cache.dtype)
    v_cache[block_ids, :, offsets] = v.to(v_cache.dtype)


def attention_prefill_varlen(
    q: torch.Tensor,  # [total_tokens, num_q_heads, head_dim]
    k: torch.Tensor,  # [total_tokens, num_kv_heads, head_dim]
    v: torch.Tensor,
    cu_seqlens: torch.Tensor,  # [num_seqs + 1] int32
    scale: float,
    window: int = 0,
) -> torch.Tensor:
    """Causal attention over packed variable-length sequences (full prefill:
    keys == the packed k/v of the same forward). GQA by head repetition.
    window > 0 = sliding-window attention."""
    num_q_heads = q.shape[1]
    num_kv_heads = k.shape[1]
    rep = num_q_heads // num_kv_heads
    out = torch.empty_like(q)
    for i in range(cu_seqlens.numel() - 1):
        s, e = int(cu_seqlens[i]), int(cu_seqlens[i + 1])
        qi = q[s:e].float().transpose(0, 1)  # [H, L, D]
        ki = k[s:e].float().repeat_interleave(rep, dim=1).transpose(0, 1)
        vi = v[s:e].float().repeat_interleave(rep, dim=1).transpose(0, 1)
        L = e - s
        scores = torch.matmul(qi, ki.transpose(-1, -2)) * scale  # [H, L, L]
        mask = torch.triu(
            torch.full((L, L), float("-inf"), device=q.device), diagonal=1
        )
        if window > 0:
            mask = mask + torch.tril(
                torch.full((L, L), float("-inf"), device=q.device),
                diagonal=-window,
            )
        scores = scores + mask
        p = torch.softmax(scores, dim=-1)
        o = torch.matmul(p, vi)  # [H, L, D]
        out[s:e] = o.transpose(0, 1).to(q.dtype)
    return out


def attention_decode_paged(
    q: torch.Tensor,  # [num_seqs, num_q_heads, head_dim]
    k_cache: torch.Tensor,  # [num_blocks, num_kv_heads, block_size, head_dim]
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,  # [num_seqs, max_blocks] int32
    seq_lens: torch.Tensor,  # [num_seqs] int32 (length INCLUDING current token)
    scale: float,
    window: int = 0,
) -> torch.Tensor:
    """Single-token decode attention against the paged KV cache.
    window > 0 = sliding-window (the query sees the last `window` keys)."""
    num_seqs, num_q_heads, head_dim = q.shape
    num_kv_heads = k_cache.shape[1]
    block_size = k_cache.shape[2]
    rep = num_q_heads // num_kv_heads
    out = torch.empty_like(q)
    for i in range(num_seqs):
        L = int(seq_lens[i])
        nblocks = (L + block_size - 1) // block_size
        bt = block_tables[i, :nblocks].long()
        # gather [L, num_kv_heads, head_dim]
        ks = k_cache[bt].permute(0, 2, 1, 3).reshape(nblocks * block_size, num_kv_heads, head_dim)[:L]
        vs = v_cache[bt].permute(0, 2, 1, 3).reshape(nblocks * block_size, num_kv_heads, head_dim)[:L]
        kf = ks.float().repeat_interleave(rep, dim=1)  # [L, H, D]
        vf = vs.float().repeat_interleave(rep, dim=1)
        qi = q[i].float()  # [H, D]
        scores = torch.einsum("hd,lhd->hl", qi, kf) * scale
        if window > 0 and L > window:
            scores[:, : L - window] = float("-inf")
        p = torch.softmax(scores, dim=-1)
        o = torch.einsum("hl,lhd->hd", p, vf)
        out[i] = o.to(q.dtype)
    return out


def attention_extend_paged(
    q: torch.Tensor,  # [total_new_tokens, num_q_heads, head_dim]
    k_cache: torch.Tensor,  # [num_blocks, num_kv_heads, block_size, head_dim]
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,  # [num_seqs, max_blocks] int32
    kv_lens: torch.Tensor,  # [num_seqs] int32 total kv length per seq
    cu_seqlens_q: torch.Tensor,  # [num_seqs + 1] int32 (packed new tokens)
    scale: float,
    window: int = 0,
) -> torch.Tensor:
    """Causal attention of each sequence's new tokens over its full paged KV
    (prefix caching / chunked prefill). New token j of seq i sits at global
    position kv_len - q_len + j. window > 0 = sliding-window attention
    (each query sees only the last `window` key positions)."""
    num_q_heads, head_dim = q.shape[1], q.shape[2]
    num_kv_heads = k_cache.shape[1]
    block_size = k_cache.shape[2]
    rep = num_q_heads // num_kv_heads
    out = torch.empty_like(q)
    for i in range(cu_seqlens_q.numel() - 1):
        s, e = int(cu_seqlens_q[i]), int(cu_seqlens_q[i + 1])
        qn = e - s
        L = int(kv_lens[i])
        off = L - qn
        nblocks = (L + block_size - 1) // block_size
        bt = block_tables[i, :nblocks].long()
        ks = k_cache[bt].permute(0, 2, 1, 3).reshape(nblocks * block_size, num_kv_heads, head_dim)[:L]
        vs = v_cache[bt].permute(0, 2, 1, 3).reshape(nblocks * block_size, num_kv_heads, head_dim)[:L]
        kf = ks.float().repeat_interleave(rep, dim=1).transpose(0, 1)  # [H, L, D]
        vf = vs.float().repeat_interleave(rep, dim=1).transpose(0, 1)
        qi = q[s:e].float().transpose(0, 1)  # [H, qn, D]
        scores = torch.matmul(qi, kf.transpose(-1, -2)) * scale  # [H, qn, L]
        kpos = torch.arange(L, device=q.device)
        qpos = torch.arange(off, L, device=q.device)
        mask = kpos[None, :] > qpos[:, None]  # [qn, L] True = hidden
        if window > 0:
            mask |= kpos[None, :] <= qpos[:, None] - window
        scores = scores.masked_fill(mask, float("-inf"))
        p = torch.softmax(scores, dim=-1)
        o = torch.matmul(p, vf)  # [H, qn, D]
        out[s:e] = o.transpose(0, 1).to(q.dtype)
    return out


def moe_topk(router_logits: torch.Tensor, k: int, renorm: bool):
    """softmax + top-k (+ renorm): (weights [T,k] f32, ids [T,k] i32)."""
    probs = torch.softmax(router_logits.float(), dim=-1)
    weights, selected = probs.topk(k, dim=-1)
    if renorm:
        weights = weights / weights.sum(dim=-1, keepdim=True)
    return weights, selected.to(torch.int32)


def moe_mix(y: torch.Tensor, weights: torch.Tensor, ids: torch.Tensor,
            expert_base: int = 0) -> torch.Tensor:
    """Weighted mix of per-(local-)expert dense outputs y [El, T, H]."""
    El, T, H = y.shape
    le = ids.long() - expert_base
    mine = (le >= 0) & (le < El)
    le = le.clamp(0, El - 1)
    t_idx = torch.arange(T, device=y.device)[:, None].expand_as(le)
    gathered = y[le, t_idx].float()  # [T, k, H]
    w = torch.where(mine, weights, torch.zeros_like(weights))
    return torch.einsum("tkh,tk->th", gathered, w.float()).to(y.dtype)


def moe_mix_rows(y: torch.Tensor, weights: torch.Tensor,
                 rows: torch.Tensor, add=None) -> torch.Tensor:
    """out[t] = sum_j weights[t,j] * y[rows[t,j]] (+ add[t]) over a flat
    [R, H] expert-output buffer."""
    gathered = y[rows.long()].float()  # [T, k, H]
    out = torch.einsum("tkh,tk->th", gathered, weights.float())
    if add is not None:
        out = out + add.float()
    return out.to(y.dtype)


def quant_fp8_rows(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-row symmetric quantization to OCP e4m3 (range +-448)."""
    amax = x.float().abs().amax(dim=1).clamp(min=1e-6)
    scale = 448.0 / amax
    q = (x.float() * scale[:, None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q, (1.0 / scale)


def greedy_sample(logits: torch.Tensor) -> torch.Tensor:
    """[num_seqs, vocab] -> [num_seqs] int64 argmax."""
    return logits.float().argmax(dim=-1)


def gumbel_sample(
    logits: torch.Tensor,  # [num_seqs, vocab]
    temperatures: torch.Tensor,  # [num_seqs] float; 0 => greedy
    uniform: torch.Tensor,  # [num_seqs, vocab] uniform(0,1) noise
) -> torch.Tensor:
    """Exact categorical sampling via the Gumbel-max trick:
    argmax(logits/T + Gumbel) ~ softmax(logits/T). T==0 rows are greedy."""
    lf = logits.float()
    t = temperatures.float().clamp(min=0.0).unsqueeze(1)
    gumbel = -torch.log(-torch.log(uniform.float().clamp(1e-20, 1.0)))
    scaled = torch.where(t > 0, lf / t.clamp(min=1e-8) + gumbel, lf)
    return scaled.argmax(dim=-1)


def softmax_scale(head_dim: int) -> float:
    return 1.0 / math.sqrt(head_dim)


# ----------------------------------------------------------------------
# Sequence-state ops (token shift, gated output norm, sink attention with
# rotated values, lightning linear attention, mamba1 conv + selective scan).
# Shared conventions: rows of a step are packed [T, ...]; cu_seqlens[s] is
# the first row of sequence s, seq_lens[s] its length INCLUDING this step's
# rows (so its first new position is seq_lens[s] - rows), state_slots[s] the
# row of every per-sequence state tensor (-1 = padding: read zeros, write
# nothing). A sequence whose first new position is 0 starts from zero state
# whatever its slot holds, so slots are reused without clearing.
# ----------------------------------------------------------------------
def _seq_spans(cu_seqlens, seq_lens, state_slots):
    cu = cu_seqlens.tolist()
    sl = seq_lens.tolist()
    slots = state_slots.tolist()
    for s in range(len(sl)):
        a, b = cu[s], cu[s + 1]
        if b > a:
            yield a, b, sl[s] - (b - a), slots[s]


def token_shift(x, shift_w, prev_state, cu_seqlens, seq_lens, state_slots,
                out_dtype):
    """xs[t] = x[t] + (x[t-1] - x[t]) * shift_w, x[-1] of a sequence being
    the last row of its previous step (prev_state) or zero at position 0.
    Stores each sequence's last row into prev_state. Returns (xs, x) cast
    to out_dtype."""
    xs = torch.empty_like(x)
    w = shift_w.float()
    for a, b, start, slot in _seq_spans(cu_seqlens, seq_lens, state_slots):
        first = (prev_state[slot].clone() if start > 0 and slot >= 0
                 else torch.zeros_like(x[a]))
        prev = torch.cat([first[None], x[a:b - 1]], 0)
        xs[a:b] = x[a:b] + (prev - x[a:b]) * w
        if slot >= 0:
            prev_state[slot] = x[b - 1]
    return xs.to(out_dtype), x.to(out_dtype)


def gated_norm_residual(x, y, gate, gate_bias, weight, eps, out_dtype=None):
    """x += rmsnorm(y * sigmoid(gate + gate_bias)) * weight, everything in
    fp32, x updated in place; gate None = no gate. Returns x cast to
    out_dtype (or None)."""
    z = y.float()
    if gate is not None:
        z = z * torch.sigmoid(gate.float() + gate_bias.float())
    r = z * torch.rsqrt(z.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    x += r
    return x.to(out_dtype) if out_dtype is not None else None


def rms_norm_f32(x, weight, eps, out_dtype):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
            * weight.float()).to(out_dtype)


def _rotate_pairs(x, angles, interleaved: bool):
    """x [..., 2*P] turned pairwise by angles [..., P] (fp32)."""
    c, s = torch.cos(angles), torch.sin(angles)
    out = torch.empty_like(x)
    if interleaved:
        u, w = x[..., 0::2], x[..., 1::2]
        out[..., 0::2] = u * c - w * s
        out[..., 1::2] = w * c + u * s
    else:
        P = x.shape[-1] // 2
        u, w = x[..., :P], x[..., P:]
        out[..., :P] = u * c - w * s
        out[..., P:] = w * c + u * s
    return out


def qk_norm_rope_cache(q, k, v, q_norm_w, k_norm_w, eps, positions,
                       inv_freq_qk, inv_freq_v, k_cache, v_cache,
                       slot_mapping, interleaved=True, rot_mag=1.0,
                       unit_norm_after=False):
    """q [T,H,D], k [T,G,D], v [T,G,V]: per-head RMS norm of q and k (weights
    or None), rotary on their first 2*len(inv_freq_qk) dims with cos and sin
    times rot_mag, then (unit_norm_after) q and k divided by their root mean
    square over the head once more, without a weight; values turned by
    their own position over all V dims (inv_freq_v None = values stored
    plain); k and v go to the paged cache. Returns q (fp32 math, q.dtype)."""
    pos = positions.float()

    def prep(t, w, inv_freq, mag=1.0, after=False):
        tf = t.float()
        if w is not None:
            tf = tf * torch.rsqrt(tf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
        if inv_freq is not None and inv_freq.numel():
            rd = 2 * inv_freq.numel()
            ang = pos[:, None, None] * inv_freq.float()[None, None, :]
            tf = torch.cat([_rotate_pairs(tf[..., :rd], ang, interleaved) * mag,
                            tf[..., rd:]], -1)
        if after:
            tf = tf * torch.rsqrt(tf.pow(2).mean(-1, keepdim=True) + eps)
        return tf

    qo = prep(q, q_norm_w, inv_freq_qk, rot_mag, unit_norm_after).to(q.dtype)
    ko = prep(k, k_norm_w, inv_freq_qk, rot_mag, unit_norm_after).to(k_cache.dtype)
    vo = prep(v, None, inv_freq_v).to(v_cache.dtype)
    bs = k_cache.shape[2]
    ok = slot_mapping >= 0
    blk = (slot_mapping[ok] // bs).long()
    off = (slot_mapping[ok] % bs).long()
    k_cache[blk, :, off] = ko[ok]
    v_cache[blk, :, off] = vo[ok]
    return qo


def attention_sink_paged(q, k_cache, v_cache, block_tables, seq_lens,
                         cu_seqlens, scale, sink=True, inv_freq_v=None,
                         interleaved=True, sink_w=None, softcap=0.0,
                         window=0, keep_first=0, maps=1):
    """Causal attention of packed new rows over each sequence's paged keys.
    maps M > 1: a key row holds M keys of D dims side by side (k_cache
    [pages, G, bs, M*D]) that share the row's value; q has G*M groups of
    query heads, group g*M + m reads key m of key/value head g.
    sink=True adds a value-less key of score 0 to every softmax (one more
    in the denominator); sink_w [H] gives that key a score per head
    instead (taken as it is: neither scaled nor capped). softcap c > 0:
    scores become c tanh(score / c). window w > 0: the row at position i
    sees key j only if i - j < w or j < keep_first. inv_freq_v: each row's
    output is turned back by its own position over the value dims. v_cache
    may be a view into k_cache's rows. q [T,H,D] -> [T,H,V] in q.dtype."""
    T, H, D = q.shape
    G, bs, V = v_cache.shape[1], v_cache.shape[2], v_cache.shape[3]
    out = torch.zeros(T, H, V, dtype=torch.float32)
    cu = cu_seqlens.tolist()
    sl = seq_lens.tolist()
    for s in range(len(sl)):
        a, b = cu[s], cu[s + 1]
        n, L = b - a, sl[s]
        if n == 0:
            continue
        nb = (L + bs - 1) // bs
        pages = block_tables[s, :nb].long()
        K = k_cache[pages].permute(1, 0, 2, 3).reshape(G, nb * bs, maps * D)[:, :L].float()
        Vv = v_cache[pages].permute(1, 0, 2, 3).reshape(G, nb * bs, V)[:, :L].float()
        if maps > 1:
            K = K.view(G, L, maps, D).transpose(1, 2).reshape(G * maps, L, D)
            Vv = Vv.repeat_interleave(maps, 0)
        K = K.repeat_interleave(H // (G * maps), 0)
        Vv = Vv.repeat_interleave(H // (G * maps), 0)
        qs = q[a:b].float().permute(1, 0, 2)  # [H, n, D]
        sc = torch.matmul(qs, K.transpose(1, 2)) * scale  # [H, n, L]
        qpos = torch.arange(L - n, L)
        if softcap > 0:
            sc = softcap * torch.tanh(sc / softcap)
        kpos = torch.arange(L)[None, :]
        mask = kpos > qpos[:, None]
        if window > 0:
            mask = mask | ((qpos[:, None] - kpos >= window)
                           & (kpos >= keep_first))
        sc = sc.masked_fill(mask[None], float("-inf"))
        m = sc.amax(-1, keepdim=True)
        if sink_w is not None:
            sk = sink_w.float()[:, None, None]
            m = torch.maximum(m, sk)
        elif sink:
            sk = torch.zeros(())
            m = m.clamp(min=0.0)
        e = torch.exp(sc - m)
        den = e.sum(-1, keepdim=True)
        if sink or sink_w is not None:
            den = den + torch.exp(sk - m)
        o = torch.matmul(e / den, Vv).permute(1, 0, 2)  # [n, H, V]
        if inv_freq_v is not None:
            ang = -qpos.float()[:, None, None] * inv_freq_v.float()[None, None, :]
            o = _rotate_pairs(o, ang, interleaved)
        out[a:b] = o
    return out.to(q.dtype)


def lightning_scan(q, k, v, decay, state, cu_seqlens, seq_lens, state_slots):
    """Per head S <- decay*S + silu(k) silu(v)^T, o = S^T silu(q); q,k
    [T,H,D], v [T,H,V], state [slots,H,D,V] fp32 (updated). -> o fp32
    [T,H,V]."""
    T, H, D = q.shape
    V = v.shape[-1]
    F = torch.nn.functional
    qf, kf, vf = F.silu(q.float()), F.silu(k.float()), F.silu(v.float())
    out = torch.zeros(T, H, V, dtype=torch.float32)
    lam = decay.float()[:, None, None]
    for a, b, start, slot in _seq_spans(cu_seqlens, seq_lens, state_slots):
        S = (state[slot].clone() if start > 0 and slot >= 0
             else torch.zeros(H, D, V))
        for t in range(a, b):
            S = lam * S + kf[t][:, :, None] * vf[t][:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        if slot >= 0:
            state[slot] = S
    return out


def gated_rmsnorm(o, weight, gate, eps, out_dtype):
    """rmsnorm(o) * weight * sigmoid(gate) over the last dim."""
    of = o.float()
    y = of * torch.rsqrt(of.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    return (y * torch.sigmoid(gate.float())).to(out_dtype)


def causal_conv_silu(x, weight, bias, state, cu_seqlens, seq_lens,
                     state_slots):
    """Depthwise causal conv over time then silu. x [T,C]; weight [C,taps]
    (last column = current row); state [slots,taps-1,C] fp32 holds each
    sequence's last taps-1 inputs (updated)."""
    T, C = x.shape
    taps = weight.shape[1]
    xf = x.float()
    out = torch.empty(T, C, dtype=torch.float32)
    for a, b, start, slot in _seq_spans(cu_seqlens, seq_lens, state_slots):
        hist = (state[slot].clone() if start > 0 and slot >= 0 and taps > 1
                else torch.zeros(taps - 1, C))
        full = torch.cat([hist, xf[a:b]], 0)  # [taps-1+n, C]
        n = b - a
        acc = bias.float()[None, :].expand(n, C).clone()
        for j in range(taps):
            acc += full[j:j + n] * weight.float()[:, j][None, :]
        out[a:b] = acc
        if slot >= 0 and taps > 1:
            state[slot] = full[n:]
    return torch.nn.functional.silu(out).to(x.dtype)


def selective_scan(u, dbc, z, dt_w, dt_b, A, Dp, state, cu_seqlens,
                   seq_lens, state_slots):
    """Mamba1 recurrence. u [T,C] (conv output), dbc [T,R+2N] = [dt|B|C],
    z [T,C] gate, dt_w [C,R], A [C,N] (negative), state [slots,C,N] fp32
    (updated). -> y [T,C] in u.dtype, y = (S.C + D u) * silu(z)."""
    T, C = u.shape
    R = dt_w.shape[1]
    N = A.shape[1]
    uf, zf, df = u.float(), z.float(), dbc.float()
    dt = torch.nn.functional.softplus(df[:, :R] @ dt_w.float().t() + dt_b.float())
    Bm, Cm = df[:, R:R + N], df[:, R + N:R + 2 * N]
    out = torch.empty(T, C, dtype=torch.float32)
    Af = A.float()
    for a, b, start, slot in _seq_spans(cu_seqlens, seq_lens, state_slots):
        S = (state[slot].clone() if start > 0 and slot >= 0
             else torch.zeros(C, N))
        for t in range(a, b):
            S = torch.exp(dt[t][:, None] * Af) * S + (dt[t] * uf[t])[:, None] * Bm[t][None, :]
            out[t] = S @ Cm[t] + Dp.float() * uf[t]
        if slot >= 0:
            state[slot] = S
    return (out * torch.nn.functional.silu(zf)).to(u.dtype)


def gelu_tanh(x):
    return torch.nn.functional.gelu(x.float(), approximate="tanh").to(x.dtype)


# ----------------------------------------------------------------------
# Stream-residual blocks (several weighted copies of the residual), layer
# norm, the short input convolution, window attention with pooled blocks,
# rotary retention, clamped GLU and grouped routing.
# ----------------------------------------------------------------------
def stream_mix_norm(xs, y, y_bias, mix, out_w, in_w, norm_w, norm_b, eps):
    """xs [s, T, C] fp32, updated in place when y is given:
        new[t] = sum_s mix[s, t] old[s] + out_w[t] * (y + y_bias)
    then u = sum_s in_w[s] new[s] and the layer norm of u (mean taken off,
    variance = mean squared deviation, eps inside the root) times norm_w
    plus norm_b -> fp32 [T, C]. in_w None: only the update."""
    if y is not None:
        yf = y.float()
        if y_bias is not None:
            yf = yf + y_bias.float()
        new = torch.einsum("st,snc->tnc", mix.float(), xs) \
            + out_w.float()[:, None, None] * yf[None]
        xs.copy_(new)
    if in_w is None:
        return None
    u = torch.einsum("s,snc->nc", in_w.float(), xs)
    mu = u.mean(-1, keepdim=True)
    d = u - mu
    var = d.pow(2).mean(-1, keepdim=True)
    return d * torch.rsqrt(var + eps) * norm_w.float() + norm_b.float()


def short_conv_residual(h, weight, state, cu_seqlens, seq_lens, state_slots,
                        out_dtype):
    """out_t = h_t + sum_j weight[:, j] h_(t - taps + 1 + j) per channel,
    causal within each sequence; h [T, C] fp32, weight [C, taps] fp32, state
    [slots, taps-1, C] fp32 = each sequence's last taps-1 inputs (updated).
    taps == 1 needs no state (state None)."""
    T, C = h.shape
    taps = weight.shape[1]
    wf = weight.float()
    out = torch.empty(T, C, dtype=torch.float32)
    for a, b, start, slot in _seq_spans(cu_seqlens, seq_lens, state_slots):
        hist = (state[slot].clone() if start > 0 and slot >= 0 and taps > 1
                else torch.zeros(taps - 1, C))
        full = torch.cat([hist, h[a:b].float()], 0)
        n = b - a
        acc = h[a:b].float().clone()
        for j in range(taps):
            acc += full[j:j + n] * wf[:, j][None, :]
        out[a:b] = acc
        if slot >= 0 and taps > 1:
            state[slot] = full[n:]
    return out.to(out_dtype)


def pool_slots_per_page(block_size: int, pool: int) -> int:
    """Pooled entries a page of block_size tokens can start."""
    return (block_size - 1) // pool + 1


def kv_write_pooled(k, v, k_cache, v_cache, kp_cache, vp_cache, slot_mapping,
                    positions, block_tables, token_seq, pool):
    """k [T,G,D], v [T,G,V] go to their pages; then every row whose position
    p ends a block of `pool` positions ((p + 1) % pool == 0) leaves the mean
    of that block's keys and values, read back from the pages (fp32 mean of
    what the cache holds), in the pooled caches kp/vp [pages, G, spp, D|V]:
    block b sits in the page of its first position p0 = b * pool, entry
    (p0 % block_size) // pool."""
    bs = k_cache.shape[2]
    ok = slot_mapping >= 0
    blk = (slot_mapping[ok] // bs).long()
    off = (slot_mapping[ok] % bs).long()
    k_cache[blk, :, off] = k[ok].to(k_cache.dtype)
    v_cache[blk, :, off] = v[ok].to(v_cache.dtype)
    pos = positions.tolist()
    seqs = token_seq.tolist()
    okl = ok.tolist()
    for t, p in enumerate(pos):
        if not okl[t] or (p + 1) % pool:
            continue
        bt = block_tables[seqs[t]]
        p0 = p + 1 - pool
        idx = torch.arange(p0, p + 1)
        pages = bt[(idx // bs).long()].long()
        offs = (idx % bs).long()
        km = k_cache[pages, :, offs].float().mean(0)  # [G, D]
        vm = v_cache[pages, :, offs].float().mean(0)
        page = int(bt[p0 // bs])
        e = (p0 % bs) // pool
        kp_cache[page, :, e] = km.to(kp_cache.dtype)
        vp_cache[page, :, e] = vm.to(vp_cache.dtype)


def attention_window_pool(q, k_cache, v_cache, kp_cache, vp_cache,
                          block_tables, seq_lens, cu_seqlens, scale, window,
                          pool, out=None, out_scale=1.0):
    """Softmax attention of packed new rows: the row at position i sees the
    keys j with 0 <= i - j < window and, in the same softmax, the pooled
    entry of every block b with b * pool + pool - 1 <= i - window.
    q [T,H,D] -> out [T,H,V] (q.dtype), times out_scale."""
    T, H, D = q.shape
    G, bs, V = v_cache.shape[1], v_cache.shape[2], v_cache.shape[3]
    res = torch.zeros(T, H, V, dtype=torch.float32)
    cu = cu_seqlens.tolist()
    sl = seq_lens.tolist()
    rep = H // G
    for s in range(len(sl)):
        a, b = cu[s], cu[s + 1]
        n, L = b - a, sl[s]
        if n == 0:
            continue
        nbk = (L + bs - 1) // bs
        pages = block_tables[s, :nbk].long()
        K = k_cache[pages].permute(1, 0, 2, 3).reshape(G, nbk * bs, D)[:, :L].float()
        Vv = v_cache[pages].permute(1, 0, 2, 3).reshape(G, nbk * bs, V)[:, :L].float()
        nblk_max = max(0, (L - 1 - window + 1) // pool)
        if nblk_max:
            p0 = torch.arange(nblk_max) * pool
            pp = block_tables[s][(p0 // bs).long()].long()
            pe = ((p0 % bs) // pool).long()
            KP = kp_cache[pp, :, pe].float().permute(1, 0, 2)  # [G, nb, D]
            VP = vp_cache[pp, :, pe].float().permute(1, 0, 2)
        for r in range(n):
            i = L - n + r
            lo = max(0, i - window + 1)
            nb = (i - window + 1) // pool if i - window + 1 > 0 else 0
            kk = K[:, lo:i + 1]
            vv = Vv[:, lo:i + 1]
            if nb:
                kk = torch.cat([KP[:, :nb], kk], 1)
                vv = torch.cat([VP[:, :nb], vv], 1)
            kk = kk.repeat_interleave(rep, 0)  # [H, m, D]
            vv = vv.repeat_interleave(rep, 0)
            sc = torch.einsum("hmd,hd->hm", kk, q[a + r].float()) * scale
            p = torch.softmax(sc, -1)
            res[a + r] = torch.einsum("hm,hmv->hv", p, vv)
    res = res * out_scale
    if out is not None:
        out.copy_(res.to(out.dtype))
        return out
    return res.to(q.dtype)


def retention_scan(q, k, v, decay, state, cu_seqlens, seq_lens, state_slots,
                   positions, inv_freq, interleaved, k_scale):
    """Linear attention with a fixed decay per head on plain (not
    activated) rows: q and k are turned by their position over their first
    2*len(inv_freq) dims, k is then multiplied by k_scale;
    S <- decay*S + k v^T, o = S^T q. -> o fp32 [T,H,V]; state updated."""
    T, H, D = q.shape
    V = v.shape[-1]
    qf, kf, vf = q.float(), k.float(), v.float()
    if inv_freq is not None and inv_freq.numel():
        rd = 2 * inv_freq.numel()
        ang = positions.float()[:, None, None] * inv_freq.float()[None, None, :]
        qf = torch.cat([_rotate_pairs(qf[..., :rd], ang, interleaved), qf[..., rd:]], -1)
        kf = torch.cat([_rotate_pairs(kf[..., :rd], ang, interleaved), kf[..., rd:]], -1)
    kf = kf * k_scale
    out = torch.zeros(T, H, V, dtype=torch.float32)
    lam = decay.float()[:, None, None]
    for a, b, start, slot in _seq_spans(cu_seqlens, seq_lens, state_slots):
        S = (state[slot].clone() if start > 0 and slot >= 0
             else torch.zeros(H, D, V))
        for t in range(a, b):
            S = lam * S + kf[t][:, :, None] * vf[t][:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        if slot >= 0:
            state[slot] = S
    return out


def head_norm_gate(o, gate, eps, heads, out, out_scale=1.0):
    """Each head's slice of o [T, heads*V] (fp32) scaled to unit RMS
    (o * rsqrt(mean(o^2) + eps), no weight), times silu(gate), times
    out_scale, into out [T, heads*V] (may be a column slice)."""
    T = o.shape[0]
    of = o.float().view(T, heads, -1)
    y = of * torch.rsqrt(of.pow(2).mean(-1, keepdim=True) + eps)
    g = gate.float()
    out.copy_((y.reshape(T, -1) * g * torch.sigmoid(g) * out_scale).to(out.dtype))
    return out


def glu_act(gu, kind, limit=0.0, alpha=1.0, row_scale=None):
    """gu [T, 2F] = [gate | up] -> [T, F]; row_scale [T] fp32 multiplies a
    row's gate and up first (the projections of a scaled input).
    "swiglu": silu(gate) * up.
    "clamped": g = min(gate, limit), u = clamp(up, -limit, limit),
               g * sigmoid(alpha g) * (u + 1).
    "gelu_tanh": gelu_tanh(gate) * up."""
    F_ = gu.shape[-1] // 2
    g, u = gu[..., :F_].float(), gu[..., F_:].float()
    if row_scale is not None:
        g, u = g * row_scale.float()[:, None], u * row_scale.float()[:, None]
    if kind == "swiglu":
        return (g * torch.sigmoid(g) * u).to(gu.dtype)
    if kind == "gelu_tanh":
        return (torch.nn.functional.gelu(g, approximate="tanh") * u).to(gu.dtype)
    g = g.clamp(max=limit)
    u = u.clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)


def moe_route_grouped(logits, top, groups, keep, score="softmax",
                      renorm=True):
    """Scores over all experts: their softmax, or (score="sigmoid") each
    logit's own sigmoid; without renorm the chosen scores are the weights as
    they are. Experts are cut into `groups`
    contiguous runs of E/groups, a run's score is its highest expert score
    and only the `keep` highest-scoring runs stay eligible; the `top` largest scores among those, their
    scores divided by their sum (+1e-20). Ties go to the lower index.
    logits [T, E] fp32 -> (weights [T, top] fp32, ids [T, top] int32)."""
    s = (torch.sigmoid(logits.float()) if score == "sigmoid"
         else torch.softmax(logits.float(), -1))
    T, E = s.shape
    per = E // groups
    gs = s.view(T, groups, per).amax(-1)
    kept = torch.topk(gs, keep, dim=-1).indices  # [T, keep]
    allow = torch.zeros(T, groups, dtype=torch.bool)
    allow.scatter_(1, kept, True)
    masked = torch.where(allow[:, :, None].expand(T, groups, per).reshape(T, E),
                         s, torch.full_like(s, -1.0))
    ids = torch.topk(masked, top, dim=-1).indices
    w = s.gather(1, ids)
    if renorm:
        w = w / (w.sum(-1, keepdim=True) + 1e-20)
    return w, ids.to(torch.int32)


# ----------------------------------------------------------------------
# Shared-norm parallel blocks with a tanh norm, latent attention, mamba2.
# ----------------------------------------------------------------------
def residual_tanh_norm(x, y, mult, alpha, weight, bias, out_dtype, xa=None):
    """x (fp32, in place) += mult * y when y is given; xa (a [T, C] view,
    any row stride) takes the new x in its own dtype; returns
    tanh(alpha x) * weight + bias in out_dtype (None without a weight)."""
    if y is not None:
        x += mult * y.float()
    if xa is not None:
        xa.copy_(x)
    if weight is None:
        return None
    return (torch.tanh(alpha.float() * x) * weight.float()
            + bias.float()).to(out_dtype)


def latent_prepare(cq, ckv, q_norm_w, kv_norm_w, eps, positions, inv_freq,
                   cache, slot_mapping):
    """Row work of latent attention before its up-projections. cq [T, Rq]:
    RMS norm times q_norm_w, returned in cq.dtype. ckv [T, Rk + 2P]: the
    first Rk columns RMS-normed times kv_norm_w, the last 2P (P =
    len(inv_freq)) turned by the row's position in interleaved pairs; the
    row goes to its place in cache [blocks, 1, bs, Rk + 2P]."""
    def unit(t):
        return t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps)

    cqn = (unit(cq.float()) * q_norm_w.float()).to(cq.dtype)
    rank = kv_norm_w.shape[0]
    f = ckv.float()
    c = unit(f[:, :rank]) * kv_norm_w.float()
    ang = positions.float()[:, None] * inv_freq.float()[None, :]
    kr = _rotate_pairs(f[:, rank:], ang, True)
    row = torch.cat([c, kr], -1).to(cache.dtype)
    bs = cache.shape[2]
    ok = slot_mapping >= 0
    cache[(slot_mapping[ok] // bs).long(), 0, (slot_mapping[ok] % bs).long()] = row[ok]
    return cqn


def latent_query(q, q_abs, positions, inv_freq, out):
    """out [T, H, Rk + 2P] = [q_abs (given as [H, T, Rk]) | the last 2P
    dims of q [T, H, D + 2P] turned by the row's position, interleaved].
    q_abs None: the first part is q's own first D dims."""
    D = q.shape[2] - 2 * inv_freq.numel()
    rank = q_abs.shape[2] if q_abs is not None else D
    ang = positions.float()[:, None, None] * inv_freq.float()[None, None, :]
    out[..., :rank] = q_abs.transpose(0, 1) if q_abs is not None else q[..., :D]
    out[..., rank:] = _rotate_pairs(q[..., D:].float(), ang, True).to(out.dtype)
    return out


def mamba2_scan(xbc, dt_raw, dt_bias, rate, Dp, state, cu_seqlens, seq_lens,
                state_slots, heads, vdim, nstate, groups):
    """Scalar-decay state-space recurrence per head: xbc [T, P*V + 2*G*N] =
    [x | B | C] (after conv and silu), dt = softplus(dt_raw + dt_bias) [T, P];
    S_h (N x V) <- exp(-rate_h dt) S_h + dt B_g x_h^T,
    y_h = S_h^T C_g + D_h x_h with g = h // (P / G). state
    [slots, P, N, V] fp32 (updated). Returns y fp32 [T, P*V]."""
    T = xbc.shape[0]
    P, V, N, G = heads, vdim, nstate, groups
    f = xbc.float()
    x = f[:, :P * V].reshape(T, P, V)
    Bm = f[:, P * V:P * V + G * N].reshape(T, G, N).repeat_interleave(P // G, 1)
    Cm = f[:, P * V + G * N:].reshape(T, G, N).repeat_interleave(P // G, 1)
    dt = torch.nn.functional.softplus(dt_raw.float() + dt_bias.float(),
                                      threshold=20.0)
    a = torch.exp(-rate.float()[None, :] * dt)  # [T, P]
    out = torch.empty(T, P, V, dtype=torch.float32)
    for lo, hi, start, slot in _seq_spans(cu_seqlens, seq_lens, state_slots):
        S = (state[slot].clone() if start > 0 and slot >= 0
             else torch.zeros(P, N, V))
        for t in range(lo, hi):
            S = a[t][:, None, None] * S + \
                (dt[t][:, None] * Bm[t])[:, :, None] * x[t][:, None, :]
            out[t] = torch.einsum("pnv,pn->pv", S, Cm[t]) \
                + Dp.float()[:, None] * x[t]
        if slot >= 0:
            state[slot] = S
    return out.reshape(T, P * V)


def gate_group_norm(y, z, weight, groups, eps, out, out_scale=1.0):
    """out = unit_rms_per_group(y * silu(z)) * weight * out_scale: the row
    is cut into `groups` equal parts, each divided by its own root mean
    square. y fp32 [T, C]; z, out [T, C] views."""
    T, C = y.shape
    g = y.float() * torch.nn.functional.silu(z.float())
    g = g.view(T, groups, C // groups)
    g = g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps)
    out.copy_((g.reshape(T, C) * weight.float() * out_scale).to(out.dtype))
    return out


# ----------------------------------------------------------------------
# Two-norm parallel blocks with per-channel branch scales, difference
# attention behind short convolutions, input-scaled experts.
# ----------------------------------------------------------------------
def residual_pair_norm(x, y1, s1, y2, s2, w1, w2, eps, out_dtype):
    """x (fp32, in place) += s1 * y1 + s2 * y2 (each when given; s per
    channel); returns (h1, h2) = x / sqrt(mean(x^2) + eps) * (1 + w) for
    each weight given (None otherwise), in out_dtype."""
    if y1 is not None:
        add = y1.float() * s1.float()
        if y2 is not None:
            add = add + y2.float() * s2.float()
        x += add
    elif y2 is not None:
        x += y2.float() * s2.float()
    if w1 is None and w2 is None:
        return None, None
    n = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return tuple((n * (1.0 + w.float())).to(out_dtype) if w is not None
                 else None for w in (w1, w2))


def query_map_order(c, heads, kv_heads, maps, dim):
    """Where channel c of a query row laid out [head, map, dim] goes in the
    order [kv head, map, head of the group, dim] the attention ops read."""
    d = c % dim
    m = (c // dim) % maps
    h = c // (dim * maps)
    r = heads // kv_heads
    return (((h // r) * maps + m) * r + h % r) * dim + d


def conv_qkv_cache(p, n_q, n_k, n_v, weight, state, cu_seqlens, seq_lens,
                   state_slots, positions, temp_coef, temp_every, heads,
                   kv_heads, maps, k_cache, v_cache, slot_mapping):
    """Causal depthwise convolution over time of the first n_q + n_k + n_v
    channels of p [T, >=C] (weight [C, taps], last column = current row, no
    bias, no activation; state [slots, taps-1, C] fp32 holds each sequence's
    last taps-1 inputs and is updated). The q channels are multiplied by
    1 + temp_coef ln(floor((pos + 1) / temp_every) + 1) (temp_every 0: by 1)
    and returned [T, n_q] in the head order of query_map_order; the k and v
    channels go to their pages (k_cache [pages, G, bs, n_k / G])."""
    T = p.shape[0]
    C = n_q + n_k + n_v
    taps = weight.shape[1]
    xf = p[:, :C].float()
    y = torch.empty(T, C, dtype=torch.float32)
    wf = weight.float()
    for a, b, start, slot in _seq_spans(cu_seqlens, seq_lens, state_slots):
        hist = (state[slot].clone() if start > 0 and slot >= 0 and taps > 1
                else torch.zeros(taps - 1, C))
        full = torch.cat([hist, xf[a:b]], 0)
        n = b - a
        acc = torch.zeros(n, C)
        for j in range(taps):
            acc += full[j:j + n] * wf[:, j][None, :]
        y[a:b] = acc
        if slot >= 0 and taps > 1:
            state[slot] = full[n:]
    q = y[:, :n_q]
    if temp_every > 0:
        pos = positions.float()
        q = q * (1.0 + temp_coef * torch.log(
            torch.floor((pos + 1.0) / temp_every) + 1.0))[:, None]
    dim = n_q // (heads * maps)
    order = query_map_order(torch.arange(n_q), heads, kv_heads, maps, dim)
    qo = torch.empty(T, n_q, dtype=p.dtype)
    qo[:, order] = q.to(p.dtype)
    if n_k:
        G, bs = k_cache.shape[1], k_cache.shape[2]
        ok = slot_mapping >= 0
        blk = (slot_mapping[ok] // bs).long()
        off = (slot_mapping[ok] % bs).long()
        k_cache[blk, :, off] = y[ok, n_q:n_q + n_k].view(-1, G, n_k // G).to(k_cache.dtype)
        v_cache[blk, :, off] = y[ok, n_q + n_k:].view(-1, G, n_v // G).to(v_cache.dtype)
    return qo


def diff_head_norm_gate(a, gate, lam, eps, mult, heads, kv_heads, out):
    """a [T, kv_heads, 2, heads / kv_heads, V]: the two maps' outputs of
    every head. o = a[:, :, 0] - lam * a[:, :, 1], divided by its root mean
    square over V, times mult, times sigmoid(gate) (gate [T, heads * V] in
    the plain head order), into out [T, heads * V] (views, any row
    stride)."""
    T = a.shape[0]
    V = a.shape[-1]
    af = a.float().view(T, kv_heads, 2, heads // kv_heads, V)
    o = (af[:, :, 0] - lam * af[:, :, 1]).reshape(T, heads, V)
    o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * mult
    out.copy_((o.reshape(T, heads * V) * torch.sigmoid(gate.float())).to(out.dtype))
    return out


def moe_glu_scaled(gu, scale, experts, ff, shared_ff):
    """gu [T, experts * 2 ff + 2 shared_ff]: per expert [gate | up], then
    the shared expert's [gate | up]. Column c of expert e becomes
    silu(s g) * (s u) with s = scale[t, e] (fp32; 0 for an expert the row
    does not use), the shared columns silu(g) * u. -> [T, experts * ff +
    shared_ff]."""
    T = gu.shape[0]
    ex = gu[:, :experts * 2 * ff].float().view(T, experts, 2, ff)
    s = scale.float()[:, :, None]
    g, u = ex[:, :, 0] * s, ex[:, :, 1] * s
    parts = [(g * torch.sigmoid(g) * u).reshape(T, experts * ff)]
    if shared_ff:
        sh = gu[:, experts * 2 * ff:].float()
        g, u = sh[:, :shared_ff], sh[:, shared_ff:]
        parts.append(g * torch.sigmoid(g) * u)
    return torch.cat(parts, -1).to(gu.dtype)


def route_scale_matrix(weights, ids, experts):
    """[T, experts] fp32: a row's weight at each expert it uses, 0 elsewhere."""
    out = torch.zeros(weights.shape[0], experts, dtype=torch.float32)
    out.scatter_(1, ids.long(), weights.float())
    return out
