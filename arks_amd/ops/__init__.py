"""Op dispatch for arks_amd.

On GPU tensors every op runs the in-tree gfx950 HIP extension
(``arks_amd._C``) — there is no eager fallback: if the extension is missing
on a CUDA/ROCm device we raise immediately so a silently-slow PyTorch path
can never masquerade as the native one. On CPU tensors ops run the plain
PyTorch reference (arks_amd/ops/ref.py) so the engine/scheduler/model layers
are unit-testable without a GPU.
"""

from __future__ import annotations

import os

import torch

from . import ref

_C = None
_C_ERR: str | None = None


def _load_extension():
    global _C, _C_ERR
    if _C is not None or _C_ERR is not None:
        return _C
    try:
        from . import _load

        _C = _load.load("arks_amd_C")  # the built .so in-tree
    except Exception as e:  # pragma: no cover - exercised only when unbuilt
        _C_ERR = f"{type(e).__name__}: {e}"
    return _C


def native_available() -> bool:
    return _load_extension() is not None


def _native():
    c = _load_extension()
    if c is None:
        raise RuntimeError(
            "arks_amd HIP extension (arks_amd._C) is not built but a GPU op was "
            "requested. Build it with `python -m arks_amd.ops.build` "
            f"(import error: {_C_ERR})"
        )
    return c


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    if x.is_cuda:
        out = torch.empty_like(x)
        _native().rmsnorm(out, x, weight, eps)
        return out
    return ref.rmsnorm(x, weight, eps)


def fused_add_rmsnorm(x, residual, weight, eps: float = 1e-6):
    """In-place on GPU: residual += x (written to residual), out = norm(residual)."""
    if x.is_cuda:
        out = torch.empty_like(x)
        _native().fused_add_rmsnorm(out, x, residual, weight, eps)
        return out, residual
    return ref.fused_add_rmsnorm(x, residual, weight, eps)


def silu_mul(gate_up: torch.Tensor) -> torch.Tensor:
    if gate_up.is_cuda:
        shape = list(gate_up.shape)
        shape[-1] //= 2
        out = gate_up.new_empty(shape)
        _native().silu_mul(out, gate_up)
        return out
    return ref.silu_mul(gate_up)


def rope_apply_inplace(positions, q, k, cos_sin, head_dim: int):
    """Rotates q and k in place (GPU). CPU path returns new tensors."""
    if q.is_cuda:
        _native().rope_inplace(positions, q, k, cos_sin, head_dim)
        return q, k
    return ref.rope_apply(positions, q, k, cos_sin, head_dim)


def rope_and_cache(positions, q, k, v, k_cache, v_cache, slot_mapping,
                   cos_sin, head_dim: int):
    """Fused RoPE + paged-cache write (GPU): rotates q/k in place and
    scatters rotated k + v into the cache in one launch. CPU path runs the
    two reference steps."""
    if q.is_cuda:
        _native().rope_and_cache(positions, q, k, v, k_cache, v_cache,
                                 slot_mapping, cos_sin, head_dim)
        return q, k
    q2, k2 = ref.rope_apply(positions, q, k, cos_sin, head_dim)
    T = q.shape[0]
    nkv = k.numel() // max(T, 1) // head_dim
    ref.reshape_and_cache(
        k2.reshape(T, nkv, head_dim), v.reshape(T, nkv, head_dim),
        k_cache, v_cache, slot_mapping,
    )
    return q2, k2


def reshape_and_cache(k, v, k_cache, v_cache, slot_mapping):
    if k.is_cuda:
        _native().reshape_and_cache(k, v, k_cache, v_cache, slot_mapping)
        return
    ref.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping)


PREFILL_QTILE = 64  # q rows per workgroup in the prefill kernel


def build_prefill_tiles(seq_lens: list[int], device) -> torch.Tensor:
    """int32 [ntiles, 2] of (seq_idx, q0) covering every sequence in 64-row
    tiles — the prefill kernel's grid."""
    tiles = []
    for i, n in enumerate(seq_lens):
        for q0 in range(0, n, PREFILL_QTILE):
            tiles.append((i, q0))
    return torch.tensor(tiles, dtype=torch.int32, device=device).reshape(-1, 2)


def attention_prefill_varlen(q, k, v, cu_seqlens, seq_lens: list[int],
                             scale: float, window: int = 0):
    """Causal varlen prefill attention. seq_lens is the host-side list of
    per-sequence lengths (used to build the q-tile grid without a D2H sync).
    window > 0 = sliding-window attention."""
    if q.is_cuda:
        out = torch.empty_like(q)
        tile_info = build_prefill_tiles(seq_lens, q.device)
        _native().attention_prefill_varlen(out, q, k, v, cu_seqlens, tile_info,
                                           scale, window)
        return out
    return ref.attention_prefill_varlen(q, k, v, cu_seqlens, scale, window)


EXTEND2_QTILE = 256  # q rows per workgroup in the 8-wave ladder kernel
E2_KVBLK = 64        # keys per LDS tile in the ladder kernel
# Sequences with at least this many new q tokens go to the 256-row ladder
# kernel; shorter ones (decode-adjacent chunks, prefix-cache hits) stay on
# the 64-row kernel where a mostly-empty 256-row tile would waste waves.
EXTEND2_MIN_QLEN = 97


def build_extend_tiles(q_lens: list[int], kv_lens: list[int] | None,
                       kv_fp8: bool, device, num_q_heads: int = 32,
                       ladder: bool = True, flash_decode: bool = True):
    """Per-seq routing for the extend dispatcher:
    (tiles64, tiles256 [n,4], decode_rows, combine_table, ws_rows).

    q_len == 1 sequences (decode steps mixed into a prefill batch) go to
    the flash-decode kernel — an extend q-tile for one query scans the
    full KV with 255 masked rows (~6x slower than the decode kernel's
    partitioned scan). Remaining sequences split between the 64-row and
    256-row extend kernels; tiles are sorted by DESCENDING key depth
    (causal q-tiles differ up to 4x in KV work and the dispatcher issues
    blocks in order — deep tiles first removes the straggler tail). When
    the batch is too small to fill the chip, deep 256-row tiles are
    additionally SPLIT over their KV range flash-decode-style (part rows
    + a combine pass over f32 partials); split parts sort first so the
    partial workspace only covers them. Build once per batch and reuse
    across all layers."""
    t64, t256, dec = [], [], []
    kvl = kv_lens if kv_lens is not None else q_lens
    for i, n in enumerate(q_lens):
        off = kvl[i] - n
        if n == 1 and flash_decode:
            dec.append(i)
        elif kv_fp8 or n < EXTEND2_MIN_QLEN or not ladder:
            for q0 in range(0, n, PREFILL_QTILE):
                t64.append((i, q0, min(kvl[i], off + q0 + PREFILL_QTILE)))
        else:
            for q0 in range(0, n, EXTEND2_QTILE):
                t256.append((i, q0, min(kvl[i], off + q0 + EXTEND2_QTILE)))
    t64.sort(key=lambda t: -t[2])
    t256.sort(key=lambda t: -t[2])
    mk64 = lambda t: torch.tensor(
        [x[:2] for x in t], dtype=torch.int32, device=device
    ).reshape(-1, 2)

    # KV-split policy for the 256-row kernel: when tiles x heads cannot
    # fill ~2 workgroups per CU, split the deepest tiles' key ranges.
    base_wgs = len(t256) * max(num_q_heads, 1)
    factor = 1
    if t256 and base_wgs < 256:
        # truly starved launches only (256 CUs, 1 block/CU kernel): the
        # partial slabs + combine cost ~2x slab traffic, so marginal
        # shortfalls are better left unsplit
        factor = min(8, -(-512 // base_wgs))
    rows, combine = [], []
    ws_rows = 0
    if factor > 1:
        split, plain = [], []
        for (i, q0, kmax) in t256:
            span = (kmax + E2_KVBLK - 1) // E2_KVBLK
            p = min(factor, max(1, span // 4))
            (split if p > 1 else plain).append((i, q0, p))
        # cap the f32 partial workspace at ~512 MB
        slab = num_q_heads * EXTEND2_QTILE * 130 * 4
        if sum(p for _, _, p in split) * slab > 512 * 1024 * 1024:
            split, plain = [], split + plain
        for (i, q0, p) in split:
            combine.append((len(rows), p, i, q0))
            for part in range(p):
                rows.append((i, q0, part, p))
        ws_rows = len(rows)
        for (i, q0, p) in plain:
            rows.append((i, q0, 0, 1))
    else:
        rows = [(i, q0, 0, 1) for (i, q0, _) in t256]
    t256_t = torch.tensor(rows, dtype=torch.int32,
                          device=device).reshape(-1, 4)
    ctab = torch.tensor(combine, dtype=torch.int32,
                        device=device).reshape(-1, 4)

    if dec:
        # gather indices: the single q row of each decode seq sits at
        # cu_seqlens_q[i]; seq-level metadata indexes with `dec` itself
        cu = [0]
        for n in q_lens:
            cu.append(cu[-1] + n)
        drows = torch.tensor([cu[i] for i in dec], dtype=torch.long,
                             device=device)
        dseqs = torch.tensor(dec, dtype=torch.long, device=device)
    else:
        drows = dseqs = None
    return mk64(t64), t256_t, (drows, dseqs), ctab, ws_rows


def attention_extend_paged(
    q, k_cache, v_cache, block_tables, kv_lens, cu_seqlens_q,
    q_lens: list[int], scale: float, window: int = 0, tiles=None,
    sink: bool = False, native=None, maps: int = 1,
):
    """Causal attention of packed NEW tokens over each sequence's full paged
    KV history (cached prefix + new tokens already written by
    reshape_and_cache). The prefix-caching / chunked-prefill attention path.
    q_lens is the host-side per-seq new-token count (tile grid without a
    D2H sync); kv_lens is the device int32 total kv length per seq.
    window > 0 = sliding-window attention. sink: every softmax also holds a
    value-less key of score 0. native: the extension whose build of these
    kernels runs (default: arks_amd_C). maps M > 1: a key row of the cache
    holds M keys side by side that share the row's value (k_cache [pages, G,
    16, M*D]); q has G*M groups of heads, group g*M + m reads key m of head
    g (tiles built without the flash-decode rows).

    Dispatch: big chunks run the 8-wave 32x32-MFMA ladder kernel
    (attn_extend2.hip, 256-row q tiles); small chunks and fp8-KV runs use
    the 4-wave 64-row kernel."""
    if q.is_cuda:
        C = native if native is not None else _native()
        sink = 1 if sink else 0
        out = torch.empty(
            (q.shape[0], q.shape[1], q.shape[2]), dtype=q.dtype, device=q.device
        )
        kv_fp8 = k_cache.dtype != torch.bfloat16
        t64, t256, (drows, dseqs), ctab, ws_rows = (
            tiles if tiles is not None
            else build_extend_tiles(q_lens, None, kv_fp8, q.device,
                                    num_q_heads=q.shape[1])
        )
        if t256.numel():
            if ws_rows:
                ws = _extend_ws(
                    ws_rows * q.shape[1] * EXTEND2_QTILE * (q.shape[2] + 2),
                    q.device,
                )
            else:
                ws = q.new_empty(0, dtype=torch.float32)
            C.attention_extend_paged2(
                out, q, k_cache, v_cache, block_tables, kv_lens, cu_seqlens_q,
                t256, ws, scale, window, sink, maps,
            )
            if ctab.numel():
                C.attention_extend2_combine(
                    out, ws, ctab, cu_seqlens_q, scale,
                )
        if t64.numel():
            C.attention_extend_paged(
                out, q, k_cache, v_cache, block_tables, kv_lens, cu_seqlens_q,
                t64, scale, window, sink, maps,
            )
        if drows is not None:
            assert maps == 1, "single rows of a two-map cache: no flash-decode"
            dq = q[drows].contiguous()
            dout = attention_decode_paged(
                dq, k_cache, v_cache,
                block_tables[dseqs].contiguous(),
                kv_lens[dseqs].contiguous(), scale, window=window,
                sink=bool(sink), native=C,
            )
            out[drows] = dout
        return out
    return ref.attention_extend_paged(
        q, k_cache, v_cache, block_tables, kv_lens, cu_seqlens_q, scale,
        window,
    )


def decode_num_partitions(num_seqs: int, num_kv_heads: int, max_blocks: int) -> int:
    """Flash-decode split factor: fill the 256 CUs (target ~2 workgroups/CU)
    when batch x kv_heads alone cannot. Each partition keeps >= 8 pages so
    all 4 waves of a workgroup get a 2-page chunk and the K-prefetch
    software pipeline has depth (bench_decode2: starved waves at <8
    pages/partition cap short-seq shapes)."""
    base = num_seqs * num_kv_heads
    target = 512
    nparts = max(1, -(-target // base))
    nparts = min(nparts, max(1, max_blocks // 8), 64)
    return nparts


def attention_decode_paged(
    q, k_cache, v_cache, block_tables, seq_lens, scale: float,
    num_partitions: int | None = None, part_out=None, window: int = 0,
    sink: bool = False, native=None,
):
    if q.is_cuda:
        C = native if native is not None else _native()
        out = torch.empty(
            (q.shape[0], q.shape[1], q.shape[2]), dtype=q.dtype, device=q.device
        )
        num_kv_heads = k_cache.shape[1]
        if num_partitions is None:
            num_partitions = decode_num_partitions(
                q.shape[0], num_kv_heads, block_tables.shape[1]
            )
        if num_partitions > 1 and part_out is None:
            gq = q.shape[1] // num_kv_heads
            part_out = torch.empty(
                q.shape[0] * num_kv_heads * num_partitions * gq * (q.shape[2] + 2),
                dtype=torch.float32, device=q.device,
            )
        elif part_out is None:
            part_out = q.new_empty(0, dtype=torch.float32)
        C.attention_decode_paged(
            out, q, k_cache, v_cache, block_tables, seq_lens, scale,
            part_out, num_partitions, window, 1 if sink else 0,
        )
        return out
    return ref.attention_decode_paged(
        q, k_cache, v_cache, block_tables, seq_lens, scale, window
    )


_EXTEND_WS: dict = {}


def _extend_ws(need: int, device):
    key = (device.index,)
    ws = _EXTEND_WS.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(need, dtype=torch.float32, device=device)
        _EXTEND_WS[key] = ws
    return ws


_SKINNY_WS: dict = {}


def skinny_gemm(x, weight, bias=None):
    """C = x @ weight^T for decode-sized M (<=64) via the split-K streaming
    MFMA kernel. Beats hipBLASLt's ~19 us latency floor on the small
    qkv/o_proj shapes and its ~46 us in-graph down-proj algo (bench_skinny /
    bench_down logs, r2); the dispatcher keeps the wide streaming shapes
    (gate_up, lm_head: N >> K) on the tuned library algos. Deterministic
    split-K (fixed-order combine, no atomics)."""
    M, K = x.shape
    N = weight.shape[0]
    out = torch.empty((M, N), dtype=x.dtype, device=x.device)
    ntiles = N // 64
    if K > N and ntiles < 128 and M > 48:
        # tall-K (down-proj shape): few N tiles, parallelism comes from
        # K-splits; the deeper-staged AB=3 variant at nsplits ~= 448/ntiles
        # measured fastest (34.6 us vs hipBLASLt's 46.4 in-graph, r2).
        # M-gated: the variant kernel is fixed at MT=4 (full 64-row cost)
        # while hipBLASLt switches to a faster algo below M~48 — routing
        # small-M down-proj here regressed b16x8k decode by 4% (r2)
        nsplits = min(-(-448 // ntiles), -(-K // 256))
        k_per_split = -(-(-(-K // nsplits)) // 32) * 32
        nsplits = -(-K // k_per_split)
        part = (_skinny_ws(nsplits, N, 64, x.device) if nsplits > 1
                else x.new_empty(0, dtype=torch.float32))
        _native().skinny_gemm_v(out, part, x, weight, bias, k_per_split,
                                nsplits, _SKINNY_TALLK_VARIANT, False)
        return out
    if ntiles >= 384:
        nsplits = 1
    else:
        nsplits = min(-(-512 // ntiles), -(-K // 256))
    k_ceil = -(-K // nsplits)
    k_per_split = -(-k_ceil // 32) * 32
    nsplits = -(-K // k_per_split)
    part = _skinny_ws(nsplits, N, M, x.device) if nsplits > 1 else x.new_empty(
        0, dtype=torch.float32
    )
    _native().skinny_gemm(out, part, x, weight, bias, k_per_split, nsplits)
    return out


def _skinny_ws(nsplits: int, N: int, M: int, device):
    mrows = ((M + 15) // 16) * 16
    key = (device.index,)
    need = nsplits * N * mrows
    ws = _SKINNY_WS.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(need, dtype=torch.float32, device=device)
        _SKINNY_WS[key] = ws
    return ws


_USE_SKINNY = os.environ.get("ARKS_SKINNY_GEMM", "1") == "1"
# Weight-elements threshold: the split-K streaming kernel beats hipBLASLt's
# ~19 us latency floor on the small decode shapes (qkv/o: 1.0-1.6x,
# bench_skinny v3); the big streaming shapes (gate_up/down/lm_head) stay on
# the tuned hipBLASLt algos which reach 5.4-6.4 TB/s there.
_SKINNY_MAX_ELEMS = 34_000_000
# tall-K decode shapes (down-proj: K > N) stream W near-HBM-rate through the
# split-K kernel and beat the library's in-graph algo (r2); wide-N shapes
# (gate_up/lm_head) stay on hipBLASLt which reaches ~6 TB/s there.
_SKINNY_TALLK_MAX_ELEMS = 80_000_000
# 7 = AB=3 deep-staged; 8 = same + non-temporal W loads
_SKINNY_TALLK_VARIANT = int(os.environ.get("ARKS_SKINNY_TALLK_V", "7"))


def linear_bf16(x, weight, bias=None):
    """Linear dispatch: the skinny split-K kernel for small decode-shaped
    GEMMs on GPU, hipBLASLt (F.linear) otherwise."""
    if (
        _USE_SKINNY
        and x.is_cuda
        and x.dim() == 2
        and 1 <= x.shape[0] <= 64
        and x.dtype == torch.bfloat16
        and weight.shape[0] % 64 == 0
        and weight.shape[1] % 32 == 0
        and (weight.numel() <= _SKINNY_MAX_ELEMS
             or (weight.shape[1] > weight.shape[0]
                 and x.shape[0] > 48
                 and weight.numel() <= _SKINNY_TALLK_MAX_ELEMS))
        and weight.is_contiguous()
        and native_available()
    ):
        return skinny_gemm(x, weight, bias)
    import torch.nn.functional as F

    return F.linear(x, weight, bias)


def rmsnorm_fp8(x, weight, eps: float = 1e-6):
    """Fused RMSNorm -> per-token fp8 e4m3: (out8, inv_scale). GPU-only
    fast path (hidden <= 8192); otherwise compose the unfused ops."""
    if x.is_cuda and x.shape[-1] <= 8192:
        out = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
        inv_scale = torch.empty(x.shape[0], dtype=torch.float32, device=x.device)
        _native().rmsnorm_fp8(out, inv_scale, x, None, weight, eps)
        return out, inv_scale
    return quant_fp8_rows(rmsnorm(x, weight, eps))


def fused_add_rmsnorm_fp8(x, residual, weight, eps: float = 1e-6):
    """Fused residual-add + RMSNorm -> fp8: (out8, inv_scale, residual)."""
    if x.is_cuda and x.shape[-1] <= 8192:
        out = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
        inv_scale = torch.empty(x.shape[0], dtype=torch.float32, device=x.device)
        _native().rmsnorm_fp8(out, inv_scale, x, residual, weight, eps)
        return out, inv_scale, residual
    y, res = fused_add_rmsnorm(x, residual, weight, eps)
    q, s = quant_fp8_rows(y)
    return q, s, res


def silu_mul_fp8(gate_up):
    """Fused SwiGLU -> per-token fp8: (out8, inv_scale)."""
    d = gate_up.shape[-1] // 2
    # dynamic-LDS default cap is 64 KiB; stay under it (d*2 bytes staged)
    if gate_up.is_cuda and d % 8 == 0 and d * 2 <= 60 * 1024:
        out = torch.empty((gate_up.shape[0], d), dtype=torch.float8_e4m3fn,
                          device=gate_up.device)
        inv_scale = torch.empty(gate_up.shape[0], dtype=torch.float32,
                                device=gate_up.device)
        _native().silu_mul_fp8(out, inv_scale, gate_up.contiguous())
        return out, inv_scale
    return quant_fp8_rows(silu_mul(gate_up))


def quant_fp8_rows(x):
    """Dynamic per-token fp8 e4m3 quantization: [M, K] bf16 ->
    ([M, K] float8_e4m3fn, [M] fp32 dequant scales) for W8A8 GEMMs
    (torch._scaled_mm rowwise)."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
        inv_scale = torch.empty(x.shape[0], dtype=torch.float32, device=x.device)
        _native().quant_fp8_rows(out, inv_scale, x.contiguous())
        return out, inv_scale
    return ref.quant_fp8_rows(x)


def moe_topk(router_logits, k: int, renorm: bool):
    """softmax + top-k + optional renorm in one kernel:
    (weights [T,k] f32, ids [T,k] i32). torch.topk tie-breaking (lower
    expert id wins)."""
    if router_logits.is_cuda:
        T = router_logits.shape[0]
        weights = torch.empty(T, k, dtype=torch.float32,
                              device=router_logits.device)
        ids = torch.empty(T, k, dtype=torch.int32,
                          device=router_logits.device)
        _native().moe_topk(weights, ids, router_logits.contiguous(), k,
                           1 if renorm else 0)
        return weights, ids
    return ref.moe_topk(router_logits, k, renorm)


def moe_mix(y, weights, ids, expert_base: int = 0):
    """out[t] = sum_i weights[t,i] * y[ids[t,i]-expert_base, t] with
    out-of-slice experts contributing 0 (TP expert parallelism)."""
    if y.is_cuda:
        El, T, H = y.shape
        out = torch.empty(T, H, dtype=y.dtype, device=y.device)
        _native().moe_mix(out, y.contiguous(), weights, ids, expert_base, El)
        return out
    return ref.moe_mix(y, weights, ids, expert_base)


def moe_mix_rows(y, weights, rows):
    """out[t] = sum_j weights[t,j] * y[rows[t,j]] — the gather-side mix
    over a flat per-pair expert-output buffer (zero-weight slots point at
    row 0)."""
    if y.is_cuda:
        T, k = weights.shape
        out = torch.empty(T, y.shape[1], dtype=y.dtype, device=y.device)
        _native().moe_mix_rows(out, y.contiguous(), weights, rows)
        return out
    return ref.moe_mix_rows(y, weights, rows)


def sample_tokens(logits, temperatures, uniform):
    """Gumbel-max categorical sampling; rows with temperature 0 are greedy."""
    if logits.is_cuda:
        out = torch.empty(logits.shape[0], dtype=torch.int64, device=logits.device)
        _native().gumbel_sample(out, logits, temperatures, uniform)
        return out
    return ref.gumbel_sample(logits, temperatures, uniform)


def greedy_sample(logits):
    if logits.is_cuda:
        out = torch.empty(logits.shape[0], dtype=torch.int64, device=logits.device)
        _native().greedy_sample(out, logits)
        return out
    return ref.greedy_sample(logits)


# ----------------------------------------------------------------------
# Sequence-state ops (arks_amd_seq_C): the kernels of the layer-list
# decoders — token shift, gated output norm into an fp32 residual, sink
# attention with rotated values, lightning linear attention, mamba1 conv
# and selective scan. Same dispatch rule as above: CUDA tensors run the HIP
# extension or fail loudly, CPU tensors run ops/ref.py.
# ----------------------------------------------------------------------
_S = None
_S_ERR: str | None = None


def _native_seq():
    global _S, _S_ERR
    if _S is None and _S_ERR is None:
        try:
            from . import _load

            _S = _load.load("arks_amd_seq_C")
        except Exception as e:
            _S_ERR = f"{type(e).__name__}: {e}"
    if _S is None:
        raise RuntimeError(
            "arks_amd sequence-state HIP extension (arks_amd_seq_C) is not "
            "built but a GPU op was requested. Build it with `python -m "
            f"arks_amd.ops.build arks_amd_seq_C` (import error: {_S_ERR})"
        )
    return _S


def seq_native_available() -> bool:
    try:
        _native_seq()
        return True
    except RuntimeError:
        return False


def ensure_built(name: str) -> None:
    """Compile one in-tree extension if its library is not there yet (a
    fresh checkout on a GPU box); a no-op once built."""
    global _S_ERR, _C_ERR
    from .build import build, built_so_path

    if built_so_path(name) is None:
        build(name=name)
        _S_ERR = _C_ERR = None


def token_shift(x, shift_w, prev_state, cu_seqlens, seq_lens, state_slots,
                token_seq, out_dtype):
    """(xs, xa): the shifted mixer input and the plain row, both cast to
    out_dtype; prev_state takes each sequence's last row."""
    if x.is_cuda:
        xs = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        xa = xs if out_dtype == torch.float32 else torch.empty_like(xs)
        _native_seq().token_shift(xs, xa, x, shift_w, prev_state, cu_seqlens,
                                  seq_lens, state_slots, token_seq)
        return xs, (x if out_dtype == torch.float32 else xa)
    return ref.token_shift(x, shift_w, prev_state, cu_seqlens, seq_lens,
                           state_slots, out_dtype)


def gated_norm_residual(x, y, gate, gate_bias, weight, eps, out_dtype=None):
    """x (fp32, in place) += rmsnorm(y * sigmoid(gate + bias)) * weight.
    Returns the new x cast to out_dtype when one is asked for."""
    if x.is_cuda:
        if out_dtype == torch.float32:
            out_dtype = None  # x itself is the fp32 copy
            ret_x = True
        else:
            ret_x = False
        xa = (torch.empty(x.shape, dtype=out_dtype, device=x.device)
              if out_dtype is not None else None)
        _native_seq().gated_norm_residual(x, xa, y, gate, gate_bias, weight, eps)
        return x if ret_x else xa
    return ref.gated_norm_residual(x, y, gate, gate_bias, weight, eps, out_dtype)


def rms_norm_f32(x, weight, eps, out_dtype):
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _native_seq().rms_norm_f32(out, x, weight, eps)
        return out
    return ref.rms_norm_f32(x, weight, eps, out_dtype)


def qk_norm_rope_cache(q, k, v, q_norm_w, k_norm_w, eps, positions,
                       inv_freq_qk, inv_freq_v, k_cache, v_cache,
                       slot_mapping, interleaved=True, rot_mag=1.0,
                       unit_norm_after=False):
    """rot_mag: factor on cos and sin; unit_norm_after: q and k are divided
    by their root mean square over the head after the rotation (no weight)."""
    if q.is_cuda:
        T, H, D = q.shape
        qo = torch.empty((T, H, D), dtype=q.dtype, device=q.device)
        _native_seq().qk_norm_rope_cache(
            qo, q, k, v, q_norm_w, k_norm_w, eps, positions, inv_freq_qk,
            inv_freq_v, k_cache, v_cache, slot_mapping, interleaved,
            float(rot_mag), bool(unit_norm_after))
        return qo
    return ref.qk_norm_rope_cache(q, k, v, q_norm_w, k_norm_w, eps, positions,
                                  inv_freq_qk, inv_freq_v, k_cache, v_cache,
                                  slot_mapping, interleaved, rot_mag,
                                  unit_norm_after)


# head sizes the MFMA kernels are built for (q/k size == value size)
_MFMA_HEAD_DIMS = (32, 64, 96, 128, 256)
_MFMA_LADDER_DIMS = (64, 128)  # 256-row ladder + flash-decode kernels


def sink_attention_tiles(q_lens, kv_lens, num_q_heads, num_kv_heads,
                         head_dim, device):
    """Work lists of the MFMA attention kernels for one step and one head
    layout (build once per step, reuse in every layer of that layout)."""
    big = head_dim in _MFMA_LADDER_DIMS
    return build_extend_tiles(
        q_lens, kv_lens, False, device, num_q_heads=num_q_heads, ladder=big,
        flash_decode=big and num_q_heads // num_kv_heads <= 8)


def attention_sink_paged(q, k_cache, v_cache, block_tables, seq_lens,
                         cu_seqlens, token_seq, scale, sink=True,
                         inv_freq_v=None, interleaved=True, max_q_len=0,
                         positions=None, tiles=None, sink_w=None,
                         softcap=0.0, window=0, keep_first=0, out=None,
                         out_scale=1.0, maps=1):
    """Causal attention of packed rows over paged keys with an optional
    sink (score 0, or sink_w per head), tanh-capped scores, a sliding
    window that keeps the first keep_first keys, and position-turned values
    (see ref.attention_sink_paged). bf16 rows with equal q/k and value head
    sizes the MFMA kernels are built for run those (then a pass that turns
    each row's output back); capped, windowed or per-head-sink attention
    runs the masked matrix-core kernels where they are built; anything else
    — float32 rows, other sizes — runs the general kernel. out: a [T, H, V]
    view (rows may be strided) to write, times out_scale. maps M > 1: a key
    row holds M keys side by side that share the row's value, and query
    head group g * M + m reads key m of key/value head g."""
    masked = (sink_w is not None or softcap > 0 or window > 0
              or out is not None or maps > 1
              or k_cache.untyped_storage().data_ptr()
              == v_cache.untyped_storage().data_ptr())
    if q.is_cuda and masked:
        T, H, D = q.shape
        V = v_cache.shape[3]
        if out is None:
            out = torch.empty((T, H, V), dtype=q.dtype, device=q.device)
        S = _native_seq()
        if not (use_masked_mfma and q.dtype == torch.bfloat16
                and S.attention_masked_mfma(
                    out, q, k_cache, v_cache, block_tables, seq_lens,
                    cu_seqlens, token_seq, scale, sink_w, softcap, window,
                    keep_first, out_scale, max_q_len == 1, maps)):
            S.attention_sink_paged(
                out, q, k_cache, v_cache, block_tables, seq_lens, cu_seqlens,
                token_seq, scale, sink, None, interleaved, max_q_len, sink_w,
                softcap, window, keep_first, out_scale, maps)
        return out
    if q.is_cuda:
        T, H, D = q.shape
        V = v_cache.shape[3]
        G = k_cache.shape[1]
        fast = (q.dtype == torch.bfloat16 and D == V and k_cache.shape[2] == 16)
        if (fast and max_q_len == 1 and T == seq_lens.shape[0]
                and D in _MFMA_LADDER_DIMS and H // G <= 8):
            # one row per sequence: the flash-decode kernel needs no host
            # work list, so it also runs inside a captured decode graph
            out = attention_decode_paged(
                q, k_cache, v_cache, block_tables, seq_lens, scale,
                sink=sink, native=_native_seq())
            if inv_freq_v is not None:
                _native_seq().unrotate_rows(out, positions, inv_freq_v,
                                            interleaved)
            return out
        if fast and tiles is not None and D in _MFMA_HEAD_DIMS:
            out = attention_extend_paged(
                q, k_cache, v_cache, block_tables, seq_lens, cu_seqlens,
                None, scale, tiles=tiles, sink=sink, native=_native_seq())
            if inv_freq_v is not None:
                _native_seq().unrotate_rows(out, positions, inv_freq_v,
                                            interleaved)
            return out
        out = torch.empty((T, H, V), dtype=q.dtype, device=q.device)
        _native_seq().attention_sink_paged(
            out, q, k_cache, v_cache, block_tables, seq_lens, cu_seqlens,
            token_seq, scale, sink, inv_freq_v, interleaved, max_q_len, None,
            0.0, 0, 0, 1.0, 1)
        return out
    res = ref.attention_sink_paged(q, k_cache, v_cache, block_tables,
                                   seq_lens, cu_seqlens, scale, sink,
                                   inv_freq_v, interleaved, sink_w, softcap,
                                   window, keep_first, maps)
    if out is None:
        return res
    out.copy_((res.float() * out_scale).to(out.dtype))
    return out


use_masked_mfma = True  # tests switch it off to compare both paths
# prompt portions over two-map key rows: the work-sorted prefill kernels
# (head sizes of the 256-row ladder kernel) instead of the masked tiles
use_ladder_maps = True
PREFILL_MAP_DIMS = (64, 128)


def seq_extension():
    """The sequence-state extension (its build of the paged attention
    kernels serves the layer-list models)."""
    return _native_seq()


SCAN_CHUNK = 64  # rows per chunk of the chunk-parallel recurrent prefill
use_lightning_mfma = True  # tests switch it off to compare both paths


def scan_chunks(q_lens: list[int], device, chunk: int = SCAN_CHUNK) -> dict:
    """Cut every sequence's rows of this step into chunks of <= `chunk`
    rows, as metadata of 'virtual sequences' the scan kernels can run in
    parallel: pass 1 scans each chunk from zero state into a scratch slot
    of its own (lens0: chunk starts at position 0), a small combine kernel
    walks each sequence's chunks in order and leaves every chunk's START
    state in its scratch slot, pass 2 scans again from those (lens1: start
    > 0) and writes the outputs. Same arithmetic as the row-by-row scan up
    to fp32 summation order."""
    rows, off = [], [0]
    for n in q_lens:
        rows += [min(chunk, n - j) for j in range(0, n, chunk)]
        off.append(len(rows))
    t = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    cu = [0]
    for r in rows:
        cu.append(cu[-1] + r)
    return {"n": len(rows), "cu": t(cu), "lens0": t(rows),
            "lens1": t([r + 1 for r in rows]), "rows": t(rows),
            "slots": t(list(range(len(rows)))), "off": t(off)}


# the lightning kernels' input convention without positions: rows pass
# through silu (no positions, no rotary table, pairing, key scale)
_SILU_ROWS = (None, None, False, 1.0)


def lightning_scan(q, k, v, decay, state, cu_seqlens, seq_lens, state_slots,
                   max_q_len=0, chunks=None):
    """chunks (scan_chunks of this step): run the prefill chunk-parallel."""
    if q.is_cuda:
        T, H, D = q.shape
        V = v.shape[2]
        S = _native_seq()
        out = torch.empty((T, H, V), dtype=torch.float32, device=q.device)
        if chunks is not None and max_q_len > SCAN_CHUNK:
            c = chunks
            part = torch.empty((c["n"], H, D, V), dtype=torch.float32,
                               device=q.device)
            # bf16 rows with head sizes the matrix-core kernels are built
            # for run those; the general kernel does the same two passes
            mfma = (q.dtype == torch.bfloat16 and use_lightning_mfma
                    and S.lightning_mfma(out, part, q, k, v, decay, c["cu"], 1,
                                         *_SILU_ROWS))
            if not mfma:
                S.lightning_scan(out, q, k, v, decay, part, c["cu"],
                                 c["lens0"], c["slots"], SCAN_CHUNK,
                                 *_SILU_ROWS)
            # the matrix-core passes keep their scratch states transposed
            S.lightning_combine(part, decay, state, c["off"], c["rows"],
                                cu_seqlens, seq_lens, state_slots, mfma)
            if mfma:
                S.lightning_mfma(out, part, q, k, v, decay, c["cu"], 2,
                                 *_SILU_ROWS)
            else:
                S.lightning_scan(out, q, k, v, decay, part, c["cu"],
                                 c["lens1"], c["slots"], SCAN_CHUNK,
                                 *_SILU_ROWS)
            return out
        S.lightning_scan(out, q, k, v, decay, state, cu_seqlens, seq_lens,
                         state_slots, max_q_len, *_SILU_ROWS)
        return out
    return ref.lightning_scan(q, k, v, decay, state, cu_seqlens, seq_lens,
                              state_slots)


def gated_rmsnorm(o, weight, gate, eps, out_dtype):
    if o.is_cuda:
        out = torch.empty(o.shape, dtype=out_dtype, device=o.device)
        _native_seq().gated_rmsnorm(out, o, weight, gate, eps)
        return out
    return ref.gated_rmsnorm(o, weight, gate, eps, out_dtype)


def causal_conv_silu(x, weight, bias, state, cu_seqlens, seq_lens,
                     state_slots, token_seq, weight_t=None):
    """weight_t: [taps, C] copy of the taps for the vectorised bf16 kernel."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _native_seq().causal_conv_silu(out, x, weight, weight_t, bias, state,
                                       cu_seqlens, seq_lens, state_slots,
                                       token_seq)
        return out
    return ref.causal_conv_silu(x, weight, bias, state, cu_seqlens, seq_lens,
                                state_slots)


def selective_scan(u, dbc, z, dt_w, dt_b, A, Dp, state, cu_seqlens, seq_lens,
                   state_slots, max_q_len=0, dt_pre=None, chunks=None):
    """dt_pre: fp32 [T, C] = dt_raw @ dt_w^T from a GEMM (else projected in
    the kernel); chunks (scan_chunks of this step): chunk-parallel prefill."""
    if u.is_cuda:
        S = _native_seq()
        out = torch.empty(u.shape, dtype=u.dtype, device=u.device)
        if chunks is not None and max_q_len > SCAN_CHUNK:
            c = chunks
            C, N = A.shape
            part = torch.empty((c["n"], C, N), dtype=torch.float32,
                               device=u.device)
            dsum = torch.empty((c["n"], C), dtype=torch.float32,
                               device=u.device)
            # pass 1 needs end states and dt sums only: the lane kernel
            # skips the outputs when it is given none
            light = dt_pre is not None and N <= 64
            S.selective_scan(None if light else out, u, dbc, z, dt_w, dt_b, A,
                             Dp, part, c["cu"], c["lens0"], c["slots"], dt_pre,
                             dsum)
            S.scan_combine(part, dsum, A, state, c["off"], cu_seqlens,
                           seq_lens, state_slots)
            S.selective_scan(out, u, dbc, z, dt_w, dt_b, A, Dp, part, c["cu"],
                             c["lens1"], c["slots"], dt_pre, None)
            return out
        S.selective_scan(out, u, dbc, z, dt_w, dt_b, A, Dp, state, cu_seqlens,
                         seq_lens, state_slots, dt_pre, None)
        return out
    return ref.selective_scan(u, dbc, z, dt_w, dt_b, A, Dp, state, cu_seqlens,
                              seq_lens, state_slots)


def gelu_tanh(x):
    """tanh-form GELU; x may be a column slice of a wider GEMM output."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _native_seq().gelu_tanh(out, x)
        return out
    return ref.gelu_tanh(x)


# ----------------------------------------------------------------------
# Stream-residual blocks, window attention with pooled blocks, rotary
# retention, clamped GLU, grouped routing (same extension, same rule).
# ----------------------------------------------------------------------
def stream_mix_norm(xs, y, y_bias, mix, out_w, in_w, norm_w, norm_b, eps):
    """Residual kept as s weighted copies xs [s, T, C] fp32. With y: every
    copy is rewritten from all old ones, new[t] = sum_s mix[s,t] old[s] +
    out_w[t] (y + y_bias). With in_w: returns layer_norm(sum_s in_w[s]
    new[s]) * norm_w + norm_b as fp32 [T, C] — the next sublayer's input,
    produced by the same pass over the rows."""
    if xs.is_cuda:
        s, T, C = xs.shape
        n = (torch.empty((T, C), dtype=torch.float32, device=xs.device)
             if in_w is not None else None)
        _native_seq().stream_mix_norm(xs, n, y, y_bias, mix, out_w, in_w,
                                      norm_w, norm_b, eps)
        return n
    return ref.stream_mix_norm(xs, y, y_bias, mix, out_w, in_w, norm_w,
                               norm_b, eps)


def short_conv_residual(h, weight, state, cu_seqlens, seq_lens, state_slots,
                        token_seq, out_dtype):
    """h + causal depthwise conv of h over time (taps = weight.shape[1],
    history of taps-1 rows per sequence in `state`), cast to out_dtype."""
    if h.is_cuda:
        out = torch.empty(h.shape, dtype=out_dtype, device=h.device)
        _native_seq().short_conv_residual(out, h, weight, state, cu_seqlens,
                                          seq_lens, state_slots, token_seq)
        return out
    return ref.short_conv_residual(h, weight, state, cu_seqlens, seq_lens,
                                   state_slots, out_dtype)


pool_slots_per_page = ref.pool_slots_per_page


def kv_write_pooled(k, v, k_cache, v_cache, kp_cache, vp_cache, slot_mapping,
                    positions, block_tables, token_seq, pool):
    """Write the step's keys/values to their pages, then the mean key and
    value of every block of `pool` positions this step completes into the
    pooled caches (see ref.kv_write_pooled for the layout)."""
    if k.is_cuda:
        _native_seq().kv_write_pooled(k, v, k_cache, v_cache, kp_cache,
                                      vp_cache, slot_mapping, positions,
                                      block_tables, token_seq, pool)
        return
    ref.kv_write_pooled(k, v, k_cache, v_cache, kp_cache, vp_cache,
                        slot_mapping, positions, block_tables, token_seq, pool)


use_window_mfma = True  # tests switch it off to compare both paths


def attention_window_pool(q, k_cache, v_cache, kp_cache, vp_cache,
                          block_tables, seq_lens, cu_seqlens, token_seq,
                          scale, window, pool, out, out_scale=1.0,
                          max_q_len=0):
    """Sliding-window softmax attention whose rows also see one pooled
    key/value per block of `pool` positions older than every key of the
    window (ref.attention_window_pool). Writes out [T, H, V] (may be a
    column slice of a wider row), scaled by out_scale."""
    if q.is_cuda:
        S = _native_seq()
        if not (use_window_mfma and q.dtype == torch.bfloat16
                and S.attention_window_pool_mfma(
                    out, q, k_cache, v_cache, kp_cache, vp_cache, block_tables,
                    seq_lens, cu_seqlens, token_seq, scale, window, pool,
                    out_scale, max_q_len == 1)):
            S.attention_window_pool(
                out, q, k_cache, v_cache, kp_cache, vp_cache, block_tables,
                seq_lens, cu_seqlens, token_seq, scale, window, pool,
                out_scale)
        return out
    return ref.attention_window_pool(q, k_cache, v_cache, kp_cache, vp_cache,
                                     block_tables, seq_lens, cu_seqlens,
                                     scale, window, pool, out, out_scale)


def retention_scan(q, k, v, decay, state, cu_seqlens, seq_lens, state_slots,
                   positions, inv_freq, interleaved, k_scale, max_q_len=0,
                   chunks=None):
    """The lightning kernels on plain rows: q and k are turned by their
    position (first 2*len(inv_freq) dims) and k scaled as they are loaded,
    nothing is activated. chunks: chunk-parallel prefill as lightning_scan."""
    if q.is_cuda:
        T, H, D = q.shape
        V = v.shape[2]
        S = _native_seq()
        out = torch.empty((T, H, V), dtype=torch.float32, device=q.device)
        rot = (positions, inv_freq, bool(interleaved), float(k_scale))
        if chunks is not None and max_q_len > SCAN_CHUNK:
            c = chunks
            part = torch.empty((c["n"], H, D, V), dtype=torch.float32,
                               device=q.device)
            mfma = (q.dtype == torch.bfloat16 and use_lightning_mfma
                    and S.lightning_mfma(out, part, q, k, v, decay, c["cu"], 1,
                                         *rot))
            if not mfma:
                S.lightning_scan(out, q, k, v, decay, part, c["cu"],
                                 c["lens0"], c["slots"], SCAN_CHUNK, *rot)
            S.lightning_combine(part, decay, state, c["off"], c["rows"],
                                cu_seqlens, seq_lens, state_slots, mfma)
            if mfma:
                S.lightning_mfma(out, part, q, k, v, decay, c["cu"], 2, *rot)
            else:
                S.lightning_scan(out, q, k, v, decay, part, c["cu"],
                                 c["lens1"], c["slots"], SCAN_CHUNK, *rot)
            return out
        S.lightning_scan(out, q, k, v, decay, state, cu_seqlens, seq_lens,
                         state_slots, max_q_len, *rot)
        return out
    return ref.retention_scan(q, k, v, decay, state, cu_seqlens, seq_lens,
                              state_slots, positions, inv_freq, interleaved,
                              k_scale)


def head_norm_gate(o, gate, eps, heads, out, out_scale=1.0):
    """Per-head unit RMS of o [T, heads*V] fp32, times silu(gate), times
    out_scale, into out (may be a column slice of a wider row)."""
    if o.is_cuda:
        _native_seq().head_norm_gate(out, o, gate, eps, heads, out_scale)
        return out
    return ref.head_norm_gate(o, gate, eps, heads, out, out_scale)


_GLU_MODES = {"swiglu": 0, "clamped": 1, "gelu_tanh": 2}


def glu_act(gu, kind, limit=0.0, alpha=1.0, out=None, row_scale=None):
    """[gate | up] rows -> activated rows (ref.glu_act); out: a [T, F]
    view (rows may be strided) to write instead of a new tensor; row_scale
    [T] fp32: a factor on each row's gate and up."""
    if gu.is_cuda:
        F_ = gu.shape[-1] // 2
        if out is None:
            out = torch.empty((gu.shape[0], F_), dtype=gu.dtype,
                              device=gu.device)
        _native_seq().glu_act(out, gu, _GLU_MODES[kind], float(limit),
                              float(alpha), row_scale)
        return out
    res = ref.glu_act(gu, kind, limit, alpha, row_scale)
    if out is None:
        return res
    out.copy_(res)
    return out


def moe_route_grouped(logits, top, groups=1, keep=1, score="softmax",
                      renorm=True, matrix=False):
    """Group-limited routing: (weights [T, top] fp32, ids [T, top] int32);
    score "softmax" or "sigmoid", renorm: the chosen scores divided by their
    sum. matrix: also a [T, E] fp32 tensor holding each row's weights at
    the experts it uses and 0 elsewhere."""
    if logits.is_cuda:
        T, E = logits.shape
        w = torch.empty((T, top), dtype=torch.float32, device=logits.device)
        ids = torch.empty((T, top), dtype=torch.int32, device=logits.device)
        mat = (torch.empty((T, E), dtype=torch.float32, device=logits.device)
               if matrix else None)
        _native_seq().moe_route_grouped(w, ids, logits.contiguous(), top,
                                        groups, keep, score == "sigmoid",
                                        bool(renorm), mat)
        return (w, ids, mat) if matrix else (w, ids)
    w, ids = ref.moe_route_grouped(logits, top, groups, keep, score, renorm)
    if matrix:
        return w, ids, ref.route_scale_matrix(w, ids, logits.shape[1])
    return w, ids


def moe_mix_seq(y, weights, ids):
    """moe_mix for callers of the sequence-state extension (any float
    dtype of y)."""
    if y.is_cuda:
        El, T, H = y.shape
        out = torch.empty(T, H, dtype=y.dtype, device=y.device)
        _native_seq().moe_mix(out, y.contiguous(), weights, ids)
        return out
    return ref.moe_mix(y, weights, ids, 0)


def moe_mix_rows_seq(y, weights, rows, add=None):
    """out[t] = sum_j weights[t, j] y[rows[t, j]] (+ add[t])."""
    if y.is_cuda:
        T, k = weights.shape
        out = torch.empty(T, y.shape[1], dtype=y.dtype, device=y.device)
        _native_seq().moe_mix_rows(out, y.contiguous(), weights, rows, add)
        return out
    return ref.moe_mix_rows(y, weights, rows, add)


# ----------------------------------------------------------------------
# Shared-norm parallel blocks with a tanh norm, latent attention, mamba2
# (same extension, same rule).
# ----------------------------------------------------------------------
def residual_tanh_norm(x, y, mult, alpha, weight, bias, out_dtype, xa=None):
    """x (fp32 residual, in place) += mult * y when y is given; xa, a
    [T, C] view of the model's dtype (any row stride), takes the new x;
    returns tanh(alpha x) * weight + bias in out_dtype (None when weight is
    None). alpha is a one-element fp32 tensor."""
    if x.is_cuda:
        h = (torch.empty(x.shape, dtype=out_dtype, device=x.device)
             if weight is not None else None)
        _native_seq().residual_tanh_norm(x, h, xa, y, float(mult), alpha,
                                         weight, bias)
        return h
    return ref.residual_tanh_norm(x, y, mult, alpha, weight, bias, out_dtype, xa)


def latent_prepare(cq, ckv, q_norm_w, kv_norm_w, eps, positions, inv_freq,
                   cache, slot_mapping):
    """Latent attention's row work before the up-projections
    (ref.latent_prepare): returns the normed query latent and writes the
    normed key/value latent with the turned shared key part to its page."""
    if cq.is_cuda:
        out = torch.empty(cq.shape, dtype=cq.dtype, device=cq.device)
        _native_seq().latent_prepare(out, cq, ckv, q_norm_w, kv_norm_w, eps,
                                     positions, inv_freq, cache, slot_mapping)
        return out
    return ref.latent_prepare(cq, ckv, q_norm_w, kv_norm_w, eps, positions,
                              inv_freq, cache, slot_mapping)


def latent_query(q, q_abs, positions, inv_freq, out):
    """out [T, H, Rk + 2P] = [q_abs ([H, T, Rk]) | turned last 2P dims of q]."""
    if q.is_cuda:
        _native_seq().latent_query(out, q, q_abs, positions, inv_freq)
        return out
    return ref.latent_query(q, q_abs, positions, inv_freq, out)


# rows per chunk of mamba2's chunk-parallel prefill: a chunk's state
# (heads x state x vdim floats) is written and read four times, so chunks
# are long; the scan itself is sequential inside a chunk either way
MAMBA2_CHUNK = 256


def mamba2_scan(xbc, dt_raw, dt_bias, rate, Dp, state, cu_seqlens, seq_lens,
                state_slots, heads, vdim, nstate, groups, max_q_len=0,
                chunks=None):
    """Scalar-decay state-space recurrence (ref.mamba2_scan); chunks
    (scan_chunks of this step): chunk-parallel prefill as lightning_scan —
    every chunk's end state and summed step sizes from zero state, a
    combine pass that leaves each chunk's start state, then the outputs."""
    if xbc.is_cuda:
        S = _native_seq()
        T = xbc.shape[0]
        out = torch.empty((T, heads * vdim), dtype=torch.float32,
                          device=xbc.device)
        if chunks is not None:
            c = chunks
            part = torch.empty((c["n"], heads, nstate, vdim),
                               dtype=torch.float32, device=xbc.device)
            dsum = torch.empty((c["n"], heads), dtype=torch.float32,
                               device=xbc.device)
            S.mamba2_scan(None, xbc, dt_raw, dt_bias, rate, Dp, part, c["cu"],
                          c["lens0"], c["slots"], heads, vdim, nstate, groups,
                          dsum)
            S.mamba2_combine(part, dsum, rate, state, c["off"], cu_seqlens,
                             seq_lens, state_slots)
            S.mamba2_scan(out, xbc, dt_raw, dt_bias, rate, Dp, part, c["cu"],
                          c["lens1"], c["slots"], heads, vdim, nstate, groups,
                          None)
            return out
        S.mamba2_scan(out, xbc, dt_raw, dt_bias, rate, Dp, state, cu_seqlens,
                      seq_lens, state_slots, heads, vdim, nstate, groups, None)
        return out
    return ref.mamba2_scan(xbc, dt_raw, dt_bias, rate, Dp, state, cu_seqlens,
                           seq_lens, state_slots, heads, vdim, nstate, groups)


def gate_group_norm(y, z, weight, groups, eps, out, out_scale=1.0):
    """out = per-group unit RMS of (y * silu(z)), times weight and out_scale
    (ref.gate_group_norm); y fp32, z and out row-strided views."""
    if y.is_cuda:
        _native_seq().gate_group_norm(out, y, z, weight, groups, eps,
                                      out_scale)
        return out
    return ref.gate_group_norm(y, z, weight, groups, eps, out, out_scale)


# ----------------------------------------------------------------------
# Two-norm parallel blocks with per-channel branch scales, difference
# attention behind short convolutions, input-scaled experts (same
# extension, same rule).
# ----------------------------------------------------------------------
def residual_pair_norm(x, y1, s1, y2, s2, w1, w2, eps, out_dtype):
    """x (fp32 residual, in place) += s1 * y1 + s2 * y2 (each when given,
    s per channel); returns (h1, h2), x divided by its root mean square
    times (1 + w1) and (1 + w2), for each weight given — two norms of the
    same rows from one pass."""
    if x.is_cuda:
        h1 = (torch.empty(x.shape, dtype=out_dtype, device=x.device)
              if w1 is not None else None)
        h2 = (torch.empty(x.shape, dtype=out_dtype, device=x.device)
              if w2 is not None else None)
        _native_seq().residual_pair_norm(x, h1, h2, y1, s1, y2, s2, w1, w2,
                                         float(eps))
        return h1, h2
    return ref.residual_pair_norm(x, y1, s1, y2, s2, w1, w2, eps, out_dtype)


def conv_qkv_cache(p, n_q, n_k, n_v, weight, weight_t, state, cu_seqlens,
                   seq_lens, state_slots, token_seq, positions, temp_coef,
                   temp_every, heads, kv_heads, maps, k_cache, v_cache,
                   slot_mapping):
    """Short causal convolution over the q | k | v channels of the
    in-projection's rows, the position-dependent query factor, the query
    heads regrouped by key map, keys and values to their pages, and the
    sequences' new histories (ref.conv_qkv_cache). weight_t: [taps, C] copy
    of the taps for the vectorised bf16 kernel. Returns q [T, n_q]."""
    if p.is_cuda:
        qo = torch.empty((p.shape[0], n_q), dtype=p.dtype, device=p.device)
        _native_seq().conv_qkv_cache(
            qo, p, n_q, n_k, n_v, weight, weight_t, state, cu_seqlens,
            seq_lens, state_slots, token_seq, positions, float(temp_coef),
            int(temp_every), heads, kv_heads, maps, k_cache, v_cache,
            slot_mapping)
        return qo
    return ref.conv_qkv_cache(p, n_q, n_k, n_v, weight, state, cu_seqlens,
                              seq_lens, state_slots, positions, temp_coef,
                              temp_every, heads, kv_heads, maps, k_cache,
                              v_cache, slot_mapping)


def diff_head_norm_gate(a, gate, lam, eps, mult, heads, kv_heads, out):
    """Two attention maps per head into one gated output row
    (ref.diff_head_norm_gate): (a1 - lam a2) at unit RMS per head, times
    mult, times sigmoid(gate)."""
    if a.is_cuda:
        _native_seq().diff_head_norm_gate(out, a, gate, float(lam), float(eps),
                                          float(mult), heads, kv_heads)
        return out
    return ref.diff_head_norm_gate(a, gate, lam, eps, mult, heads, kv_heads,
                                   out)


def moe_glu_scaled(gu, scale, experts, ff, shared_ff):
    """Activated rows of all experts side by side, each expert's gate and
    up scaled by the row's weight for it, plus the shared expert's
    (ref.moe_glu_scaled)."""
    if gu.is_cuda:
        out = torch.empty((gu.shape[0], experts * ff + shared_ff),
                          dtype=gu.dtype, device=gu.device)
        _native_seq().moe_glu_scaled(out, gu, scale, experts, ff, shared_ff)
        return out
    return ref.moe_glu_scaled(gu, scale, experts, ff, shared_ff)
