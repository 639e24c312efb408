"""Layer-list decoders (config.HybridModelConfig): a stack of blocks, each
with one mixer of arks_amd/models/mixers.py and an optional dense
feed-forward, around an fp32 residual stream.

What an architecture fixes is a BlockArrangement. Fusolix's is:
  - the residual is `streams` weighted copies xs[s] (all equal to the scaled
    embedding at first); sublayer q of a layer reads u = sum_s in_q[s] xs[s],
    and its result y rewrites every copy from all old ones:
    xs[t] <- sum_s mix_q[s, t] xs[s] + out_q[t] y; the model's output is
    the sum of the copies
  - layer norm (weight and bias) on each sublayer's INPUT, then a short
    causal depthwise convolution added to its own input (h + conv(h)); its
    last taps-1 inputs are per-sequence state, per layer and sublayer
  - mixer "parallel" (models/mixers.py ParallelMixer), feed-forward
    ClampedGLU or GroupedMoE (models/feedforward.py)
  Kernel plan per sublayer: stream_mix_norm (applies the previous
  sublayer's y to the copies, reads the next input and normalises it, one
  pass) -> short_conv_residual -> sublayer.

Gagorax's is:
  - the sublayers read the residual x itself and the RMS norm sits on each
    sublayer's OUTPUT:  x += norm(sublayer(x)) * w
  - token shift: the mixer reads x_t + (x_{t-1} - x_t) * s (x_{-1} = 0);
    the last row of every step is per-sequence state in every block
  - gated residual: the sublayer's result is multiplied by
    sigmoid(W_g x + b_g) (x unshifted) before that norm
  - feed-forward = W_down gelu_tanh(W_up x); logits = head(norm(x)) * scale

Kernel plan per block (bf16 serving; fp32 runs the same kernels on float
rows): token_shift -> GEMM(mixer in) .. mixer kernels .. GEMM(mixer out),
GEMM(gate) -> gated_norm_residual [-> GEMM(up|gate) -> gelu_tanh ->
GEMM(down) -> gated_norm_residual]. The feed-forward's up projection and
its residual gate read the same row, so they are one fused GEMM.

Legalix's is:
  - ONE norm per layer, a tanh norm without statistics,
    h = tanh(alpha x) w + b, read by both sublayers;
    x += mult * (mixer(h) + ff(h)) (SharedNormBlock)
  - mixers "attention" (capped scores, window with kept first tokens),
    "latent_attention", "mamba2"; feed-forward GLU with tanh-GELU
  - a run of layers may loop: the same weights run `times` passes, each
    pass with caches and states of its own; every pass starts with
    x <- W_loop [x | x0], x0 the scaled embedding
  Kernel plan per layer: residual_tanh_norm (adds the previous layer's
  result to the fp32 residual and norms, one pass) -> ONE GEMM for every
  in-projection of the layer [mixer | gate | up] -> mixer kernels and
  glu_act, each writing its columns of one buffer -> ONE GEMM over
  [W_o | W_down], whose fp32 accumulation is the sum of both sublayers.

Rivolix's is:
  - TWO norms of the same x per layer, RMS norms whose stored weight is the
    distance from one, one in front of the mixer and one in front of the
    feed-forward; each branch's result is multiplied per channel (ls1, ls2)
    where it joins the residual:
    x += ls1 * mixer(n1(x)) + ls2 * ff(n2(x)) (DualNormBlock)
  - mixers "attention" (two-map difference attention behind short
    convolutions; a layer may read an earlier layer's key/value pages) and
    "attention_2" (values are the keys; rotary with ramp-scaled
    frequencies, then unit RMS of q and k); feed-forward InputScaledMoE;
    the logits are taken with the embedding table
  Kernel plan per layer: residual_pair_norm (adds the previous layer's two
  results, scaled, to the fp32 residual and writes both normed rows, one
  pass) -> mixer and feed-forward, each with GEMMs of its own (their
  inputs differ).

The per-layer cache is a dict of tensors (paged KV for attention, slot
state for the recurrent mixers and the token shift), allocated by
allocate_cache() from each mixer's cache_layout(). A sequence that starts at
position 0 ignores whatever its slot holds, so slots and pages are reused
without clearing. Tensor parallelism is not implemented for these models.
"""

from __future__ import annotations

import zlib
from dataclasses import dataclass

import torch
import torch.nn as nn

from .. import ops
from ..config import HybridModelConfig
from ..engine.forward_batch import ForwardBatch
from ..parallel.comm import get_tp_world_size
from .feedforward import GLU, build_feedforward
from .mixers import build_mixer, linear, linear_f32, _param


@dataclass(frozen=True)
class BlockArrangement:
    token_shift: bool = True
    gated_residual: bool = True
    # "output": RMS norm on each sublayer's result (HybridBlock);
    # "input": layer norm with bias in front of each sublayer, residual in
    # weighted copies, short input convolution (StreamBlock);
    # "shared": one tanh norm in front of both sublayers, which run side by
    # side (SharedNormBlock);
    # "dual": two RMS norms of the same rows, one per sublayer, the
    # sublayers side by side, a per-channel scale on each result
    # (DualNormBlock)
    norm_place: str = "output"


ARRANGEMENTS = {
    "Gagorax": BlockArrangement(),
    "Fusolix": BlockArrangement(token_shift=False, gated_residual=False,
                                norm_place="input"),
    "Legalix": BlockArrangement(token_shift=False, gated_residual=False,
                                norm_place="shared"),
    "Rivolix": BlockArrangement(token_shift=False, gated_residual=False,
                                norm_place="dual"),
}


class HybridBlock(nn.Module):
    def __init__(self, width: int, spec: dict, eps: float, dtype,
                 arr: BlockArrangement):
        super().__init__()
        if arr.norm_place != "output":
            raise NotImplementedError(arr.norm_place)
        f32 = torch.float32
        self.arr, self.eps, self.width = arr, eps, width
        self.mixer = build_mixer(spec["type"], spec["mixer"], width, eps, dtype)
        self.norm1 = _param(width, dtype=f32)
        self.shift = _param(width, dtype=f32) if arr.token_shift else None
        self.rg1 = _param(width, width, dtype=dtype) if arr.gated_residual else None
        self.rg1_b = _param(width, dtype=f32) if arr.gated_residual else None
        self.ff = spec["mlp"]["ff"] if spec.get("mlp") is not None else 0
        if self.ff:
            gate_rows = width if arr.gated_residual else 0
            self.norm2 = _param(width, dtype=f32)
            self.up_gate = _param(self.ff + gate_rows, width, dtype=dtype)
            self.down = _param(width, self.ff, dtype=dtype)
            self.rg2_b = _param(width, dtype=f32) if arr.gated_residual else None

    def weight_map(self) -> dict:
        m = {"mix." + k: v for k, v in self.mixer.weight_map().items()}
        m["norm1"] = (self.norm1, 0)
        if self.shift is not None:
            m["shift"] = (self.shift, 0)
        if self.rg1 is not None:
            m["rg1"] = (self.rg1, 0)
            m["rg1.b"] = (self.rg1_b, 0)
        if self.ff:
            m["norm2"] = (self.norm2, 0)
            m["mlp.up"] = (self.up_gate, 0)
            m["mlp.down"] = (self.down, 0)
            if self.arr.gated_residual:
                m["rg2"] = (self.up_gate, self.ff)
                m["rg2.b"] = (self.rg2_b, 0)
        return m

    def cache_layout(self, block_size: int, dtype) -> dict:
        out = dict(self.mixer.cache_layout(block_size, dtype))
        if self.shift is not None:
            out["shift"] = ("slot", (self.width,), torch.float32)
        return out

    def forward(self, x, batch: ForwardBatch, cache: dict, dtype) -> None:
        """x: fp32 residual rows [T, width], updated in place."""
        if self.shift is not None:
            xs, xa = ops.token_shift(
                x, self.shift, cache["shift"], batch.cu_seqlens,
                batch.seq_lens, batch.state_slots, batch.token_seq, dtype)
        else:
            xs = xa = x.to(dtype)
        y = self.mixer(xs, batch, cache)
        g = linear(xa, self.rg1) if self.rg1 is not None else None
        xa = ops.gated_norm_residual(x, y, g, self.rg1_b, self.norm1, self.eps,
                                     dtype if self.ff else None)
        if self.ff:
            ug = linear(xa, self.up_gate)
            h = ops.gelu_tanh(ug[:, :self.ff])
            y = linear(h, self.down)
            g = ug[:, self.ff:] if self.arr.gated_residual else None
            ops.gated_norm_residual(x, y, g, self.rg2_b, self.norm2, self.eps, None)


class StreamBlock(nn.Module):
    """One layer of the stream arrangement: up to two sublayers (mixer,
    feed-forward), each with its layer norm, input convolution and the
    three small tensors that connect it to the residual copies."""

    def __init__(self, width: int, spec: dict, streams: int, taps: int,
                 eps: float, dtype):
        super().__init__()
        f32 = torch.float32
        self.width, self.taps, self.eps = width, taps, eps
        self.mixer = build_mixer(spec["type"], spec["mixer"], width, eps, dtype)
        self.ffn = (build_feedforward(spec["mlp"], width, dtype)
                    if spec.get("mlp") is not None else None)
        self.nsub = 2 if self.ffn is not None else 1
        for q in range(1, self.nsub + 1):
            setattr(self, f"norm{q}", _param(width, dtype=f32))
            setattr(self, f"norm{q}_b", _param(width, dtype=f32))
            setattr(self, f"hc{q}_in", _param(streams, dtype=f32))
            setattr(self, f"hc{q}_out", _param(streams, dtype=f32))
            setattr(self, f"hc{q}_mix", _param(streams, streams, dtype=f32))
            if taps:
                setattr(self, f"canon{q}", _param(width, taps, dtype=f32))

    def weight_map(self) -> dict:
        m = {"mix." + k: v for k, v in self.mixer.weight_map().items()}
        if self.ffn is not None:
            m.update({"mlp." + k: v for k, v in self.ffn.weight_map().items()})
        for q in range(1, self.nsub + 1):
            m[f"norm{q}"] = (getattr(self, f"norm{q}"), 0)
            m[f"norm{q}.b"] = (getattr(self, f"norm{q}_b"), 0)
            for leaf in ("in", "out", "mix"):
                m[f"hc{q}.{leaf}"] = (getattr(self, f"hc{q}_{leaf}"), 0)
            if self.taps:
                m[f"canon{q}"] = (getattr(self, f"canon{q}"), 0)
        return m

    def cache_layout(self, block_size: int, dtype) -> dict:
        out = {"mix." + k: v
               for k, v in self.mixer.cache_layout(block_size, dtype).items()}
        if self.taps > 1:
            for q in range(1, self.nsub + 1):
                out[f"canon{q}"] = ("slot", (self.taps - 1, self.width),
                                    torch.float32)
        return out

    def sublayers(self):
        """(index, module, cache prefix) of each sublayer in order."""
        yield 1, self.mixer, "mix."
        if self.ffn is not None:
            yield 2, self.ffn, None


class SharedNormBlock(nn.Module):
    """x += mult * (mixer(h) + ff(h)) with h = tanh(alpha x) w + b: both
    sublayers are split modules (in_spans / core / out_cols), so the block
    owns one in-projection [mixer rows | gate | up] and one out-projection
    [W_o | W_down]; the sum of the two results is the out GEMM's own fp32
    accumulation."""

    def __init__(self, width: int, spec: dict, eps: float, dtype, arch: str,
                 ff_act: str = "gelu_tanh"):
        super().__init__()
        f32 = torch.float32
        self.width = width
        self.mixer = build_mixer(spec["type"], spec["mixer"], width, eps, dtype,
                                 arch=arch, own_projections=False)
        mlp = spec.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
        self.ffn = (GLU(width, mlp["ff"], dtype, act=ff_act,
                        own_projections=False) if mlp is not None else None)
        self.parts = [("mix.", self.mixer)] + (
            [("mlp.", self.ffn)] if self.ffn is not None else [])
        self.rows = [sum(n for _, n, _ in m.in_spans()) for _, m in self.parts]
        self.cols = [m.out_cols for _, m in self.parts]
        self.w_in = _param(sum(self.rows), width, dtype=dtype)
        self.w_out = _param(width, sum(self.cols), dtype=dtype)
        self.norm_w = _param(width, dtype=f32)
        self.norm_b = _param(width, dtype=f32)
        self.norm_alpha = _param(dtype=f32)

    def weight_map(self) -> dict:
        m = {"norm1": (self.norm_w, 0), "norm1.b": (self.norm_b, 0),
             "norm1.alpha": (self.norm_alpha, 0)}
        row = col = 0
        for (prefix, part), cols in zip(self.parts, self.cols):
            for name, n, has_b in part.in_spans():
                assert not has_b
                m[prefix + name] = (self.w_in, row)
                row += n
            out_name = "o" if prefix == "mix." else "down"
            m[prefix + out_name] = (self.w_out, 0, col, (self.width, cols))
            col += cols
            m.update({prefix + k: v for k, v in part.extra_weights().items()})
        return m

    def cache_layout(self, block_size: int, dtype) -> dict:
        return dict(self.mixer.cache_layout(block_size, dtype))

    def forward(self, h, batch: ForwardBatch, cache: dict) -> torch.Tensor:
        """h: the normed rows; returns mixer(h) + ff(h) in h's dtype."""
        p = linear(h, self.w_in)
        buf = torch.empty((h.shape[0], sum(self.cols)), dtype=h.dtype,
                          device=h.device)
        row = col = 0
        for (_, part), rows, cols in zip(self.parts, self.rows, self.cols):
            part.core(p[:, row:row + rows], batch, cache,
                      buf[:, col:col + cols], 1.0)
            row += rows
            col += cols
        return linear(buf, self.w_out)


class DualNormBlock(nn.Module):
    """x += ls1 * mixer(n1(x)) + ls2 * ff(n2(x)), n_q(x) = x / rms(x) *
    (1 + norm_q). The sum and both norms are one kernel of the model's
    forward (ops.residual_pair_norm); this module holds the weights and the
    two sublayers. kv_from: the layer run whose key/value pages the mixer
    reads instead of pages of its own."""

    def __init__(self, width: int, spec: dict, eps: float, dtype, arch: str):
        super().__init__()
        f32 = torch.float32
        self.width = width
        self.mixer = build_mixer(spec["type"], spec["mixer"], width, eps, dtype,
                                 arch=arch)
        self.kv_from = spec["mixer"].get("kv_from")
        self.ffn = (build_feedforward(spec["mlp"], width, dtype, arch)
                    if spec.get("mlp") is not None else None)
        self.norm1 = _param(width, dtype=f32)
        self.ls1 = _param(width, dtype=f32)
        if self.ffn is not None:
            self.norm2 = _param(width, dtype=f32)
            self.ls2 = _param(width, dtype=f32)
        else:
            self.norm2 = self.ls2 = None

    def weight_map(self) -> dict:
        m = {"mix." + k: v for k, v in self.mixer.weight_map().items()}
        m["norm1"], m["ls1"] = (self.norm1, 0), (self.ls1, 0)
        if self.ffn is not None:
            m.update({"mlp." + k: v for k, v in self.ffn.weight_map().items()})
            m["norm2"], m["ls2"] = (self.norm2, 0), (self.ls2, 0)
        return m

    def cache_layout(self, block_size: int, dtype) -> dict:
        return dict(self.mixer.cache_layout(block_size, dtype))


class HybridForCausalLM(nn.Module):
    supports_float32 = True
    has_sequence_state = True  # engine: state slots, no prefix reuse

    def __init__(self, cfg: HybridModelConfig, dtype=torch.bfloat16):
        super().__init__()
        if get_tp_world_size() != 1:
            raise NotImplementedError(
                f"{cfg.architecture}: tensor parallelism is not implemented")
        self.cfg, self.dtype = cfg, dtype
        arr = ARRANGEMENTS[cfg.architecture]
        W = cfg.hidden_size
        self.arr = arr
        self.embed = _param(cfg.vocab_size, W, dtype=dtype)
        if arr.norm_place == "input":
            self.layers = nn.ModuleList(
                StreamBlock(W, spec, cfg.streams, cfg.conv_taps,
                            cfg.rms_norm_eps, dtype)
                for spec in cfg.layers)
        elif arr.norm_place == "shared":
            self.layers = nn.ModuleList(
                SharedNormBlock(W, spec, cfg.rms_norm_eps, dtype,
                                cfg.architecture)
                for spec in cfg.layers)
        elif arr.norm_place == "dual":
            self.layers = nn.ModuleList(
                DualNormBlock(W, spec, cfg.rms_norm_eps, dtype,
                              cfg.architecture)
                for spec in cfg.layers)
        else:
            self.layers = nn.ModuleList(
                HybridBlock(W, spec, cfg.rms_norm_eps, dtype, arr)
                for spec in cfg.layers)
        # layer runs in execution order (a looped layer once per pass, each
        # run with a cache of its own) and the runs that open a pass
        if hasattr(cfg, "layer_runs"):
            self.run_order, loop_starts = cfg.layer_runs()
        else:
            self.run_order, loop_starts = list(range(len(self.layers))), []
        self.loop_starts = frozenset(loop_starts)
        self.final_norm = _param(W, dtype=torch.float32)
        self._wmap = {"embed": (self.embed, 0),
                      "final.norm": (self.final_norm, 0)}
        if getattr(cfg, "tied_head", False):
            self.head = self.embed  # logits through the embedding table
        else:
            self.head = _param(cfg.vocab_size, W, dtype=dtype)
            self._wmap["head"] = (self.head, 0)
        if arr.norm_place == "input":
            self.final_norm_b = _param(W, dtype=torch.float32)
            self._wmap["final.norm.b"] = (self.final_norm_b, 0)
            self.register_buffer("sum_w", torch.ones(cfg.streams),
                                 persistent=False)
        if arr.norm_place == "shared":
            self.final_norm_b = _param(W, dtype=torch.float32)
            self.final_norm_alpha = _param(dtype=torch.float32)
            self._wmap["final.norm.b"] = (self.final_norm_b, 0)
            self._wmap["final.norm.alpha"] = (self.final_norm_alpha, 0)
            if getattr(cfg, "loop", None):
                self.loop_in = _param(W, 2 * W, dtype=dtype)
                self._wmap["loop.in"] = (self.loop_in, 0)
        for i, layer in enumerate(self.layers):
            for k, v in layer.weight_map().items():
                self._wmap[f"l{i}.{k}"] = v
        self._loaded: set = set()
        self.residual_tap = None  # tests/tools: called with (layer, x)

    # ------------------------------------------------------------ cache
    def cache_layout(self, block_size: int) -> list:
        """One dict per layer RUN: every pass of a looped layer has pages
        and state of its own."""
        return [self.layers[i].cache_layout(block_size, self.dtype)
                for i in self.run_order]

    def kv_block_bytes(self, block_size: int) -> int:
        total = 0
        for layout in self.cache_layout(block_size):
            for kind, shape, dt in layout.values():
                if kind == "paged":
                    total += int(torch.tensor(shape).prod()) * dt.itemsize
        return max(total, 1)

    def state_slot_bytes(self) -> int:
        total = 0
        for layout in self.cache_layout(16):
            for kind, shape, dt in layout.values():
                if kind == "slot":
                    total += int(torch.tensor(shape).prod()) * dt.itemsize
        return total

    def allocate_cache(self, num_blocks: int, block_size: int, num_slots: int,
                       device) -> list:
        caches = []
        for layout in self.cache_layout(block_size):
            c = {}
            for name, (kind, shape, dt) in layout.items():
                lead = num_blocks if kind == "paged" else num_slots
                c[name] = torch.zeros((lead, *shape), dtype=dt, device=device)
            caches.append(c)
        return caches

    # ------------------------------------------------------------ forward
    def forward(self, batch: ForwardBatch, caches: list) -> torch.Tensor:
        """fp32 logits for batch.logits_indices rows (all rows if None)."""
        if self.arr.norm_place == "input":
            return self._forward_streams(batch, caches)
        if self.arr.norm_place == "shared":
            return self._forward_shared(batch, caches)
        if self.arr.norm_place == "dual":
            return self._forward_dual(batch, caches)
        x = self.embed[batch.input_ids].float()
        for i, layer in enumerate(self.layers):
            layer(x, batch, caches[i], self.dtype)
            if self.residual_tap is not None:
                self.residual_tap(i, x)
        if batch.logits_indices is not None:
            x = x[batch.logits_indices]
        xn = ops.rms_norm_f32(x, self.final_norm, self.cfg.rms_norm_eps, self.dtype)
        return linear_f32(xn, self.head) * self.cfg.logit_scale

    def _forward_streams(self, batch: ForwardBatch, caches: list) -> torch.Tensor:
        """Stream arrangement: the previous sublayer's result is applied to
        the residual copies by the kernel that reads the next sublayer's
        input, so each sublayer costs one pass over the copies."""
        cfg, dtype = self.cfg, self.dtype
        x0 = self.embed[batch.input_ids].float() * cfg.embed_scale
        xs = x0.unsqueeze(0).repeat(cfg.streams, 1, 1)
        pend = (None, None, None, None)  # y, its fp32 bias, mix, out
        for i, layer in enumerate(self.layers):
            cache = caches[i]
            for q, module, prefix in layer.sublayers():
                n = ops.stream_mix_norm(
                    xs, *pend, getattr(layer, f"hc{q}_in"),
                    getattr(layer, f"norm{q}"), getattr(layer, f"norm{q}_b"),
                    layer.eps)
                if layer.taps:
                    h = ops.short_conv_residual(
                        n, getattr(layer, f"canon{q}"), cache.get(f"canon{q}"),
                        batch.cu_seqlens, batch.seq_lens, batch.state_slots,
                        batch.token_seq, dtype)
                else:
                    h = n.to(dtype)
                sub = ({k[len(prefix):]: v for k, v in cache.items()
                        if k.startswith(prefix)} if prefix else None)
                y = module(h, batch, sub)
                pend = (y, getattr(module, "out_bias", None),
                        getattr(layer, f"hc{q}_mix"),
                        getattr(layer, f"hc{q}_out"))
            if self.residual_tap is not None:
                ops.stream_mix_norm(xs, *pend, None, None, None, layer.eps)
                pend = (None, None, None, None)
                self.residual_tap(i, xs.sum(0))
        n = ops.stream_mix_norm(xs, *pend, self.sum_w, self.final_norm,
                                self.final_norm_b, cfg.rms_norm_eps)
        if batch.logits_indices is not None:
            n = n[batch.logits_indices]
        return linear_f32(n.to(dtype), self.head) * cfg.logit_scale

    def _forward_shared(self, batch: ForwardBatch, caches: list) -> torch.Tensor:
        """Shared-norm arrangement: a layer's result waits until the kernel
        that norms the next layer's input adds it to the residual, so each
        layer costs one pass over the fp32 rows."""
        cfg, dtype = self.cfg, self.dtype
        mult = cfg.residual_mult
        x = self.embed[batch.input_ids].float()
        if cfg.embed_scale != 1.0:
            x *= cfg.embed_scale
        cat = None
        if self.loop_starts:
            # [x | x0] rows of the loop's input projection; the right half
            # is written once
            W = cfg.hidden_size
            cat = torch.empty((x.shape[0], 2 * W), dtype=dtype, device=x.device)
            cat[:, W:] = x
        y = None
        for run, i in enumerate(self.run_order):
            layer = self.layers[i]
            if run in self.loop_starts:
                ops.residual_tanh_norm(x, y, mult, None, None, None, dtype,
                                       xa=cat[:, :cfg.hidden_size])
                x = linear_f32(cat, self.loop_in)
                y = None
            h = ops.residual_tanh_norm(x, y, mult, layer.norm_alpha,
                                       layer.norm_w, layer.norm_b, dtype)
            y = layer(h, batch, caches[run])
            if self.residual_tap is not None:
                ops.residual_tanh_norm(x, y, mult, None, None, None, dtype)
                y = None
                self.residual_tap(run, x)
        if batch.logits_indices is not None:
            x = x[batch.logits_indices]
            y = y[batch.logits_indices] if y is not None else None
        n = ops.residual_tanh_norm(x, y, mult, self.final_norm_alpha,
                                   self.final_norm, self.final_norm_b, dtype)
        return linear_f32(n, self.head) * cfg.logit_scale

    def _forward_dual(self, batch: ForwardBatch, caches: list) -> torch.Tensor:
        """Two-norm arrangement: a layer's two results wait until the kernel
        that norms the next layer's inputs adds them, scaled per channel, to
        the residual, so each layer costs one pass over the fp32 rows."""
        cfg, dtype = self.cfg, self.dtype
        eps = cfg.rms_norm_eps
        x = self.embed[batch.input_ids].float()
        pend = (None, None, None, None)  # y1, ls1, y2, ls2
        for i, layer in enumerate(self.layers):
            h1, h2 = ops.residual_pair_norm(x, *pend, layer.norm1, layer.norm2,
                                            eps, dtype)
            cache = caches[i]
            if layer.kv_from is not None:
                src = caches[layer.kv_from]
                cache = {**cache, "k": src["k"], "v": src["v"]}
            y1 = layer.mixer(h1, batch, cache)
            y2 = layer.ffn(h2, batch, None) if layer.ffn is not None else None
            pend = (y1, layer.ls1, y2, layer.ls2)
            if self.residual_tap is not None:
                ops.residual_pair_norm(x, *pend, None, None, eps, dtype)
                pend = (None, None, None, None)
                self.residual_tap(i, x)
        if batch.logits_indices is not None:
            x = x[batch.logits_indices]
            pend = tuple(t[batch.logits_indices] if t is not None and j % 2 == 0
                         else t for j, t in enumerate(pend))
        n, _ = ops.residual_pair_norm(x, *pend, self.final_norm, None, eps,
                                      dtype)
        return linear_f32(n, self.head) * cfg.logit_scale

    # ------------------------------------------------------------ weights
    @staticmethod
    def _span(entry, w):
        """The part of a parameter one checkpoint tensor fills. Entries are
        (param, row) for row spans of fused parameters, or (param, row, col,
        shape[, index[, transposed]]) for column spans and for slices of
        stacked, pre-transposed parameters."""
        p, row = entry[0], entry[1]
        if len(entry) == 2:
            return p.data[row:row + w.shape[0]] if w.dim() else p.data
        col, shape = entry[2], entry[3]
        d = p.data
        if len(entry) > 4 and entry[4] is not None:
            d = d[entry[4]]
        if len(entry) > 5 and entry[5]:
            d = d.t()
        return d[row:row + shape[0], col:col + shape[1]]

    def load_hf_state_dict(self, tensors: dict) -> None:
        """Tensors by their checkpoint names ('embed', 'l<i>.mix.q', ...);
        fused parameters are filled span by span, in any order."""
        for name, w in tensors.items():
            if name not in self._wmap:
                raise KeyError(f"unexpected tensor {name!r}")
            p = self._wmap[name][0]
            span = self._span(self._wmap[name], w)
            if span.shape != w.shape:
                raise ValueError(f"{name}: shape {tuple(w.shape)} does not fit "
                                 f"{tuple(span.shape)}")
            span.copy_(w.to(p.dtype))
            self._loaded.add(name)
        if len(self._loaded) == len(self._wmap):
            self.finish_loading()

    def finish_loading(self) -> None:
        for layer in self.layers:
            if hasattr(layer.mixer, "finish_loading"):
                layer.mixer.finish_loading()

    def missing_tensors(self) -> list:
        return sorted(set(self._wmap) - self._loaded)

    @torch.no_grad()
    def random_init(self, seed: int = 0) -> None:
        """Seeded random weights with activations of order one at every
        block (benchmarks and tests; checkpoints load by name instead)."""
        dev = self.embed.device
        self._loaded.clear()
        streams = getattr(self.cfg, "streams", 1)
        for name, entry in self._wmap.items():
            p, row = entry[0], entry[1]
            s = (seed * 1000003 + zlib.crc32(name.encode())) % (2 ** 63 - 1)
            g = torch.Generator(device=dev).manual_seed(s)
            leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
            # rows of this tensor inside its (possibly fused) parameter
            if len(entry) > 2:
                shape = list(entry[3])
            else:
                shape = list(p.shape)
                if p.dim() >= 1:
                    nxt = sorted(e[1] for e in self._wmap.values()
                                 if e[0] is p and len(e) == 2 and e[1] > row)
                    shape[0] = (nxt[0] if nxt else p.shape[0]) - row

            def rn(std):
                return torch.randn(shape, generator=g, device=dev,
                                   dtype=torch.float32) * std

            if leaf.endswith(".alpha"):
                w = 0.5 + 0.5 * torch.rand(shape, generator=g, device=dev)
            elif self.arr.norm_place == "dual" and (
                    leaf.endswith("norm") or leaf in ("norm1", "norm2")):
                w = rn(0.1)  # stored as the distance from one
            elif leaf in ("ls1", "ls2"):
                w = 0.5 + rn(0.1)
            elif leaf in ("mix.lq1", "mix.lk1", "mix.lq2", "mix.lk2"):
                w = rn(0.3)
            elif leaf in ("mix.q.conv", "mix.k.conv", "mix.v.conv"):
                w = rn(0.5)
            elif leaf.endswith("norm") or leaf in ("norm1", "norm2"):
                w = 1.0 + rn(0.1)
            elif leaf == "mix.dt_bias":
                w = rn(0.5) - 1.0
            elif leaf == "mix.sink":
                w = rn(1.0)
            elif leaf.startswith("canon"):
                w = rn(0.3)
            elif leaf.startswith("hc") and leaf.endswith(".in"):
                w = 1.0 / streams + rn(0.2)
            elif leaf.startswith("hc") and leaf.endswith(".out"):
                w = 1.0 + rn(0.3)
            elif leaf.startswith("hc") and leaf.endswith(".mix"):
                w = torch.eye(streams, device=dev) + rn(0.15)
            elif leaf.endswith("router"):
                w = rn(2.0 * shape[-1] ** -0.5)
            elif leaf == "shift":
                w = torch.rand(shape, generator=g, device=dev)
            elif leaf == "mix.A_log":
                w = torch.log(1.0 + 7.0 * torch.rand(shape, generator=g, device=dev))
            elif leaf == "mix.dt.b":
                w = rn(0.5) - 3.0
            elif leaf.endswith(".b") or leaf == "mix.D":
                w = rn(0.3)
            elif leaf == "embed":
                w = rn(1.0 / getattr(self.cfg, "embed_scale", 1.0))
            else:
                w = rn(shape[-1] ** -0.5)
            self.load_hf_state_dict({name: w})
