"""Feed-forward sublayers of the layer-list decoders, each with its
constants as constructor parameters:

- GLU: W_down act(W_gate x, W_up x) for the activations of ops.glu_act.
- ClampedGLU: W_down act(W_gate x, W_up x) with the gate capped from above,
  the up branch clamped on both sides and offset by one:
  g = min(gate, limit), u = clamp(up, -limit, limit),
  act = g * sigmoid(alpha g) * (u + 1). Gate and up are one fused GEMM.
- GroupedMoE: `experts` small silu-GLU feed-forwards of which every row
  uses `top`; the router's softmax runs over all experts in fp32, experts
  are cut into `groups` contiguous runs and only the `keep` runs holding the
  highest single scores stay eligible; the chosen scores are renormalised.
  The gate|up matrices of all experts are stacked in ONE [experts * 2ff,
  width] matrix in the checkpoint's own [out, in] layout; the down matrices
  are kept pre-transposed ([in, out] per expert) like the framework's other
  sparse feed-forward (models/llama_family.py MoEMLP). Two execution paths
  as there: up to DENSE_TOKENS rows every expert runs on every row — one
  linear() for all gate|up projections (no per-expert copies of the rows),
  one batched GEMM down — with data-independent shapes, so the step can be
  captured; above it the (row, expert) pairs are sorted by expert and every
  expert runs plain GEMMs on its own segment (its row block of the stacked
  matrix).
- InputScaledMoE: `experts` small silu-GLU feed-forwards of which every row
  uses the `top` with the highest sigmoid (or softmax) score; the score
  multiplies the expert's INPUT, expert(s h), and the results are summed as
  they are; a shared expert of its own size runs on every row. Since
  W (s h) = s (W h), the factor is applied to the gate and up projections
  of h in the activation kernel, in fp32. One matrix holds every gate|up
  projection, per expert and then the shared one, one matrix [width,
  experts * ff + shared_ff] every down projection. Up to DENSE_TOKENS rows
  the step is three GEMMs with data-independent shapes: all gate|up
  projections, an activation whose factor is 0 for the experts a row does
  not use (so their columns are exactly 0), and ONE down GEMM over all
  columns, which sums the chosen experts and the shared one. Above it the
  (row, expert) pairs are sorted by expert as in GroupedMoE.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops
from .mixers import _param, linear, linear_f32


class GLU(nn.Module):
    """W_down act(W_gate x, W_up x); act is one of ops.glu_act's kinds
    ("gelu_tanh": gelu_tanh(gate) * up; "swiglu"; "clamped"). Gate and up
    are one fused GEMM. Without projections of its own it follows the split
    protocol of models/mixers.py (in_spans, core, out_cols), so that a block
    can fuse them with its mixer's."""

    def __init__(self, width: int, ff: int, dtype, act: str = "gelu_tanh",
                 limit: float = 0.0, alpha: float = 1.0,
                 own_projections: bool = True):
        super().__init__()
        self.ff, self.act = ff, act
        self.limit, self.alpha = float(limit), float(alpha)
        self.out_cols = ff
        if own_projections:
            self.gate_up = _param(2 * ff, width, dtype=dtype)
            self.down = _param(width, ff, dtype=dtype)

    def in_spans(self) -> list:
        return [("gate", self.ff, False), ("up", self.ff, False)]

    def extra_weights(self) -> dict:
        return {}

    def weight_map(self) -> dict:
        return {"gate": (self.gate_up, 0), "up": (self.gate_up, self.ff),
                "down": (self.down, 0)}

    def core(self, p, batch, cache, out, out_scale) -> None:
        assert out_scale == 1.0
        ops.glu_act(p, self.act, self.limit, self.alpha, out=out)

    def forward(self, h, batch=None, cache=None) -> torch.Tensor:
        gu = linear(h, self.gate_up)
        return linear(ops.glu_act(gu, self.act, self.limit, self.alpha),
                      self.down)


class ClampedGLU(GLU):
    def __init__(self, width: int, ff: int, limit: float, dtype,
                 alpha: float = 1.702):
        super().__init__(width, ff, dtype, act="clamped", limit=limit,
                         alpha=alpha)


class GroupedMoE(nn.Module):
    DENSE_TOKENS = 256  # see models/llama_family.py MoEMLP.DENSE_TOKENS

    def __init__(self, width: int, experts: int, ff: int, top: int,
                 groups: int, keep: int, dtype):
        super().__init__()
        assert experts % groups == 0 and keep <= groups
        assert top <= keep * (experts // groups)
        self.E, self.ff, self.top = experts, ff, top
        self.groups, self.keep, self.width = groups, keep, width
        self.router = _param(experts, width, dtype=dtype)
        self.w13 = _param(experts * 2 * ff, width, dtype=dtype)
        self.w2 = _param(experts, ff, width, dtype=dtype)

    def weight_map(self) -> dict:
        m = {"router": (self.router, 0)}
        W, ff = self.width, self.ff
        for e in range(self.E):
            m[f"e{e}.gate"] = (self.w13, e * 2 * ff, 0, (ff, W))
            m[f"e{e}.up"] = (self.w13, e * 2 * ff + ff, 0, (ff, W))
            # (param, row, col, shape, expert index, transposed)
            m[f"e{e}.down"] = (self.w2, 0, 0, (W, ff), e, True)
        return m

    def forward(self, h, batch=None, cache=None) -> torch.Tensor:
        T = h.shape[0]
        E, ff, W, k = self.E, self.ff, self.width, self.top
        z = linear_f32(h, self.router)  # fp32 logits
        weights, ids = ops.moe_route_grouped(z, k, self.groups, self.keep)
        if T <= self.DENSE_TOKENS:
            gu = linear(h, self.w13)  # [T, E * 2ff]
            a = ops.glu_act(gu.view(T * E, 2 * ff), "swiglu")
            y = torch.bmm(a.view(T, E, ff).transpose(0, 1), self.w2)
            return ops.moe_mix_seq(y, weights, ids)
        # (row, expert) pairs sorted by expert: every expert runs two plain
        # GEMMs on its own contiguous segment, nothing is padded (one host
        # read of the segment sizes)
        flat = ids.reshape(-1).long()
        order = torch.argsort(flat, stable=True)
        tok = torch.div(order, k, rounding_mode="floor")
        counts = torch.bincount(flat, minlength=E).tolist()
        xs = h[tok]
        gu = torch.empty((T * k, 2 * ff), dtype=h.dtype, device=h.device)
        at = 0
        for e, n in enumerate(counts):
            if n:
                torch.mm(xs[at:at + n],
                         self.w13[e * 2 * ff:(e + 1) * 2 * ff].t(),
                         out=gu[at:at + n])
            at += n
        a = ops.glu_act(gu, "swiglu")
        y = torch.empty((T * k, W), dtype=h.dtype, device=h.device)
        at = 0
        for e, n in enumerate(counts):
            if n:
                torch.mm(a[at:at + n], self.w2[e], out=y[at:at + n])
            at += n
        inv = torch.empty_like(order)
        inv[order] = torch.arange(T * k, device=h.device)
        return ops.moe_mix_rows_seq(y, weights, inv.view(T, k).to(torch.int32))


class InputScaledMoE(nn.Module):
    DENSE_TOKENS = 256  # see models/llama_family.py MoEMLP.DENSE_TOKENS

    def __init__(self, width: int, experts: int, ff: int, top: int, dtype,
                 shared_ff: int = 0, score: str = "sigmoid",
                 renorm: bool = False):
        super().__init__()
        assert 1 <= top <= experts and score in ("sigmoid", "softmax")
        self.E, self.ff, self.top, self.sff = experts, ff, top, int(shared_ff)
        self.width, self.score, self.renorm = width, score, renorm
        self.router = _param(experts, width, dtype=dtype)
        self.w_gu = _param(experts * 2 * ff + 2 * self.sff, width, dtype=dtype)
        self.w_down = _param(width, experts * ff + self.sff, dtype=dtype)

    def weight_map(self) -> dict:
        m = {"router": (self.router, 0)}
        W, ff, E, sff = self.width, self.ff, self.E, self.sff
        for e in range(E):
            m[f"e{e}.gate"] = (self.w_gu, e * 2 * ff)
            m[f"e{e}.up"] = (self.w_gu, e * 2 * ff + ff)
            m[f"e{e}.down"] = (self.w_down, 0, e * ff, (W, ff))
        if sff:
            m["shared.gate"] = (self.w_gu, E * 2 * ff)
            m["shared.up"] = (self.w_gu, E * 2 * ff + sff)
            m["shared.down"] = (self.w_down, 0, E * ff, (W, sff))
        return m

    def forward(self, h, batch=None, cache=None) -> torch.Tensor:
        T = h.shape[0]
        E, ff, sff, k = self.E, self.ff, self.sff, self.top
        z = linear_f32(h, self.router)  # fp32 logits
        if T <= self.DENSE_TOKENS:
            _, _, scale = ops.moe_route_grouped(
                z, k, 1, 1, self.score, self.renorm, matrix=True)
            gu = linear(h, self.w_gu)
            return linear(ops.moe_glu_scaled(gu, scale, E, ff, sff),
                          self.w_down)
        weights, ids = ops.moe_route_grouped(z, k, 1, 1, self.score,
                                             self.renorm)
        # (row, expert) pairs sorted by expert: every expert runs two plain
        # GEMMs on its own contiguous segment (one host read of the sizes)
        flat = ids.reshape(-1).long()
        order = torch.argsort(flat, stable=True)
        tok = torch.div(order, k, rounding_mode="floor")
        counts = torch.bincount(flat, minlength=E).tolist()
        xs = h[tok]
        gu = torch.empty((T * k, 2 * ff), dtype=h.dtype, device=h.device)
        at = 0
        for e, n in enumerate(counts):
            if n:
                torch.mm(xs[at:at + n],
                         self.w_gu[e * 2 * ff:(e + 1) * 2 * ff].t(),
                         out=gu[at:at + n])
            at += n
        a = ops.glu_act(gu, "swiglu", row_scale=weights.reshape(-1)[order])
        y = torch.empty((T * k, self.width), dtype=h.dtype, device=h.device)
        at = 0
        for e, n in enumerate(counts):
            if n:
                torch.mm(a[at:at + n],
                         self.w_down[:, e * ff:(e + 1) * ff].t(),
                         out=y[at:at + n])
            at += n
        inv = torch.empty_like(order)
        inv[order] = torch.arange(T * k, device=h.device)
        shared = None
        if sff:
            sa = ops.glu_act(linear(h, self.w_gu[E * 2 * ff:]), "swiglu")
            shared = linear(sa, self.w_down[:, E * ff:])
        return ops.moe_mix_rows_seq(y, torch.ones_like(weights),
                                    inv.view(T, k).to(torch.int32), shared)


def build_feedforward(mlp: dict, width: int, dtype, arch: str = "") -> nn.Module:
    kind = mlp.get("kind", "dense")
    if arch == "Rivolix":
        if kind != "moe":
            raise ValueError(f"unknown feed-forward kind {kind!r}")
        r = mlp["router"]
        return InputScaledMoE(width, r["experts"], mlp["expert"]["ff"],
                              r["top"], dtype,
                              shared_ff=(mlp.get("shared") or {}).get("ff", 0))
    if kind == "dense":
        return ClampedGLU(width, mlp["ff"], mlp["limit"], dtype)
    if kind == "moe":
        r = mlp["router"]
        return GroupedMoE(width, r["experts"], mlp["expert"]["ff"], r["top"],
                          r["groups"]["count"], r["groups"]["keep"], dtype)
    raise ValueError(f"unknown feed-forward kind {kind!r}")
