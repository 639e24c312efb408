"""A slow float64 model of the Legalix design, one function per mechanism,
written from the design's equations and sharing nothing with arks_amd.

A model is (cfg, weights): cfg the dict of config.json, weights a dict of
float64 tensors by checkpoint name. forward() runs one whole sequence and
returns the logits of every position and the residual after every layer
run (a looped layer counts once per pass); there is no cache: every
position looks back over the full prefix, the recurrence starts from zero
at position 0.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


# ------------------------------------------------------------- small pieces
def tanh_norm(x, alpha, w, b):
    """Norm without statistics: tanh(alpha x) w + b."""
    return torch.tanh(alpha * x) * w + b


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + z.clamp(min=0.0)


def rotary_freqs(base, dims):
    i = torch.arange(dims // 2, dtype=F64)
    return torch.tensor(float(base), dtype=F64) ** (-2.0 * i / dims)


def rotate(x, pos, base, dims, interleaved):
    """x [n, heads, D]: the first `dims` dims of every head turn by the
    angle pos * base^(-2i/dims); pair i is (i, i + dims/2), or (2i, 2i+1)
    when interleaved. The other dims pass."""
    if dims == 0:
        return x
    half = dims // 2
    a = pos.to(F64)[:, None, None] * rotary_freqs(base, dims)[None, None, :]
    c, s = torch.cos(a), torch.sin(a)
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * c - v * s
        out[..., half:dims] = v * c + u * s
    return out


# ------------------------------------------------------------------ mixers
def attend(q, k, v, scale, size=None, keep=0, cap=0.0, sink=None):
    """q [n, H, D], k [n, G, D], v [n, G, V] -> [n, H, V]. Row i sees j <= i
    with i - j < size or j < keep (size None: every j <= i); scores
    cap * tanh(s / cap) when cap > 0; sink [H]: exp(sink_h) joins the
    denominator."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=F64)
    for i in range(n):
        seen = [j for j in range(i + 1)
                if size is None or i - j < size or j < keep]
        for hh in range(H):
            g = hh // (H // G)
            s = (k[seen, g] @ q[i, hh]) * scale
            if cap > 0:
                s = cap * torch.tanh(s / cap)
            mx = s.max() if sink is None else torch.maximum(s.max(), sink[hh])
            e = torch.exp(s - mx)
            den = e.sum() + (0.0 if sink is None else torch.exp(sink[hh] - mx))
            out[i, hh] = (e / den) @ v[seen, g]
    return out


def window_attention(h, w, m):
    """Grouped-query softmax attention: half-split rotary on the first
    rot.dims dims, tanh-capped scores, row i sees j <= i with
    i - j < mask.size or j < mask.keep_first."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(n)
    q = (h @ w["q"].T).view(n, H, D)
    k = (h @ w["k"].T).view(n, G, D)
    v = (h @ w["v"].T).view(n, G, V)
    q = rotate(q, pos, m["rot"]["base"], m["rot"]["dims"], False)
    k = rotate(k, pos, m["rot"]["base"], m["rot"]["dims"], False)
    out = attend(q, k, v, m["scale"], int(m["mask"]["size"]),
                 int(m["mask"]["keep_first"]), float(m["softcap"]))
    return out.reshape(n, H * V) @ w["o"].T


def latent_attention(h, w, m, eps):
    """Queries and keys/values through low-rank latents; one rotated key
    part shared by every head; causal; a per-head sink in the softmax's
    denominator."""
    n = h.shape[0]
    H, D, R, V, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(n)
    cq = unit_rms(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).view(n, H, D + R)
    q_plain, q_rot = q[..., :D], q[..., D:]
    ckv = h @ w["dkv"].T
    c = unit_rms(ckv[:, :rank], eps) * w["dkv.norm"]
    k_rot = ckv[:, rank:].view(n, 1, R)
    base = m["rot"]["base"]
    q_rot = rotate(q_rot, pos, base, R, True)
    k_rot = rotate(k_rot, pos, base, R, True)[:, 0]
    k_plain = (c @ w["uk"].T).view(n, H, D)
    v = (c @ w["uv"].T).view(n, H, V)
    k = torch.cat([k_plain, k_rot[:, None, :].expand(n, H, R)], -1)
    out = attend(torch.cat([q_plain, q_rot], -1), k, v, m["scale"],
                 sink=w["sink"])
    return out.reshape(n, H * V) @ w["o"].T


def causal_conv(x, taps_w, bias):
    """x [n, C], taps_w [C, taps] (last column: the current row)."""
    n, _ = x.shape
    taps = taps_w.shape[1]
    out = bias[None, :].repeat(n, 1)
    for t in range(n):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                out[t] += taps_w[:, j] * x[src]
    return out


def ssm_scan(x, B, C, dt, rate, skip):
    """x [n, P, V], B and C [n, G, N], dt [n, P], rate and skip [P]:
    S_h <- exp(-rate_h dt) S_h + dt B x_h^T (N x V), y_h = S_h^T C + skip x."""
    n, P, V = x.shape
    G, N = B.shape[1], B.shape[2]
    y = torch.zeros(n, P, V, dtype=F64)
    for hh in range(P):
        g = hh // (P // G)
        S = torch.zeros(N, V, dtype=F64)
        for t in range(n):
            S = torch.exp(-rate[hh] * dt[t, hh]) * S \
                + dt[t, hh] * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S.T @ C[t, g] + skip[hh] * x[t, hh]
    return y


def group_unit_rms(y, parts, eps):
    n, c = y.shape
    return unit_rms(y.view(n, parts, c // parts), eps).reshape(n, c)


def mamba2(h, w, m, eps):
    n = h.shape[0]
    P, V, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = P * V
    p = h @ w["in"].T
    z = p[:, :inner]
    xbc = silu(causal_conv(p[:, inner:2 * inner + 2 * G * N], w["conv"],
                           w["conv.b"]))
    x = xbc[:, :inner].view(n, P, V)
    B = xbc[:, inner:inner + G * N].view(n, G, N)
    C = xbc[:, inner + G * N:].view(n, G, N)
    dt = softplus(p[:, 2 * inner + 2 * G * N:] + w["dt_bias"])  # [n, P]
    y = ssm_scan(x, B, C, dt, torch.exp(w["A_log"]), w["D"])
    y = group_unit_rms(y.reshape(n, inner) * silu(z), m["norm_groups"], eps)
    return (y * w["norm"]) @ w["o"].T


def dense_ff(h, w):
    return (gelu_tanh(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


# ------------------------------------------------------------------- model
def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def layer_runs(cfg):
    """Layer indices in execution order, and the runs before which the loop's
    input projection is applied."""
    L = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(L)), set()
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = list(range(a))
    marks = set()
    for _ in range(times if b > a else 0):
        marks.add(len(order))
        order += list(range(a, b))
    order += list(range(b, L))
    return order, marks


def forward(cfg, weights, tokens):
    eps = cfg["norm"]["eps"]
    mult = cfg["residual_mult"]
    x0 = weights["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    x = x0.clone()
    order, marks = layer_runs(cfg)
    after = []
    for run, i in enumerate(order):
        if run in marks:
            x = torch.cat([x, x0], -1) @ weights["loop.in"].T
        spec = cfg["layers"][i]
        lw = sub(weights, f"l{i}.")
        h = tanh_norm(x, lw["norm1.alpha"], lw["norm1"], lw["norm1.b"])
        mw = sub(lw, "mix.")
        if spec["type"] == "attention":
            y = window_attention(h, mw, spec["mixer"])
        elif spec["type"] == "latent_attention":
            y = latent_attention(h, mw, spec["mixer"], eps)
        elif spec["type"] == "mamba2":
            y = mamba2(h, mw, spec["mixer"], eps)
        else:
            raise ValueError(spec["type"])
        if spec.get("mlp") is not None:
            y = y + dense_ff(h, sub(lw, "mlp."))
        x = x + mult * y
        after.append(x.clone())
    xn = tanh_norm(x, weights["final.norm.alpha"], weights["final.norm"],
                   weights["final.norm.b"])
    return xn @ weights["head"].T, after


# ------------------------------------------------------- configs and weights
def attention_spec(heads=4, kv_heads=2, dim=16, vdim=8, rot_dims=8, size=9,
                   keep_first=2, softcap=5.0, base=10000.0, scale=None, ff=48):
    return {"type": "attention", "mixer": {
        "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
        "rot": {"base": base, "dims": rot_dims},
        "mask": {"size": size, "keep_first": keep_first},
        "scale": dim ** -0.5 if scale is None else scale, "softcap": softcap},
        "mlp": {"kind": "dense", "ff": ff} if ff else None}


def latent_spec(heads=4, dim=8, rot_dim=4, vdim=12, kv_rank=10, q_rank=14,
                base=10000.0, scale=None, ff=48):
    return {"type": "latent_attention", "mixer": {
        "heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
        "kv_rank": kv_rank, "q_rank": q_rank,
        "rot": {"base": base, "dims": rot_dim},
        "scale": (dim + rot_dim) ** -0.5 if scale is None else scale},
        "mlp": {"kind": "dense", "ff": ff} if ff else None}


def mamba2_spec(heads=4, vdim=6, state=5, groups=2, norm_groups=2, conv=3,
                ff=48):
    return {"type": "mamba2", "mixer": {
        "heads": heads, "vdim": vdim, "state": state, "groups": groups,
        "norm_groups": norm_groups, "conv": conv},
        "mlp": {"kind": "dense", "ff": ff} if ff else None}


def make_config(layers, width=40, vocab=96, loop=None, mult=0.7, eps=1e-5,
                embed_scale=3.0):
    cfg = {"architecture": "Legalix", "vocab": vocab, "width": width,
           "embedding": {"scale": embed_scale}, "norm": {"eps": eps},
           "residual_mult": mult, "layers": list(layers)}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def tensor_shapes(cfg):
    W, out = cfg["width"], {}
    out["embed"] = (cfg["vocab"], W)
    out["head"] = (cfg["vocab"], W)
    if cfg.get("loop"):
        out["loop.in"] = (W, 2 * W)
    for name in ("final.norm",):
        out[name], out[name + ".b"], out[name + ".alpha"] = (W,), (W,), ()
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        out[p + "norm1"], out[p + "norm1.b"], out[p + "norm1.alpha"] = (W,), (W,), ()
        if spec["type"] == "attention":
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out[p + "mix.q"], out[p + "mix.k"] = (H * D, W), (G * D, W)
            out[p + "mix.v"], out[p + "mix.o"] = (G * V, W), (W, H * V)
        elif spec["type"] == "latent_attention":
            H, D, R, V = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            out[p + "mix.dq"], out[p + "mix.dq.norm"] = (m["q_rank"], W), (m["q_rank"],)
            out[p + "mix.uq"] = (H * (D + R), m["q_rank"])
            out[p + "mix.dkv"] = (m["kv_rank"] + R, W)
            out[p + "mix.dkv.norm"] = (m["kv_rank"],)
            out[p + "mix.uk"], out[p + "mix.uv"] = (H * D, m["kv_rank"]), (H * V, m["kv_rank"])
            out[p + "mix.sink"], out[p + "mix.o"] = (H,), (W, H * V)
        else:
            P, V, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            ch = P * V + 2 * G * N
            out[p + "mix.in"] = (2 * P * V + 2 * G * N + P, W)
            out[p + "mix.conv"], out[p + "mix.conv.b"] = (ch, m["conv"]), (ch,)
            for leaf in ("dt_bias", "A_log", "D"):
                out[p + "mix." + leaf] = (P,)
            out[p + "mix.norm"], out[p + "mix.o"] = (P * V,), (W, P * V)
        if spec.get("mlp") is not None:
            ff = spec["mlp"]["ff"]
            out[p + "mlp.gate"], out[p + "mlp.up"] = (ff, W), (ff, W)
            out[p + "mlp.down"] = (W, ff)
    return out


def random_weights(cfg, seed=0):
    """Random weights, rounded to bfloat16 (what a checkpoint holds), as
    float64. Sinks, biases and decays are of order one so that leaving any
    of them out shows."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]

        def rn(std):
            return torch.randn(shape, generator=g, dtype=F64) * std

        if name.endswith(".alpha"):
            t = 0.5 + 0.5 * torch.rand(shape, generator=g, dtype=F64)
        elif name.endswith("norm1") or name.endswith("final.norm") or leaf == "norm":
            t = 1.0 + rn(0.2)
        elif leaf == "b":
            t = rn(0.2)
        elif leaf == "embed":
            t = rn(1.0 / cfg["embedding"]["scale"])
        elif leaf == "in" and name == "loop.in":
            t = rn((shape[1] / 2) ** -0.5)
        elif leaf == "sink":
            t = rn(1.0) + 1.0
        elif leaf == "A_log":
            t = torch.log(0.3 + 3.0 * torch.rand(shape, generator=g, dtype=F64))
        elif leaf == "dt_bias":
            t = rn(0.7) - 1.0
        elif leaf == "D":
            t = rn(0.5)
        elif leaf == "conv":
            t = rn(0.5)
        else:
            t = rn(shape[-1] ** -0.5)
        w[name] = t.to(torch.bfloat16).to(F64)
    return w
