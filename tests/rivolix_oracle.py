"""A slow float64 model of the Rivolix design, one function per mechanism,
written from the design's equations and sharing nothing with arks_amd.

A model is (cfg, weights): cfg the dict of config.json, weights a dict of
float64 tensors by checkpoint name. forward() runs one whole sequence and
returns the logits of every position and the residual after every layer;
there is no cache: every position looks back over the full prefix, and a
convolution sees zeros before position 0.

The design in short: x <- x + s1 * mixer(n1(x)) + s2 * ff(n2(x)) with two
RMS norms of the same x (weights stored as offsets from one) and a
per-channel scale on each branch. Mixers: "attention" (two softmax maps per
head over the same values, combined as a difference and re-normed; short
convolutions behind q/k/v; a query temperature that grows with the log of
the position; sigmoid output gate; optionally the keys and values of an
earlier layer) and "attention_2" (values are the raw keys; partial
half-split rotary with ramped frequency scaling, then unit RMS on q and k).
Feed-forward: sigmoid-routed experts whose score scales their INPUT, plus an
always-on shared expert. Logits through the embedding table.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


# ------------------------------------------------------------- small pieces
def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight is the distance from one."""
    return unit_rms(x, eps) * (1.0 + w)


def silu(z):
    return z / (1.0 + torch.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def causal_conv(u, taps_w):
    """u [n, C], taps_w [C, K]: y_t = sum_j taps_w[:, j] u_(t-K+1+j)."""
    n, C = u.shape
    K = taps_w.shape[1]
    pad = torch.cat([torch.zeros(K - 1, C, dtype=F64), u], 0)
    y = torch.zeros(n, C, dtype=F64)
    for j in range(K):
        y += taps_w[:, j] * pad[j:j + n]
    return y


def softmax_attend(q, k, v, scale):
    """q [n, Hq, D], k [n, Hk, D], v [n, Hk, V], Hq a multiple of Hk; query
    head h reads key/value head h // (Hq / Hk); row i sees j <= i."""
    n, Hq, _ = q.shape
    rep = Hq // k.shape[1]
    out = torch.zeros(n, Hq, v.shape[2], dtype=F64)
    for h in range(Hq):
        g = h // rep
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(torch.ones(n, n).triu(1).bool(), -math.inf)
        out[:, h] = torch.softmax(s, -1) @ v[:, g]
    return out


def query_temperature(pos, coef, every):
    """1 + coef ln(floor((p + 1) / every) + 1)."""
    return 1.0 + coef * torch.log(torch.floor((pos.to(F64) + 1.0) / every) + 1.0)


def difference_weight(w, diff):
    return (math.exp(float((w["lq1"] * w["lk1"]).sum()))
            - math.exp(float((w["lq2"] * w["lk2"]).sum())) + diff)


# ------------------------------------------------------------------ mixers
def difference_keys_values(h, w, m):
    """What a difference-attention layer keeps per token: convolved keys
    [n, G, 2, D] and convolved values [n, G, V]."""
    G, D, V = m["kv_heads"], m["dim"], m["vdim"]
    k = causal_conv(h @ w["k"].T, w["k.conv"])
    v = causal_conv(h @ w["v"].T, w["v.conv"])
    return k.view(-1, G, 2, D), v.view(-1, G, V)


def difference_attention(h, w, m, eps, kv=None):
    """kv: (keys, values) of the layer this one borrows from, else its own."""
    n = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv(h @ w["q"].T, w["q.conv"])
    pos = torch.arange(n)
    q = q * query_temperature(pos, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None]
    q = q.view(n, H, 2, D)
    k, v = kv if kv is not None else difference_keys_values(h, w, m)
    a1 = softmax_attend(q[:, :, 0], k[:, :, 0], v, m["scale"])
    a2 = softmax_attend(q[:, :, 1], k[:, :, 1], v, m["scale"])
    lam = difference_weight(w, m["diff"])
    o = unit_rms(a1 - lam * a2, eps) * (1.0 - m["diff"])
    o = o.reshape(n, H * V) * sigmoid(h @ w["g"].T)
    return o @ w["o"].T


def ramped_freqs(rot):
    """Rotary frequencies f_i = base^(-2i/dims), divided by `factor` where
    the wavelength is long, untouched where it is short, blended between;
    and the factor on cos and sin."""
    dims, base = rot["dims"], rot["base"]
    i = torch.arange(dims // 2, dtype=F64)
    f = torch.tensor(float(base), dtype=F64) ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0

    def turn_dim(t):
        return dims * math.log(sc["original"] / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(sc["fast"])), 0)
    hi = min(math.ceil(turn_dim(sc["slow"])), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    f = f / sc["factor"] * ramp + f * (1.0 - ramp)
    return f, 0.1 * math.log(sc["factor"]) + 1.0


def rotate_half(x, pos, rot):
    """x [n, heads, D]: dims i and i + dims/2 of the first `dims` turn by
    pos * f_i; cos and sin carry the scaling's factor."""
    dims = rot["dims"]
    if dims == 0:
        return x
    half = dims // 2
    f, mag = ramped_freqs(rot)
    a = pos.to(F64)[:, None, None] * f[None, None, :]
    c, s = torch.cos(a) * mag, torch.sin(a) * mag
    out = x.clone()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def key_value_attention(h, w, m, eps):
    """attention_2: the values are the keys as projected."""
    n = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    pos = torch.arange(n)
    q = (h @ w["q"].T).view(n, H, D)
    k = (h @ w["k"].T).view(n, G, D)
    v = k.clone()
    q = unit_rms(rotate_half(q, pos, m["rot"]), eps)
    k = unit_rms(rotate_half(k, pos, m["rot"]), eps)
    o = softmax_attend(q, k, v, m["scale"])
    return o.reshape(n, H * D) @ w["o"].T


# ------------------------------------------------------------ feed-forward
def expert(h, w):
    return (silu(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def routed_experts(h, w, mlp, margins=None):
    """Scores sigmoid(W_router h); the `top` highest-scoring experts run on
    score * h and their results are summed as they are; the shared expert
    runs on h. margins (a list) receives, per row, how far the last chosen
    score lies above the first one left out."""
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = sigmoid(h @ w["router"].T)
    if margins is not None and E > top:
        ranked = torch.sort(s, -1, descending=True).values
        margins.append(ranked[:, top - 1] - ranked[:, top])
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=F64)
    chosen = torch.topk(s, top, dim=-1).indices
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            out[t] += expert(s[t, e] * h[t], sub(w, f"e{e}."))
    if mlp.get("shared"):
        out = out + expert(h, sub(w, "shared."))
    return out


# ------------------------------------------------------------------- model
def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, margins=None):
    eps = cfg["norm"]["eps"]
    x = weights["embed"][torch.tensor(tokens)].clone()
    after, kept = [], {}
    for i, spec in enumerate(cfg["layers"]):
        lw = sub(weights, f"l{i}.")
        mw, m = sub(lw, "mix."), spec["mixer"]
        h = offset_norm(x, lw["norm1"], eps)
        if spec["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kept[i] = difference_keys_values(h, mw, m)
            y = difference_attention(h, mw, m, eps, kept[i if src is None else src])
        elif spec["type"] == "attention_2":
            y = key_value_attention(h, mw, m, eps)
        else:
            raise ValueError(spec["type"])
        y = y * lw["ls1"]
        if spec.get("mlp") is not None:
            h2 = offset_norm(x, lw["norm2"], eps)
            y = y + routed_experts(h2, sub(lw, "mlp."), spec["mlp"],
                                   margins) * lw["ls2"]
        x = x + y
        after.append(x.clone())
    xn = offset_norm(x, weights["final.norm"], eps)
    return xn @ weights["embed"].T, after


def clear_choices(cfg, weights, tokens, least=0.008, after=3):
    """Rows at which, and for `after` rows before which, every layer's
    router chooses by a margin of at least `least`: a run in reduced
    precision may choose otherwise at a close call, and then computes
    another function at that row and, through the convolutions' taps and the
    newest keys, near it."""
    margins = []
    forward(cfg, weights, tokens, margins)
    ok = torch.ones(len(tokens), dtype=torch.bool)
    for m in margins:
        ok &= m >= least
    near = ok.clone()
    for d in range(1, after + 1):
        near[d:] &= ok[:-d]
    return near


# ------------------------------------------------------- configs and weights
def moe_spec(experts=6, top=2, ff=24, shared_ff=40):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top},
            "shared": {"ff": shared_ff} if shared_ff else None}


def difference_spec(heads=6, kv_heads=3, dim=8, vdim=12, conv=4, diff=0.2,
                    coef=0.4, every=5, scale=None, kv_from=None, mlp="default"):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "conv": conv, "diff": diff, "q_temp": {"coef": coef, "every": every},
         "scale": dim ** -0.5 if scale is None else scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m,
            "mlp": moe_spec() if mlp == "default" else mlp}


def key_value_spec(heads=6, kv_heads=2, dim=16, rot_dims=8, base=10000.0,
                   scaling="default", scale=None, mlp="default"):
    if scaling == "default":
        scaling = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = scaling
    return {"type": "attention_2", "mixer": {
        "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
        "rot": rot, "scale": dim ** -0.5 if scale is None else scale},
        "mlp": moe_spec() if mlp == "default" else mlp}


def make_config(layers, width=40, vocab=96, eps=1e-5):
    return {"architecture": "Rivolix", "vocab": vocab, "width": width,
            "norm": {"eps": eps}, "layers": list(layers)}


def tensor_shapes(cfg):
    W, out = cfg["width"], {}
    out["embed"] = (cfg["vocab"], W)
    out["final.norm"] = (W,)
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        out[p + "norm1"], out[p + "ls1"] = (W,), (W,)
        H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        if spec["type"] == "attention":
            K = m["conv"]
            out[p + "mix.q"], out[p + "mix.q.conv"] = (H * 2 * D, W), (H * 2 * D, K)
            if m.get("kv_from") is None:
                out[p + "mix.k"], out[p + "mix.k.conv"] = (G * 2 * D, W), (G * 2 * D, K)
                out[p + "mix.v"], out[p + "mix.v.conv"] = (G * V, W), (G * V, K)
            for leaf in ("lq1", "lk1", "lq2", "lk2"):
                out[p + "mix." + leaf] = (D,)
            out[p + "mix.g"], out[p + "mix.o"] = (H * V, W), (W, H * V)
        else:
            out[p + "mix.q"], out[p + "mix.k"] = (H * D, W), (G * D, W)
            out[p + "mix.o"] = (W, H * D)
        mlp = spec.get("mlp")
        if mlp is not None:
            out[p + "norm2"], out[p + "ls2"] = (W,), (W,)
            out[p + "mlp.router"] = (mlp["router"]["experts"], W)
            parts = [(f"e{e}", mlp["expert"]["ff"])
                     for e in range(mlp["router"]["experts"])]
            if mlp.get("shared"):
                parts.append(("shared", mlp["shared"]["ff"]))
            for name, ff in parts:
                out[p + f"mlp.{name}.gate"] = (ff, W)
                out[p + f"mlp.{name}.up"] = (ff, W)
                out[p + f"mlp.{name}.down"] = (W, ff)
    return out


def random_weights(cfg, seed=0):
    """Random weights, rounded to bfloat16 (what a checkpoint holds), as
    float64. Norm offsets, branch scales, taps and the four vectors of the
    difference weight are of order one so that leaving any of them out
    shows."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]

        def rn(std):
            return torch.randn(shape, generator=g, dtype=F64) * std

        if leaf in ("norm1", "norm2", "norm"):
            t = rn(0.3)
        elif leaf in ("ls1", "ls2"):
            t = 0.7 + rn(0.3)
        elif leaf == "conv":
            t = rn(0.6)
        elif leaf in ("lq1", "lk1", "lq2", "lk2"):
            t = rn(0.5)
        elif leaf == "router":
            t = rn(2.0 * shape[-1] ** -0.5)
        elif leaf == "embed":
            t = rn(1.0)
        else:
            t = rn(shape[-1] ** -0.5)
        w[name] = t.to(torch.bfloat16).to(F64)
    return w
