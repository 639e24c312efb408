"""Legalix through the engine, and its mechanisms one by one, against the
plain float64 model of tests/legalix_oracle.py.

Engine cases write a small random checkpoint, build an engine on it and
replay a step plan with the product's trace replay (the scheduler's pages
and state slots, the runner's batches, the model's kernels); op cases drive
single ops with inputs made so that a fault shows (one key that must win on
either side of a window's edge, among the kept first keys, far back, at a
page border; a sink that takes all the weight; decays of 0 and 1). CPU
cases run the reference ops, gpu-marked ones the HIP kernels in float32 and
bfloat16.
"""

import io
import json
import os

import numpy as np
import pytest
import torch

import legalix_oracle as O

CASES = [
    pytest.param("cpu", "float32", id="cpu-f32"),
    pytest.param("cuda", "float32", id="gpu-f32", marks=pytest.mark.gpu),
    pytest.param("cuda", "bfloat16", id="gpu-bf16", marks=pytest.mark.gpu),
]
TOL = {"float32": 2e-4, "bfloat16": 6e-2}
TDT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64

A, L, M = O.attention_spec, O.latent_spec, O.mamba2_spec


# ------------------------------------------------------------------ helpers
def write_checkpoint(path, cfg, seed=0):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    w = O.random_weights(cfg, seed)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in w.items()},
              os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    return w


def make_engine(path, device, dtype, max_tokens=256, **kw):
    from arks_amd.config import EngineConfig
    from arks_amd.engine import LLMEngine

    cfg = EngineConfig(model_path=str(path), device=device, dtype=dtype,
                       kv_cache_blocks=-(-max_tokens // 16), max_num_seqs=4,
                       max_model_len=max_tokens, max_num_batched_tokens=max_tokens,
                       enable_prefix_caching=False, **kw)
    return LLMEngine(cfg)


def replay(engine, tmp_path, steps):
    """steps: lists of (request id, tokens, end?); logits of every token.
    Returns {id: [n_tokens, vocab]}."""
    from arks_amd.engine.trace import replay as trace_replay

    out = tmp_path / "out"
    out.mkdir(exist_ok=True)
    lines = [json.dumps({
        "step": n,
        "entries": [{"id": i, "tokens": t, "want": list(range(len(t)))}
                    for i, t, _ in step],
        "end": [i for i, _, e in step if e]}) for n, step in enumerate(steps)]
    trace_replay(engine, lines, str(out), log=io.StringIO())
    got = {}
    V = engine.model_cfg.vocab_size
    for n, step in enumerate(steps):
        arr = np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, V)
        at = 0
        for i, t, _ in step:
            got.setdefault(i, []).append(arr[at:at + len(t)])
            at += len(t)
    return {i: np.concatenate(v) for i, v in got.items()}


def rel_err(got, want):
    """Largest row error over the rms of all logits."""
    want = want.numpy() if isinstance(want, torch.Tensor) else want
    d = got - want
    return float((np.sqrt((d ** 2).mean(-1)) / np.sqrt((want ** 2).mean())).max())


def portions(tokens, sizes):
    out, at, k = [], 0, 0
    while at < len(tokens):
        n = sizes[k % len(sizes)]
        out.append(tokens[at:at + n])
        at += n
        k += 1
    return out


def toks(n, vocab=96, seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def oracle_logits(cfg, w, t):
    return O.forward(cfg, w, t)[0]


# --------------------------------------------------- the model in the engine
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("spec", [A(), A(ff=0), L(), L(ff=0), M(), M(ff=0)],
                         ids=["attention", "attention-alone", "latent",
                              "latent-alone", "mamba2", "mamba2-alone"])
def test_one_layer(tmp_path, device, dtype, spec):
    cfg = O.make_config([spec])
    w = write_checkpoint(tmp_path / "m", cfg)
    t = toks(45)
    eng = make_engine(tmp_path / "m", device, dtype)
    got = replay(eng, tmp_path, [[("a", t, True)]])["a"]
    assert rel_err(got, oracle_logits(cfg, w, t)) < TOL[dtype]


@pytest.mark.parametrize("device,dtype", CASES)
def test_residual_after_every_layer_run(tmp_path, device, dtype):
    """Four layers of which the middle two run three passes: eight runs,
    each pass with its own pages and state, the loop's input projection in
    front of every pass."""
    cfg = O.make_config([M(), A(), L(ff=0), M(ff=0)], loop=(1, 3, 3))
    w = write_checkpoint(tmp_path / "m", cfg)
    t = toks(21)
    _, after = O.forward(cfg, w, t)
    assert len(after) == 8
    eng = make_engine(tmp_path / "m", device, dtype)
    seen = {}
    eng.runner.model.residual_tap = lambda i, x: seen.__setitem__(
        i, x.detach().clone().float().cpu())
    replay(eng, tmp_path, [[("a", t, True)]])
    assert sorted(seen) == list(range(8))
    for i, want in enumerate(after):
        err = (seen[i].double() - want).abs().max() / want.abs().max()
        assert float(err) < (1e-4 if dtype == "float32" else 4e-2), i


def model_config():
    """All three mixers, the window (9, first 2 kept) and the conv history
    crossed many times by short portions, a loop over two of four layers."""
    return O.make_config([M(), A(), L(), A(size=5, keep_first=0, ff=0)],
                         loop=(1, 3, 2))


@pytest.mark.parametrize("device,dtype", CASES)
def test_prefill_against_decode_and_portions(tmp_path, device, dtype):
    cfg = model_config()
    w = write_checkpoint(tmp_path / "m", cfg)
    t = toks(70)
    want = oracle_logits(cfg, w, t)
    for name, plan in {
        "decode": [t[:9]] + [[x] for x in t[9:]],
        "small": portions(t, [2, 3, 5, 2, 7]),
        "odd": portions(t, [13, 1, 2, 17]),
        "tokens": [[x] for x in t[:40]],
    }.items():
        eng = make_engine(tmp_path / "m", device, dtype)
        steps = [[("a", p, False)] for p in plan]
        got = replay(eng, tmp_path, steps)["a"]
        assert rel_err(got, want[:len(got)]) < TOL[dtype], name


@pytest.mark.parametrize("device,dtype", CASES)
def test_mixed_batches_and_reuse(tmp_path, device, dtype):
    """Unequal requests side by side, portions beside single tokens; more
    requests than state slots over time and a pool just large enough, so
    pages and slots are given back and taken again."""
    cfg = model_config()
    w = write_checkpoint(tmp_path / "m", cfg)
    reqs = {c: toks(n, seed=s) for c, n, s in
            [("a", 61, 1), ("b", 18, 2), ("c", 33, 3), ("d", 5, 4),
             ("e", 47, 5), ("f", 29, 6), ("g", 40, 7)]}
    want = {c: oracle_logits(cfg, w, t) for c, t in reqs.items()}
    at = {c: 0 for c in reqs}
    live, waiting, steps = [], list(reqs), []
    sizes = [7, 1, 2, 16, 1, 1, 3, 11]
    k = 0
    while live or waiting:
        while waiting and len(live) < 4 and \
                sum(-(-len(reqs[c]) // 16) for c in live + waiting[:1]) <= 12:
            live.append(waiting.pop(0))
        step = []
        for c in list(live):
            if (k + ord(c)) % 5 == 0 and len(live) > 1:
                k += 1
                continue  # this request sits the step out
            n = min(sizes[k % len(sizes)], len(reqs[c]) - at[c])
            k += 1
            part = reqs[c][at[c]:at[c] + n]
            at[c] += n
            done = at[c] == len(reqs[c])
            step.append((c, part, done))
            if done:
                live.remove(c)
        if step:
            steps.append(step)
    eng = make_engine(tmp_path / "m", device, dtype, max_tokens=192)
    got = replay(eng, tmp_path, steps)
    for c in reqs:
        assert got[c].shape[0] == len(reqs[c])
        assert rel_err(got[c], want[c]) < TOL[dtype], c


@pytest.mark.parametrize("device,dtype", CASES)
def test_long_decode(tmp_path, device, dtype):
    cfg = O.make_config([M(), A(size=24, keep_first=3), L()])
    w = write_checkpoint(tmp_path / "m", cfg)
    t = toks(150)
    want = oracle_logits(cfg, w, t)
    eng = make_engine(tmp_path / "m", device, dtype)
    steps = [[("a", t[:5], False)]] + [[("a", [x], False)] for x in t[5:]]
    got = replay(eng, tmp_path, steps)["a"]
    assert rel_err(got, want) < TOL[dtype]


OTHER_SIZES = {
    "no-loop-mult-one": dict(layers=[A(), M()], mult=1.0, embed_scale=1.0),
    "loop-of-one-pass": dict(layers=[L(), M()], loop=(0, 2, 1)),
    "loop-of-one-layer": dict(layers=[A(), M(), L()], loop=(1, 2, 3)),
    "loop-at-the-end": dict(layers=[M(ff=0), A()], loop=(1, 2, 2)),
    "loop-of-no-pass": dict(layers=[A(), M(), L()], loop=(1, 2, 0)),
    "one-kv-head": dict(layers=[A(heads=6, kv_heads=1, dim=8, vdim=12)]),
    "all-kv-heads": dict(layers=[A(heads=3, kv_heads=3, dim=12, vdim=12,
                                   rot_dims=12)]),
    "no-kept-window-one": dict(layers=[A(size=1, keep_first=0)]),
    "window-above-prompt": dict(layers=[A(size=500, keep_first=0)]),
    "kept-above-window": dict(layers=[A(size=3, keep_first=11)]),
    "tight-cap": dict(layers=[A(softcap=0.3, scale=2.0)]),
    "rotary-two-dims": dict(layers=[A(rot_dims=2, base=7.0)]),
    "latent-one-head": dict(layers=[L(heads=1, dim=6, rot_dim=2, vdim=5,
                                      kv_rank=7, q_rank=3)]),
    "latent-wide": dict(layers=[L(heads=3, dim=4, rot_dim=12, vdim=4,
                                  kv_rank=20, q_rank=9, base=50.0)], width=24),
    "mamba2-one-group": dict(layers=[M(heads=3, groups=1, norm_groups=1,
                                       state=9, vdim=10, conv=2)]),
    "mamba2-group-per-head": dict(layers=[M(heads=4, groups=4, norm_groups=8,
                                            state=3, vdim=4, conv=5)]),
    "odd-everything": dict(layers=[
        M(heads=2, vdim=7, state=5, groups=1, norm_groups=2, conv=3, ff=50),
        A(heads=3, kv_heads=1, dim=10, vdim=6, rot_dims=4, ff=0),
        L(heads=2, dim=6, rot_dim=2, vdim=3, kv_rank=5, q_rank=7, ff=37)],
        width=44, vocab=97, loop=(0, 3, 2)),
    "mamba2-no-conv-history": dict(layers=[M(conv=1, state=20, vdim=70,
                                             heads=2, groups=1,
                                             norm_groups=5)]),
}


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", list(OTHER_SIZES))
def test_other_sizes(tmp_path, device, dtype, name):
    cfg = O.make_config(**OTHER_SIZES[name])
    w = write_checkpoint(tmp_path / "m", cfg, seed=3)
    t = toks(38, vocab=cfg["vocab"], seed=9)
    want = oracle_logits(cfg, w, t)
    eng = make_engine(tmp_path / "m", device, dtype)
    steps = [[("a", p, False)] for p in portions(t, [11, 2, 1, 6])]
    got = replay(eng, tmp_path, steps)["a"]
    assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("device,dtype", [
    pytest.param("cuda", "float32", id="gpu-f32", marks=pytest.mark.gpu),
    pytest.param("cuda", "bfloat16", id="gpu-bf16", marks=pytest.mark.gpu)])
def test_matrix_core_sizes(tmp_path, device, dtype, monkeypatch):
    """Head sizes the matrix-core attention kernels are built for, prompts
    across 64-row tile edges and chunk edges of the recurrent prefill, a
    window that ends inside a key tile."""
    cfg = O.make_config(
        [M(heads=4, vdim=64, state=16, groups=2, norm_groups=2, conv=4),
         A(heads=4, kv_heads=2, dim=64, vdim=64, rot_dims=32, size=70,
           keep_first=5),
         L(heads=4, dim=32, rot_dim=32, vdim=32, kv_rank=64, q_rank=48)],
        width=64)
    w = write_checkpoint(tmp_path / "m", cfg)
    t = toks(200, seed=11)
    want = oracle_logits(cfg, w, t)
    from arks_amd import ops
    from arks_amd.models.mixers import LatentAttention

    monkeypatch.setattr(LatentAttention, "EXPAND_ROWS", 100)
    monkeypatch.setattr(ops, "MAMBA2_CHUNK", 64)  # 130 rows: three chunks
    eng = make_engine(tmp_path / "m", device, dtype, max_tokens=512)
    plan = [t[:130], t[130:131], t[131:197], t[197:198], t[198:199], t[199:]]
    got = replay(eng, tmp_path, [[("a", p, False)] for p in plan])["a"]
    assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("device,dtype", [
    pytest.param("cuda", "float32", id="gpu-f32", marks=pytest.mark.gpu),
    pytest.param("cuda", "bfloat16", id="gpu-bf16", marks=pytest.mark.gpu)])
def test_matrix_core_sizes_in_mixed_batches(tmp_path, device, dtype, monkeypatch):
    """The matrix-core kernels with several sequences in a step: prompt
    tiles of unequal requests, single rows beside portions, windows and
    kept keys inside key tiles, both latent forms, a looped layer pair,
    pages and slots taken again by later requests."""
    from arks_amd.models.mixers import LatentAttention

    monkeypatch.setattr(LatentAttention, "EXPAND_ROWS", 48)
    cfg = O.make_config(
        [M(heads=4, vdim=64, state=16, groups=2, norm_groups=2, conv=4),
         A(heads=4, kv_heads=2, dim=64, vdim=64, rot_dims=32, size=40,
           keep_first=3),
         L(heads=4, dim=32, rot_dim=32, vdim=32, kv_rank=64, q_rank=48)],
        width=64, loop=(1, 3, 2))
    w = write_checkpoint(tmp_path / "m", cfg)
    reqs = {c: toks(n, seed=s) for c, n, s in
            [("a", 150, 1), ("b", 70, 2), ("c", 101, 3), ("d", 9, 4),
             ("e", 66, 5)]}
    want = {c: oracle_logits(cfg, w, t) for c, t in reqs.items()}
    at = {c: 0 for c in reqs}
    live, waiting, steps = [], list(reqs), []
    sizes = [67, 1, 1, 50, 2, 1, 33, 1, 90]
    k = 0
    while live or waiting:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        step = []
        for c in list(live):
            n = min(sizes[k % len(sizes)], len(reqs[c]) - at[c])
            k += 1
            step.append((c, reqs[c][at[c]:at[c] + n], at[c] + n == len(reqs[c])))
            at[c] += n
            if at[c] == len(reqs[c]):
                live.remove(c)
        steps.append(step)
    eng = make_engine(tmp_path / "m", device, dtype, max_tokens=352)
    got = replay(eng, tmp_path, steps)
    for c in reqs:
        assert rel_err(got[c], want[c]) < TOL[dtype], c


@pytest.mark.parametrize("device,dtype", CASES)
def test_latent_attention_per_head_form(tmp_path, device, dtype, monkeypatch):
    """Steps with a long portion up-project the context's latents into
    per-head keys and values instead of moving the up-projections to the
    query: same logits, portions of both kinds in one replay, a second
    request beside it."""
    from arks_amd.models.mixers import LatentAttention

    monkeypatch.setattr(LatentAttention, "EXPAND_ROWS", 6)
    cfg = O.make_config([L(), L(heads=2, dim=12, rot_dim=6, vdim=5, kv_rank=9,
                               q_rank=8, ff=0)], loop=(0, 2, 2))
    w = write_checkpoint(tmp_path / "m", cfg)
    ta, tb = toks(60, seed=2), toks(41, seed=3)
    eng = make_engine(tmp_path / "m", device, dtype)
    steps = [[("a", ta[:21], False)], [("a", ta[21:24], False), ("b", tb[:30], False)],
             [("a", ta[24:43], False), ("b", tb[30:31], False)],
             [("a", ta[43:], True), ("b", tb[31:], True)]]
    got = replay(eng, tmp_path, steps)
    assert rel_err(got["a"], oracle_logits(cfg, w, ta)) < TOL[dtype]
    assert rel_err(got["b"], oracle_logits(cfg, w, tb)) < TOL[dtype]


@pytest.mark.parametrize("device,dtype", CASES)
def test_greedy_generation(tmp_path, device, dtype):
    """LLMEngine.generate (scheduler, sampler, captured decode steps on the
    GPU) picks the oracle's tokens; three prompts share the batch."""
    from arks_amd.engine import SamplingParams

    cfg = model_config()
    w = write_checkpoint(tmp_path / "m", cfg)
    prompts = [toks(19, seed=4), toks(3, seed=5), toks(34, seed=6)]
    eng = make_engine(tmp_path / "m", device, dtype)
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True,
                                                temperature=0.0))
    for p, o in zip(prompts, outs):
        seq = list(p)
        for tok in o:
            logits = oracle_logits(cfg, w, seq)[-1]
            top2 = torch.topk(logits, 2).values
            if float(top2[0] - top2[1]) > (1e-3 if dtype == "float32" else 0.15):
                assert tok == int(logits.argmax()), (len(seq), tok)
            seq.append(tok)


# ------------------------------------------------------- mechanisms alone
def _dev(device):
    return torch.device(device)


def _rounded(x, dtype):
    """What the op will see: the value after rounding to its row dtype."""
    return x.to(TDT[dtype]).to(F64)


class Paged:
    """A sequence's keys and values in pages handed out in a scrambled
    order, and steps of rows over them through ops.attention_sink_paged.
    shared: the value is the first V columns of the key's row (one cache)."""

    def __init__(self, dev, dtype, G, D, V, n, shared=False):
        self.dev, self.dt, self.shared = dev, TDT[dtype], shared
        nblk = -(-n // 16)
        g = torch.Generator().manual_seed(7)
        self.table = torch.randperm(nblk + 3, generator=g)[:nblk].to(torch.int32)
        self.k = torch.full((nblk + 3, G, 16, D), 9.0, dtype=self.dt, device=dev)
        self.v = (self.k[..., :V] if shared else
                  torch.full((nblk + 3, G, 16, V), 9.0, dtype=self.dt, device=dev))
        self.len = 0

    def step(self, q, k, v, **kw):
        """Rows [len, len + n) join the cache; returns their outputs."""
        from arks_amd import ops

        n = q.shape[0]
        pos = torch.arange(self.len, self.len + n)
        blk, off = self.table[pos // 16].long(), pos % 16
        self.k[blk.to(self.dev), :, off.to(self.dev)] = k.to(self.dt).to(self.dev)
        if not self.shared:
            self.v[blk.to(self.dev), :, off.to(self.dev)] = v.to(self.dt).to(self.dev)
        self.len += n
        i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=self.dev)
        out = ops.attention_sink_paged(
            q.to(self.dt).to(self.dev), self.k, self.v,
            self.table[None].to(self.dev), i32([self.len]), i32([0, n]),
            i32([0] * n), kw.pop("scale"), False, None, True, n,
            pos.to(self.dev), **kw)
        return out.double().cpu()


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("decode", [False, True], ids=["prompt", "decoded"])
def test_window_and_kept_edges_decide(device, dtype, decode):
    """Among hundreds of keys one gets a huge score. Where it sits decides
    what the last row returns: the oldest key of the window, the last of the
    kept first keys, a key on either side of a page border inside the
    window and the row's own key give their value; the newest key behind
    the window and the first key that is not kept are invisible."""
    dev = _dev(device)
    H, G, D, V = 4, 2, 16, 8
    size, keep, n = 40, 5, 300
    i = n - 1
    g = torch.Generator().manual_seed(5)
    base_k = torch.randn(n, G, D, generator=g, dtype=F64) * 0.1
    v = _rounded(torch.randn(n, G, V, generator=g, dtype=F64), dtype)
    e = torch.zeros(D, dtype=F64)
    e[3] = 1.0
    for hot, visible in [(i - size + 1, True), (i - size, False),
                         (keep - 1, True), (keep, False), (0, True),
                         (271, True), (272, True), (150, False), (i, True)]:
        k = base_k.clone()
        k[hot, :] = 40.0 * e
        k = _rounded(k, dtype)
        q = torch.zeros(n, H, D, dtype=F64)
        q[i, :] = 8.0 * e
        want = O.attend(q, k, v, 0.5, size, keep)[i]
        assert torch.allclose(want[0], v[hot, 0], atol=1e-6) == visible, hot
        pg = Paged(dev, dtype, G, D, V, n)
        cut = n - 1 if decode else n - 37
        kw = dict(scale=0.5, window=size, keep_first=keep)
        pg.step(q[:cut], k[:cut], v[:cut], **kw)
        got = pg.step(q[cut:], k[cut:], v[cut:], **kw)[-1]
        tol = 1e-4 if dtype == "float32" else 2e-2
        assert torch.allclose(got, want, atol=tol, rtol=tol), (hot, visible)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("decode", [False, True], ids=["prompt", "decoded"])
def test_far_key_and_sink_over_shared_rows(device, dtype, decode):
    """Latent attention's cache: the value is the leading part of the key's
    row. One key far back (position 2 of 400, and one just before a page
    border) must win; with a sink far above every score the row returns
    next to nothing; with a sink at the level of the winning score, half."""
    dev = _dev(device)
    H, D, V, n = 3, 24, 16, 400
    i = n - 1
    g = torch.Generator().manual_seed(6)
    base = torch.randn(n, 1, D, generator=g, dtype=F64) * 0.1
    e = torch.zeros(D, dtype=F64)
    e[20] = 1.0  # a column behind the value part
    q = torch.zeros(n, H, D, dtype=F64)
    q[i, :] = 6.0 * e
    for hot in (2, 15, 399 - 64):
        k = base.clone()
        k[hot, 0, 20] = 10.0  # score 60 * scale
        k = _rounded(k, dtype)
        v = k[..., :V]
        for sink, share in [(None, 1.0), ([-50.0] * H, 1.0),
                            ([30.0, 30.0, 90.0], None)]:
            sk = None if sink is None else torch.tensor(sink, dtype=F64)
            want = O.attend(q, k, v, 0.5, sink=sk)[i]
            if share is not None:
                assert torch.allclose(want[0], v[hot, 0] * share, atol=1e-5)
            else:
                assert torch.allclose(want[0], v[hot, 0] * 0.5, atol=1e-3)
                assert float(want[2].abs().max()) < 1e-6
            pg = Paged(dev, dtype, 1, D, V, n, shared=True)
            cut = n - 1 if decode else n - 70
            kw = dict(scale=0.5, sink_w=None if sk is None
                      else sk.float().to(dev))
            pg.step(q[:cut], k[:cut], None, **dict(kw))
            got = pg.step(q[cut:], k[cut:], None, **dict(kw))[-1]
            tol = 1e-4 if dtype == "float32" else 2e-2
            assert torch.allclose(got, want, atol=tol, rtol=tol), (hot, sink)


@pytest.mark.parametrize("device,dtype", CASES)
def test_capped_scores(device, dtype):
    """Two keys whose raw scores are 40 and 80 end up next to the cap both
    and share the weight almost evenly; without the cap the larger one
    takes everything."""
    dev = _dev(device)
    H, G, D, V, n = 2, 1, 8, 8, 20
    e = torch.zeros(D, dtype=F64)
    e[1] = 1.0
    k = torch.zeros(n, G, D, dtype=F64)
    k[4, 0], k[11, 0] = 10.0 * e, 20.0 * e
    g = torch.Generator().manual_seed(2)
    v = _rounded(torch.randn(n, G, V, generator=g, dtype=F64), dtype)
    q = torch.zeros(n, H, D, dtype=F64)
    q[n - 1, :] = 4.0 * e
    want = O.attend(q, k, v, 1.0, cap=5.0)[n - 1]
    plain = O.attend(q, k, v, 1.0)[n - 1]
    assert torch.allclose(plain[0], v[11, 0], atol=1e-6)
    assert not torch.allclose(want[0], v[11, 0], atol=0.05)
    pg = Paged(dev, dtype, G, D, V, n)
    got = pg.step(q, k, v, scale=1.0, softcap=5.0)[-1]
    tol = 1e-4 if dtype == "float32" else 2e-2
    assert torch.allclose(got, want, atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", ["bfloat16"])
@pytest.mark.gpu
@pytest.mark.parametrize("D,V,H,G,shared", [
    (64, 64, 4, 2, False), (128, 128, 8, 1, False), (128, 64, 2, 2, False),
    (96, 96, 3, 1, False), (96, 64, 5, 1, True), (320, 256, 16, 1, True),
    (576, 512, 16, 1, True), (576, 512, 128, 1, True), (64, 32, 4, 4, False),
    (192, 128, 4, 4, False), (96, 64, 2, 1, False)])
def test_masked_matrix_core_kernels_against_general(dtype, D, V, H, G, shared):
    """Random rows through the matrix-core kernels (prompt tiles, single
    rows) and through the general kernel: window edges inside key tiles,
    kept keys, caps and sinks, three unequal sequences in one step."""
    from arks_amd import ops

    dev = torch.device("cuda")
    g = torch.Generator().manual_seed(D + V)
    lens, news = [150, 67, 261], [150, 3, 70]
    nblk = sum(-(-n // 16) for n in lens)
    perm = torch.randperm(nblk, generator=g).to(torch.int32)
    table = torch.zeros(3, max(-(-n // 16) for n in lens), dtype=torch.int32)
    at = 0
    for s, n in enumerate(lens):
        nb = -(-n // 16)
        table[s, :nb] = perm[at:at + nb]
        at += nb
    kc = (torch.randn(nblk, G, 16, D, generator=g) * 0.5).to(torch.bfloat16).to(dev)
    vc = kc[..., :V] if shared else \
        torch.randn(nblk, G, 16, V, generator=g).to(torch.bfloat16).to(dev)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    for single in (False, True):
        rows = [1, 1, 1] if single else news
        T = sum(rows)
        q = torch.randn(T, H, D, generator=g).to(torch.bfloat16).to(dev)
        cu = [0]
        for r in rows:
            cu.append(cu[-1] + r)
        tseq = sum(([s] * r for s, r in enumerate(rows)), [])
        for kw in [dict(window=37, keep_first=6, softcap=4.0),
                   dict(sink_w=torch.tensor([0.5 * h - 1 for h in range(H)],
                                            device=dev)),
                   dict(window=100, keep_first=0)]:
            res = []
            for fast in (True, False):
                ops.use_masked_mfma = fast
                try:
                    out = torch.zeros(T, H * V + 8, dtype=torch.bfloat16,
                                      device=dev)[:, :H * V].unflatten(-1, (H, V))
                    ops.attention_sink_paged(
                        q, kc, vc, table.to(dev), i32(lens), i32(cu), i32(tseq),
                        D ** -0.5, False, None, True, max(rows), None,
                        out=out, out_scale=0.5, **kw)
                    res.append(out.float().cpu())
                finally:
                    ops.use_masked_mfma = True
            assert torch.allclose(res[0], res[1], atol=2e-2, rtol=2e-2), (single, kw)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("P,V,N,G", [(4, 6, 5, 2), (2, 70, 20, 1), (3, 16, 130, 3)])
def test_mamba2_scan_portions(device, dtype, P, V, N, G):
    """The recurrence over portions of 1, 2, 70 and 65 rows (chunk-parallel
    above 64 rows on the GPU) into a junk-filled slot, against the plain
    scan of the whole sequence; heads with decay next to 1 and next to 0."""
    from arks_amd import ops

    dev = _dev(device)
    dt_ = TDT[dtype]
    n = 138
    g = torch.Generator().manual_seed(N)
    r = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    xbc = _rounded(r(n, P * V + 2 * G * N) * 0.7, dtype)
    dt_raw = _rounded(r(n, P), dtype)
    bias = r(P).float().double()
    rate = torch.exp(r(P)).float().double()
    rate[0], rate[-1] = 1e-6, 60.0
    skip = r(P).float().double()
    want = O.ssm_scan(
        xbc[:, :P * V].view(n, P, V), xbc[:, P * V:P * V + G * N].view(n, G, N),
        xbc[:, P * V + G * N:].view(n, G, N), O.softplus(dt_raw + bias), rate,
        skip).reshape(n, P * V)
    state = torch.full((3, P, N, V), 7.0, dtype=torch.float32, device=dev)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    got, at = [], 0
    for rows in (1, 2, 70, 65):
        chunks = (ops.scan_chunks([rows], dev, 32)
                  if dev.type == "cuda" and rows > 32 else None)
        got.append(ops.mamba2_scan(
            xbc[at:at + rows].to(dt_).to(dev), dt_raw[at:at + rows].to(dt_).to(dev),
            bias.float().to(dev), rate.float().to(dev), skip.float().to(dev),
            state, i32([0, rows]), i32([at + rows]), i32([1]), P, V, N, G,
            rows, chunks).double().cpu())
        at += rows
    got = torch.cat(got)
    err = (got - want).abs().max() / want.abs().max()
    assert float(err) < (2e-5 if dtype == "float32" else 1e-4)
    assert float(state[0].min()) == 7.0 and float(state[2].max()) == 7.0


@pytest.mark.parametrize("device,dtype", CASES)
def test_row_ops(device, dtype):
    """The tanh norm with its residual add and strided copy, the gated group
    norm, the GELU GLU into a strided output, and latent attention's row
    work, each against the oracle's formula."""
    from arks_amd import ops

    dev = _dev(device)
    dt_ = TDT[dtype]
    tol = 1e-5 if dtype == "float32" else 2e-2
    g = torch.Generator().manual_seed(3)
    r = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    T, C = 9, 40
    x, y = r(T, C).float().double(), _rounded(r(T, C), dtype)
    w, b = r(C).float().double(), r(C).float().double()
    alpha = torch.tensor(0.7, dtype=F64).float().double()
    xd = x.float().to(dev)
    wide = torch.zeros(T, 2 * C, dtype=dt_, device=dev)
    h = ops.residual_tanh_norm(xd, y.to(dt_).to(dev), 0.3, alpha.float().to(dev),
                               w.float().to(dev), b.float().to(dev), dt_,
                               xa=wide[:, C:])
    assert torch.allclose(xd.double().cpu(), x + 0.3 * y, atol=1e-6)
    assert torch.allclose(h.double().cpu(), O.tanh_norm(x + 0.3 * y, alpha, w, b),
                          atol=tol, rtol=tol)
    assert torch.allclose(wide[:, C:].double().cpu(), x + 0.3 * y, atol=tol, rtol=tol)
    assert float(wide[:, :C].abs().max()) == 0.0
    # gated group norm into a column slice
    z = _rounded(r(T, C), dtype)
    yy = r(T, C).float().double()
    out = torch.zeros(T, C + 8, dtype=dt_, device=dev)
    ops.gate_group_norm(yy.float().to(dev), z.to(dt_).to(dev), w.float().to(dev),
                        5, 1e-5, out[:, 8:])
    want = O.group_unit_rms(yy * O.silu(z), 5, 1e-5) * w
    assert torch.allclose(out[:, 8:].double().cpu(), want, atol=tol, rtol=tol)
    # GELU GLU into a column slice
    gu = _rounded(r(T, 2 * C), dtype)
    out = torch.zeros(T, C + 8, dtype=dt_, device=dev)
    ops.glu_act(gu.to(dt_).to(dev), "gelu_tanh", out=out[:, :C])
    assert torch.allclose(out[:, :C].double().cpu(),
                          O.gelu_tanh(gu[:, :C]) * gu[:, C:], atol=tol, rtol=tol)
    # latent rows: normed query latent; normed latent and turned key part
    # in the row's place of the cache
    Rq, Rk, P = 14, 10, 3
    p = _rounded(r(T, Rq + Rk + 2 * P), dtype)
    qw, kw = r(Rq).float().double(), r(Rk).float().double()
    pos = torch.arange(5, 5 + T)
    freq = O.rotary_freqs(100.0, 2 * P)
    cache = torch.zeros(4, 1, 16, Rk + 2 * P, dtype=dt_, device=dev)
    slots = torch.arange(20, 20 + T)
    pd = p.to(dt_).to(dev)
    cq = ops.latent_prepare(pd[:, :Rq], pd[:, Rq:], qw.float().to(dev),
                            kw.float().to(dev), 1e-5, pos.to(dev),
                            freq.float().to(dev), cache, slots.to(dev))
    assert torch.allclose(cq.double().cpu(), O.unit_rms(p[:, :Rq], 1e-5) * qw,
                          atol=tol, rtol=tol)
    rows = cache.view(-1, Rk + 2 * P)[20:20 + T].double().cpu()
    assert torch.allclose(rows[:, :Rk], O.unit_rms(p[:, Rq:Rq + Rk], 1e-5) * kw,
                          atol=tol, rtol=tol)
    turned = O.rotate(p[:, None, Rq + Rk:], pos, 100.0, 2 * P, True)[:, 0]
    assert torch.allclose(rows[:, Rk:], turned, atol=tol, rtol=tol)
    assert float(cache.view(-1, Rk + 2 * P)[:20].abs().max()) == 0.0
