"""Trace replay: feed given token ids through a served model step by step
and write the logits of chosen rows — no sampling, no scheduling decisions
of its own. Every step's composition (which requests, how many new tokens
each) comes from the trace; pages, state slots, batch preparation, the
forward pass and the kernels are the engine's (Scheduler.schedule_plan,
ModelRunner.forward_logits).

    bin/trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Standard input, one JSON object per line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}],
     "end": ["a"]}
entries: each request's next tokens (a request is admitted at its first
entry and may skip steps); want: indices into this entry's tokens whose
logits are written; end: requests whose pages and slots are given back after
the step. A step with wanted rows writes OUT/<step>.f32, little-endian
float32 [rows, vocab] in entry order; every step prints "done <step>".
"""

from __future__ import annotations

import argparse
import json
import os
import sys

MAX_LIVE_REQUESTS = 4  # state slots of a replay engine


def build_engine(model_dir: str, dtype: str, max_tokens: int,
                 enforce_eager: bool = False):
    import torch

    from .. import ops
    from ..config import EngineConfig
    from .engine import LLMEngine

    on_gpu = torch.cuda.is_available()
    cfg = EngineConfig(model_path=model_dir, dtype=dtype,
                       device="cuda" if on_gpu else "cpu",
                       enforce_eager=enforce_eager)
    mc = cfg.model_config()
    if on_gpu and getattr(mc, "layers", None) is not None:
        # a fresh checkout compiles the kernels this model needs, once
        ops.ensure_built("arks_amd_seq_C")
    elif on_gpu:
        ops.ensure_built("arks_amd_C")
    bs = cfg.block_size
    cfg.kv_cache_blocks = max(1, -(-max_tokens // bs))
    cfg.max_num_seqs = MAX_LIVE_REQUESTS
    cfg.max_model_len = max(max_tokens, bs)
    cfg.max_num_batched_tokens = max(max_tokens, bs)
    cfg.enable_prefix_caching = False  # rows of every given token must run
    return LLMEngine(cfg)


def replay(engine, lines, out_dir: str, log=sys.stdout) -> None:
    import numpy as np

    from .sequence import SamplingParams, Sequence

    sched, runner = engine.scheduler, engine.runner
    live: dict[str, Sequence] = {}
    for line in lines:
        line = line.strip()
        if not line:
            continue
        step = json.loads(line)
        plan, rows, base = [], [], 0
        for e in step["entries"]:
            toks = [int(t) for t in e["tokens"]]
            if not toks:
                continue
            seq = live.get(e["id"])
            if seq is None:
                seq = Sequence(toks, SamplingParams(ignore_eos=True),
                               request_id=str(e["id"]))
                sched.add(seq)
                live[e["id"]] = seq
            else:
                seq.prompt_token_ids.extend(toks)
            plan.append((seq, len(toks)))
            rows += [base + int(w) for w in e.get("want", [])]
            base += len(toks)
        if plan:
            sb = sched.schedule_plan(plan)
            if rows:
                logits = runner.forward_logits(sb, rows)
                arr = logits.float().cpu().numpy().astype("<f4")
                assert arr.shape[0] == len(rows), (arr.shape, len(rows))
                tmp = os.path.join(out_dir, f".{step['step']}.part")
                with open(tmp, "wb") as f:
                    f.write(np.ascontiguousarray(arr).tobytes())
                os.replace(tmp, os.path.join(out_dir, f"{step['step']}.f32"))
            else:
                runner.forward_logits(sb)
        for rid in step.get("end", []):
            seq = live.pop(rid, None)
            if seq is not None:
                sched.finish(seq)
        print(f"done {step['step']}", file=log, flush=True)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                 formatter_class=argparse.RawTextHelpFormatter)
    ap.add_argument("--model", required=True)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--out", required=True)
    ap.add_argument("--max-tokens", type=int, required=True)
    ap.add_argument("--enforce-eager", action="store_true",
                    help="no hipGraph replay of decode steps")
    a = ap.parse_args(argv)
    os.makedirs(a.out, exist_ok=True)
    # keep stdout for the protocol: everything else a library prints goes
    # to stderr
    proto = os.fdopen(os.dup(1), "w")
    os.dup2(2, 1)
    try:
        engine = build_engine(a.model, a.dtype, a.max_tokens, a.enforce_eager)
    except ValueError as e:
        if a.dtype == "float32" and "bfloat16 only" in str(e):
            print(e, file=sys.stderr)
            return 3
        raise
    print(f"trace_run: {engine.model_cfg.architecture} in {a.dtype} on "
          f"{engine.runner.device}", file=sys.stderr, flush=True)
    replay(engine, sys.stdin, a.out, log=proto)
    return 0


if __name__ == "__main__":
    sys.exit(main())
