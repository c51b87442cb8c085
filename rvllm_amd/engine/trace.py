"""Trace replay: feeds given token ids through a model step by step and writes
logits.  It samples nothing and has no forward pass, cache or loader of its
own: every step goes through ``ModelRunner.step``, the step function that
generation uses.

The reference has the pieces of this as debugging switches — prompt ids from a
file (v3/crates/rvllm-bench/src/main.rs:938-965), a dump of one row of logits
(v3/crates/rvllm-runtime/src/gemma4_bring_up.rs:5766-5785), forced tokens with
logits read each step in its perplexity run (gemma4_bring_up.rs:3095-3112) —
but no program that replays a trace.

Input, one JSON object a line on standard input:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
Output: ``<out>/<step>.f32`` (little-endian float32 ``[wanted, vocab]``, in the
order of the entries and of ``want``) for every step that wants something, and
a line ``done <step>`` on standard output after every step.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
from pathlib import Path


def parse_args(argv=None) -> argparse.Namespace:
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=["bfloat16", "float32"],
                   help="bfloat16: the kernels and precisions that serving uses; float32: everything in true 32-bit")
    p.add_argument("--out", required=True, help="folder for the <step>.f32 files")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens that live requests hold at any time (each rounded up to a multiple of 64); "
                        "the cache pool is made for this many")
    p.add_argument("--max-live", type=int, default=4, help="most requests that are live at a time (default 4)")
    p.add_argument("--page-size", type=int, default=None, help="tokens per cache page (default: the engine's)")
    p.add_argument("--device", default="cuda:0")
    return p.parse_args(argv)


def main(argv=None) -> int:
    args = parse_args(argv)
    print("[trace_run] loading (the first call in a fresh checkout compiles the kernels)", file=sys.stderr, flush=True)
    import numpy as np
    import torch

    from ..config.engine_config import EngineConfig
    from .runner import ModelRunner

    max_live = int(args.max_live)
    cfg = EngineConfig(dtype=args.dtype, device=args.device)
    if args.page_size is not None:
        cfg.page_size = args.page_size
    max_tokens = max(int(args.max_tokens), cfg.page_size)
    cfg.max_cache_tokens = max_tokens
    cfg.max_model_len = max_tokens
    cfg.max_num_seqs = max_live
    cfg.max_num_batched_tokens = max_tokens
    cfg.max_prefill_chunk = max_tokens
    runner = ModelRunner.from_model_dir(args.model, cfg)
    out_dir = Path(args.out)
    out_dir.mkdir(parents=True, exist_ok=True)
    print("[trace_run] ready", file=sys.stderr, flush=True)

    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            rid = e["id"]
            if not runner.cache.has_request(rid):
                if len(runner.cache.requests) >= max_live:
                    raise SystemExit(f"trace_run: step {step} starts request {rid!r} while {max_live} are live; "
                                     f"end one first or raise --max-live")
                runner.add_request(rid)
            entries.append((rid, e["tokens"], e.get("want", [])))
        logits = runner.step(entries)
        if logits.shape[0] > 0:
            data = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
            tmp = out_dir / f".{step}.f32.tmp"
            data.tofile(tmp)
            os.replace(tmp, out_dir / f"{step}.f32")
        else:
            torch.cuda.synchronize()
        for rid in rec.get("end", []):
            if runner.cache.has_request(rid):
                runner.release(rid)
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
