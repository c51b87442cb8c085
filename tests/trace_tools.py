"""Traces for the replay tests: the four ways of cutting the same requests
into steps, a driver for ``bin/trace_run`` and the comparison with the plain
implementation."""

from __future__ import annotations

import json
import random
import subprocess
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parent.parent


def make_sequences(vocab: int, lengths, seed: int) -> dict[str, list[int]]:
    rng = random.Random(seed)
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(lengths)}


def step(n, entries, end=()):
    return {"step": n, "entries": entries, "end": list(end)}


def trace_whole(seqs, first_step=0, prefix="w"):
    """Each request alone and whole, logits wanted everywhere."""
    steps = []
    for i, (name, ids) in enumerate(seqs.items()):
        rid = f"{prefix}-{name}"
        steps.append(step(first_step + i, [{"id": rid, "tokens": ids, "want": list(range(len(ids)))}], [rid]))
    return steps


def trace_tail(seqs, tail=32, first_step=0, prefix="t"):
    """Most of each request in one step, the last ``tail`` tokens one by one."""
    steps = []
    n = first_step
    for name, ids in seqs.items():
        rid = f"{prefix}-{name}"
        head = max(1, len(ids) - tail)
        steps.append(step(n, [{"id": rid, "tokens": ids[:head], "want": list(range(head))}]))
        n += 1
        for i in range(head, len(ids)):
            steps.append(step(n, [{"id": rid, "tokens": [ids[i]], "want": [0]}], [rid] if i == len(ids) - 1 else []))
            n += 1
        if head == len(ids):
            steps[-1]["end"] = [rid]
    return steps


def trace_portions(seqs, seed=0, first_step=0, prefix="p", sizes=(2, 3, 5, 7, 16, 17, 33, 64, 2, 1, 2)):
    """Portions of changing size, down to two tokens (and single ones)."""
    rng = random.Random(seed)
    steps = []
    n = first_step
    for name, ids in seqs.items():
        rid = f"{prefix}-{name}"
        i = 0
        while i < len(ids):
            size = min(rng.choice(sizes), len(ids) - i)
            last = i + size == len(ids)
            steps.append(step(n, [{"id": rid, "tokens": ids[i:i + size], "want": list(range(size))}],
                              [rid] if last else []))
            i += size
            n += 1
    return steps


def trace_mixed(seqs, seed=0, first_step=0, prefix="m", max_live=4, decode_tail=12, sizes=(2, 3, 5, 9, 16, 31)):
    """Up to ``max_live`` requests at once: portions of some beside single
    decoded tokens of others; a request may sit out a step; new requests start
    as others end, so that pages are given back and used again."""
    rng = random.Random(seed)
    waiting = list(seqs.items())
    live: dict[str, tuple[list[int], int]] = {}
    steps = []
    n = first_step
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.6):
            name, ids = waiting.pop(0)
            live[f"{prefix}-{name}"] = (ids, 0)
        entries, ended = [], []
        for rid, (ids, done) in list(live.items()):
            if len(live) > 1 and rng.random() < 0.15:
                continue  # left out of this step
            left = len(ids) - done
            size = 1 if left <= decode_tail else min(rng.choice(sizes), left - decode_tail)
            entries.append({"id": rid, "tokens": ids[done:done + size], "want": list(range(size))})
            if done + size == len(ids):
                ended.append(rid)
                del live[rid]
            else:
                live[rid] = (ids, done + size)
        if entries:
            steps.append(step(n, entries, ended))
            n += 1
    return steps


def required_tokens(steps, round_to=64) -> int:
    """The most tokens that live requests hold at any time in the trace, each
    request's count rounded up to a multiple of ``round_to``: the smallest
    --max-tokens the trace may be replayed with."""
    held: dict[str, int] = {}
    most = 0
    for st in steps:
        for e in st["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        most = max(most, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in st["end"]:
            held.pop(rid, None)
    return most


def collect(steps, outputs: dict, vocab: int) -> dict[str, np.ndarray]:
    """Logits by request id, in token order, from per-step outputs."""
    by_request: dict[str, list[np.ndarray]] = {}
    for st in steps:
        wanted = sum(len(e["want"]) for e in st["entries"])
        if wanted == 0:
            continue
        arr = np.asarray(outputs[st["step"]]).reshape(wanted, vocab)
        row = 0
        for e in st["entries"]:
            k = len(e["want"])
            by_request.setdefault(e["id"], []).append(arr[row:row + k])
            row += k
    return {rid: np.concatenate(parts) for rid, parts in by_request.items()}


def run_in_process(runner, steps) -> dict[int, np.ndarray]:
    outputs = {}
    for st in steps:
        entries = []
        for e in st["entries"]:
            if not runner.cache.has_request(e["id"]):
                runner.add_request(e["id"])
            entries.append((e["id"], e["tokens"], e["want"]))
        logits = runner.step(entries)
        if logits.shape[0]:
            outputs[st["step"]] = logits.float().cpu().numpy()
        for rid in st["end"]:
            runner.release(rid)
        runner.cache.check()
    return outputs


def run_trace_program(model_dir, dtype: str, steps, out_dir, max_tokens: int, extra=(), timeout=300):
    """Drive bin/trace_run as a user would: one line in, wait for ``done``."""
    cmd = [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype, "--out",
           str(out_dir), "--max-tokens", str(max_tokens), *extra]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)
    try:
        for st in steps:
            proc.stdin.write(json.dumps(st) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {st['step']}", f"expected 'done {st['step']}', got {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=timeout) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    outputs = {}
    for st in steps:
        f = Path(out_dir) / f"{st['step']}.f32"
        if sum(len(e["want"]) for e in st["entries"]):
            outputs[st["step"]] = np.fromfile(f, dtype="<f4")
        else:
            assert not f.exists()
    return outputs


# Largest difference allowed between the engine's logits and the plain
# implementation's (computed in 64-bit), as a fraction of the largest logit of
# the sequence.  32-bit: a few hundred roundings of 6e-8 each.  bfloat16: the
# residual stream is rounded to 8 bits of mantissa (4e-3) after every branch.
TOLERANCE = {"float32": 2e-5, "bfloat16": 3e-2}


def compare(got: np.ndarray, want: torch.Tensor, dtype: str, what: str = "") -> float:
    want = want.detach().double().numpy()
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    assert np.isfinite(got).all(), f"{what}: logits are not finite"
    scale = np.abs(want).max()
    err = np.abs(got - want).max(axis=-1)
    worst = int(err.argmax())
    assert err[worst] <= TOLERANCE[dtype] * scale, (
        f"{what}: first position over tolerance is {int(np.argmax(err > TOLERANCE[dtype] * scale))}, worst is "
        f"{worst} with |diff| {err[worst]:.3e} against scale {scale:.3e} (allowed {TOLERANCE[dtype] * scale:.3e})")
    return float(err[worst] / scale)
