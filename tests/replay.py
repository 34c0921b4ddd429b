"""Traces for the step function, in the format ``bin/trace_run`` reads, and the means to
run them (in process on an ``EngineCore``, or through the program) and to compare what
comes back with the plain implementation.

A trace is a list of step records ``{"step", "entries": [{"id", "tokens", "want"}], "end"}``.
Four ways of cutting the same requests:

    whole        each request alone, the whole prompt in one step
    tail         most of it in one step, the last 32 tokens one by one
    portions     portions of changing size, down to two tokens
    mixed        up to four live requests, portions of some beside single tokens of others,
                 requests ending and starting so that their pages are used again
"""

from __future__ import annotations

import json
import os
import random
import subprocess
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def whole(requests: dict[str, list[int]]) -> list[dict]:
    steps = []
    for k, (rid, ids) in enumerate(requests.items()):
        steps.append({"step": k, "entries": [{"id": rid, "tokens": ids, "want": list(range(len(ids)))}], "end": [rid]})
    return steps


def tail(requests: dict[str, list[int]], last: int = 32) -> list[dict]:
    steps, k = [], 0
    for rid, ids in requests.items():
        head = max(1, len(ids) - last)
        steps.append({"step": k, "entries": [{"id": rid, "tokens": ids[:head], "want": list(range(head))}], "end": []})
        k += 1
        for i in range(head, len(ids)):
            steps.append({"step": k, "entries": [{"id": rid, "tokens": [ids[i]], "want": [0]}],
                          "end": [rid] if i == len(ids) - 1 else []})
            k += 1
        if head == len(ids):
            steps[-1]["end"] = [rid]
    return steps


def portions(requests: dict[str, list[int]], seed: int = 0, sizes=(2, 3, 5, 16, 17, 31, 2, 64, 7)) -> list[dict]:
    rng = random.Random(seed)
    steps, k = [], 0
    for rid, ids in requests.items():
        at, turn = 0, rng.randrange(len(sizes))
        while at < len(ids):
            n = min(sizes[turn % len(sizes)], len(ids) - at)
            if len(ids) - at - n == 1:   # never leave a single token: portions go down to two
                n += 1
            turn += 1
            end = at + n >= len(ids)
            steps.append({"step": k, "entries": [{"id": rid, "tokens": ids[at:at + n], "want": list(range(n))}],
                          "end": [rid] if end else []})
            at += n
            k += 1
    return steps


def mixed(requests: dict[str, list[int]], seed: int = 0, max_live: int = 4, decode_tail: int = 12,
          skip_chance: float = 0.15) -> list[dict]:
    """Requests are admitted in order while fewer than ``max_live`` are live.  A live request
    feeds portions of random size (2..40) until only ``decode_tail`` tokens are left, then
    single tokens.  Now and then a request sits a step out."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live: dict[str, int] = {}   # id -> tokens fed
    steps, k = [], 0
    while waiting or live:
        while waiting and len(live) < max_live and (not live or rng.random() < 0.6):
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, ended = [], []
        for rid in list(live):
            ids, at = requests[rid], live[rid]
            if len(live) > 1 and rng.random() < skip_chance:
                continue
            left = len(ids) - at
            if left <= decode_tail or left == 1:
                n = 1
            else:
                n = min(rng.choice([2, 3, 4, 7, 8, 9, 15, 16, 17, 33, 40]), left - decode_tail)
                if n == 1:
                    n = min(2, left)
            entries.append({"id": rid, "tokens": ids[at:at + n], "want": list(range(n))})
            live[rid] = at + n
            if live[rid] >= len(ids):
                ended.append(rid)
                del live[rid]
        if not entries:
            continue
        rng.shuffle(entries)
        steps.append({"step": k, "entries": entries, "end": ended})
        k += 1
    return steps


def scheduled(requests: dict[str, list[int]], seed: int = 0, max_live: int = 4, budget: int = 96,
              decode_tail: int = 10) -> list[dict]:
    """Steps as a scheduler under a small token budget makes them: the live requests that are past their
    prompt bring one token each (logits wanted), and the budget's rest goes to the next portions of one or two
    prompts (logits wanted at a prompt's last token only)."""
    rng = random.Random(seed)
    waiting = list(requests.items())
    live: dict[str, int] = {}
    steps, k = [], 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, _ = waiting.pop(0)
            live[rid] = 0
        entries, ended, left, portions = [], [], budget, 0
        for rid in list(live):
            ids, at = requests[rid], live[rid]
            prompt = len(ids) - decode_tail
            if at >= prompt or len(ids) - at == 1:
                n, want = 1, [0]
            else:
                if portions == 2 or left < 2:
                    continue
                n = min(prompt - at, left, rng.choice([5, 17, 40, 64, budget]))
                if n < 2:
                    continue
                if len(ids) - at - n == 1:
                    n += 1
                want = [n - 1] if at + n >= prompt else []
                portions += 1
            left -= n
            entries.append({"id": rid, "tokens": ids[at:at + n], "want": want})
            live[rid] = at + n
            if live[rid] >= len(ids):
                ended.append(rid)
                del live[rid]
        if not entries:
            continue
        steps.append({"step": k, "entries": entries, "end": ended})
        k += 1
    return steps


def peak_tokens(steps: list[dict], round_to: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up to ``round_to``."""
    held: dict[str, int] = {}
    peak = 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return peak


# ------------------------------------------------------------------ running


def run_in_process(core, steps: list[dict]) -> dict[int, torch.Tensor]:
    from atom_amd.engine.core import StepEntry

    out = {}
    for s in steps:
        entries = [StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]]
        logits = core.step(entries)
        if logits is not None:
            out[s["step"]] = logits.detach().to("cpu", torch.float32)
        for rid in s["end"]:
            core.close(rid)
        core.manager.check()
    return out


def run_program(model_dir: str, dtype: str, steps: list[dict], out_dir: str, max_tokens: int, vocab: int,
                env: dict | None = None, timeout: int = 600, extra: list[str] | None = None) -> dict[int, torch.Tensor]:
    """Drives ``bin/trace_run``: one step a line, waiting for its ``done`` before the next."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens), *(extra or [])]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, env=env)
    try:
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline()
            if line.strip() != f"done {s['step']}":
                raise RuntimeError(f"trace_run answered {line!r} to step {s['step']} (exit {proc.poll()})")
        proc.stdin.close()
        rc = proc.wait(timeout=timeout)
    finally:
        if proc.poll() is None:
            proc.kill()
    if rc != 0:
        raise RuntimeError(f"trace_run exited with {rc}")
    out = {}
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        path = os.path.join(out_dir, f"{s['step']}.f32")
        if wanted:
            data = np.fromfile(path, dtype="<f4")
            assert data.size == wanted * vocab, f"step {s['step']}: {data.size} floats for {wanted} rows of {vocab}"
            out[s["step"]] = torch.from_numpy(data.reshape(wanted, vocab).copy())
        else:
            assert not os.path.exists(path)
    return out


# ------------------------------------------------------------------ comparing


def collect(steps: list[dict], results: dict[int, torch.Tensor]) -> dict[str, dict[int, torch.Tensor]]:
    """request -> position -> logits row, from what the steps returned."""
    fed: dict[str, int] = {}
    rows: dict[str, dict[int, torch.Tensor]] = {}
    for s in steps:
        r = 0
        for e in s["entries"]:
            start = fed.get(e["id"], 0)
            for w in e["want"]:
                rows.setdefault(e["id"], {})[start + w] = results[s["step"]][r]
                r += 1
            fed[e["id"]] = start + len(e["tokens"])
        if s["step"] in results:
            assert r == results[s["step"]].shape[0]
        for rid in s["end"]:
            fed.pop(rid, None)
    return rows


# Tolerances, as a fraction of the largest logit of the request.  float32: the engine and the
# float64 reference differ by accumulated float32 rounding only.  bfloat16: activations and
# weights carry 8 bits of mantissa (2^-8 = 0.4 % per rounding).
TOL = {"float32": dict(max=3e-5, mean=3e-6), "bfloat16": dict(max=3e-2, mean=5e-3)}


def first_bad(rows: dict[int, torch.Tensor], want: torch.Tensor, dtype: str):
    """None if every row is within tolerance, else a description of the first that is not."""
    scale = float(want.abs().max())
    tol = TOL[dtype]
    for pos in sorted(rows):
        diff = (rows[pos].double() - want[pos].double()).abs()
        if not torch.isfinite(rows[pos]).all():
            return f"position {pos}: not finite"
        if float(diff.max()) > tol["max"] * scale or float(diff.mean()) > tol["mean"] * scale:
            return (f"position {pos}: max diff {float(diff.max()):.3e} mean {float(diff.mean()):.3e} "
                    f"(scale {scale:.3f}, allowed {tol['max'] * scale:.3e} / {tol['mean'] * scale:.3e})")
    return None


def check(steps, results, requests, oracle: dict[str, torch.Tensor], dtype: str, what: str = "", every: bool = True):
    rows = collect(steps, results)
    for rid, ids in requests.items():
        got = rows.get(rid, {})
        if every:
            assert len(got) == len(ids), f"{what} request {rid}: {len(got)} of {len(ids)} positions came back"
        else:
            assert got, f"{what} request {rid}: nothing came back"
        bad = first_bad(got, oracle[rid], dtype)
        assert bad is None, f"{what} request {rid} ({len(ids)} tokens): {bad}"
