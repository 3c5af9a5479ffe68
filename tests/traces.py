"""Builders of replay traces (the JSON steps ``bin/trace_run`` reads) and an in-process
replayer that drives a ``ModelRunner`` exactly as that program does."""
from __future__ import annotations

import itertools
import json
import os
import subprocess
import sys
from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def random_requests(vocab: int, lengths: Sequence[int], seed: int) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, vocab, (n,), generator=g).tolist()
            for i, n in enumerate(lengths)}


def rounded(n: int, to: int = 64) -> int:
    return -(-n // to) * to


def trace_whole(reqs: Dict[str, List[int]]) -> Tuple[List[dict], int]:
    """Each request alone, its whole token list in one step, every position wanted."""
    steps = [{"step": i, "entries": [{"id": k, "tokens": t, "want": list(range(len(t)))}],
              "end": [k]} for i, (k, t) in enumerate(reqs.items())]
    return steps, max(rounded(len(t)) for t in reqs.values())


def trace_tail(reqs: Dict[str, List[int]], tail: int = 32) -> Tuple[List[dict], int]:
    """All but the last ``tail`` tokens in one step, then the rest one token per step."""
    steps = []
    for k, t in reqs.items():
        head = max(1, len(t) - tail)
        steps.append({"step": len(steps), "entries": [
            {"id": k, "tokens": t[:head], "want": list(range(head))}], "end": []})
        for p in range(head, len(t)):
            steps.append({"step": len(steps), "entries": [
                {"id": k, "tokens": [t[p]], "want": [0]}], "end": []})
        steps[-1]["end"] = [k]
    return steps, max(rounded(len(t)) for t in reqs.values())


PORTIONS = [7, 2, 16, 3, 24, 2, 33, 5, 2, 64, 9, 2, 17]


def trace_portions(reqs: Dict[str, List[int]]) -> Tuple[List[dict], int]:
    """Each request alone in portions of changing size, down to two tokens, crossing page
    edges in the middle of a portion."""
    steps = []
    for k, t in reqs.items():
        pos, sizes = 0, itertools.cycle(PORTIONS)
        while pos < len(t):
            n = min(next(sizes), len(t) - pos)
            steps.append({"step": len(steps), "entries": [
                {"id": k, "tokens": t[pos:pos + n], "want": list(range(n))}], "end": []})
            pos += n
        steps[-1]["end"] = [k]
    return steps, max(rounded(len(t)) for t in reqs.values())


def trace_mixed(reqs: Dict[str, List[int]], live: int = 4, prompt_frac: float = 0.6,
                seed: int = 0) -> Tuple[List[dict], int]:
    """Up to ``live`` requests at a time: portions of the prompts of some beside single
    (decoded) tokens of others; a request is sometimes left out of a step; finished requests
    end and later ones take their pages.  Returns the steps and the smallest --max-tokens
    that holds them (so pages are used again)."""
    rng = np.random.default_rng(seed)
    waiting = list(reqs.items())
    running: List[list] = []          # [id, tokens, pos, prompt_len]
    steps, peak = [], 0
    sizes = itertools.cycle(PORTIONS)
    while waiting or running:
        while waiting and len(running) < live:
            k, t = waiting.pop(0)
            running.append([k, t, 0, max(1, int(len(t) * prompt_frac))])
        peak = max(peak, sum(rounded(len(r[1])) for r in running))
        entries, ended = [], []
        for r in running:
            k, t, pos, plen = r
            if len(running) > 1 and rng.random() < 0.15:
                continue                                   # left out of this step
            n = min(next(sizes), plen - pos) if pos < plen else 1
            entries.append({"id": k, "tokens": t[pos:pos + n], "want": list(range(n))})
            r[2] = pos + n
            if r[2] >= len(t):
                ended.append(k)
        if not entries:
            continue
        steps.append({"step": len(steps), "entries": entries, "end": ended})
        running = [r for r in running if r[0] not in ended]
    return steps, peak


def collect(steps: List[dict], outputs: Dict[int, torch.Tensor], vocab: int
            ) -> Dict[str, Dict[int, torch.Tensor]]:
    """Per request: logits by absolute position, gathered from the per-step outputs."""
    pos: Dict[str, int] = {}
    got: Dict[str, Dict[int, torch.Tensor]] = {}
    for s in steps:
        row = 0
        out = outputs.get(s["step"])
        for e in s["entries"]:
            p0 = pos.get(e["id"], 0)
            for w in e["want"]:
                got.setdefault(e["id"], {})[p0 + w] = out[row]
                row += 1
            pos[e["id"]] = p0 + len(e["tokens"])
        if out is not None:
            assert row == out.shape[0] and out.shape[1] == vocab
    return got


def replay_in_process(runner, steps: List[dict]) -> Dict[int, torch.Tensor]:
    """What ``bin/trace_run`` does, without the process around it."""
    from rust_llm_inference_server_amd.engine import StepEntry
    ids: Dict[str, int] = {}
    counter = itertools.count()
    outputs = {}
    for s in steps:
        entries = []
        for e in s["entries"]:
            if e["id"] not in ids:
                ids[e["id"]] = next(counter)
            seq = ids[e["id"]]
            runner.reserve(seq, runner.num_computed(seq) + len(e["tokens"]))
            entries.append(StepEntry(seq, e["tokens"], e["want"]))
        if entries:
            logits = runner.step(entries)
            if logits.shape[0]:
                outputs[s["step"]] = logits.float().cpu()
        for k in s["end"]:
            if k in ids:
                runner.free(ids.pop(k))
        runner.cache.check_invariants()
    return outputs


def replay_program(folder: str, dtype: str, steps: List[dict], max_tokens: int, out_dir: str,
                   vocab: int, timeout: int = 600) -> Dict[int, torch.Tensor]:
    """Run ``bin/trace_run`` as a child process, feeding a step only after ``done`` came back
    for the one before."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype",
           dtype, "--out", out_dir, "--max-tokens", str(max_tokens)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {s['step']}", f"trace_run answered {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=timeout) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    outputs = {}
    for s in steps:
        path = os.path.join(out_dir, f"{s['step']}.f32")
        if any(e["want"] for e in s["entries"]):
            data = np.fromfile(path, dtype="<f4")
            outputs[s["step"]] = torch.from_numpy(data.reshape(-1, vocab).copy())
        else:
            assert not os.path.exists(path)
    return outputs
