"""Builds replay traces in the three ways of cutting a set of requests into steps, runs
``bin/trace_run`` on them and collects the logits per (request, position)."""
import json
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def steps_whole(requests, first_step=0):
    """Each request alone, whole, all positions wanted."""
    steps, where = [], {}
    for k, (rid, toks) in enumerate(requests.items()):
        s = first_step + k
        steps.append({"step": s, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}],
                      "end": [rid]})
        where[s] = [(rid, p) for p in range(len(toks))]
    return steps, where


def steps_tail(requests, tail=32, first_step=0):
    """Each request alone: all but the last ``tail`` tokens in one step, the rest one by one."""
    steps, where, s = [], {}, first_step
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append({"step": s, "entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}],
                      "end": [rid] if head == len(toks) else []})
        where[s] = [(rid, p) for p in range(head)]
        s += 1
        for p in range(head, len(toks)):
            steps.append({"step": s, "entries": [{"id": rid, "tokens": [toks[p]], "want": [0]}],
                          "end": [rid] if p == len(toks) - 1 else []})
            where[s] = [(rid, p)]
            s += 1
    return steps, where


def steps_batches(requests, batch_size, decoded, first_step=0):
    """Batches of ``batch_size`` requests that start together: the first step brings each request's
    tokens but its last ``decoded[rid]``, then every live request goes on by one token; shorter
    requests end earlier; one batch after another."""
    steps, where, s = [], {}, first_step
    ids = list(requests)
    for b in range(0, len(ids), batch_size):
        batch = ids[b:b + batch_size]
        head = {r: max(1, len(requests[r]) - decoded.get(r, 0)) for r in batch}
        done = {r: head[r] for r in batch}
        entries = [{"id": r, "tokens": requests[r][:head[r]], "want": list(range(head[r]))} for r in batch]
        ending = [r for r in batch if done[r] == len(requests[r])]
        steps.append({"step": s, "entries": entries, "end": ending})
        where[s] = [(r, p) for r in batch for p in range(head[r])]
        s += 1
        live = [r for r in batch if r not in ending]
        while live:
            entries = [{"id": r, "tokens": [requests[r][done[r]]], "want": [0]} for r in live]
            where[s] = [(r, done[r]) for r in live]
            for r in live:
                done[r] += 1
            ending = [r for r in live if done[r] == len(requests[r])]
            steps.append({"step": s, "entries": entries, "end": ending})
            s += 1
            live = [r for r in live if r not in ending]
    return steps, where


def run_trace(model_dir, dtype, steps, where, vocab, max_tokens, out_dir, env=None, timeout=600):
    """Runs bin/trace_run, one step after each "done"; returns {(request, position): logits}."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, env=env)
    try:
        for st in steps:
            proc.stdin.write(json.dumps(st) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {st['step']}", f"trace_run said {line!r} after step {st['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=timeout) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    out = {}
    for s, keys in where.items():
        path = os.path.join(out_dir, f"{s}.f32")
        if not keys:
            assert not os.path.exists(path)
            continue
        data = np.fromfile(path, dtype="<f4").reshape(len(keys), vocab)
        for k, row in zip(keys, data):
            out[k] = row
    return out
