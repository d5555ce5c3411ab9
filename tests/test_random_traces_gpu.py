"""Traces drawn at random (seeded) through bin/trace_run against the plain implementation: batches
of one to seven requests that start together, each with its own prompt and decode length, places
wanted at random (some steps want nothing, some requests are never asked), one batch after another
in a cache of exactly the size the trace's own rule gives (each live request's tokens rounded up to
64), so that every slot and page is used again."""
import random

import numpy as np
import pytest
import torch

import plain_llama as P
import trace_util as TU
from tiny_configs import ALL

pytestmark = pytest.mark.gpu


def draw_trace(cfg, seed):
    rng = random.Random(seed)
    gen = torch.Generator().manual_seed(seed)
    vocab, longest = cfg["vocab_size"], min(cfg["max_position_embeddings"], 260)
    steps, where, requests, need, s = [], {}, {}, 0, 0

    def wanted(n):
        u = rng.random()
        return [] if u < 0.15 else (list(range(n)) if u < 0.5 else sorted(rng.sample(range(n), rng.randint(1, n))))

    for b in range(rng.randint(3, 5)):
        ids = [f"b{b}r{i}" for i in range(rng.randint(1, 7))]
        total = {r: rng.randint(1, longest) for r in ids}
        for r in ids:
            requests[r] = torch.randint(0, vocab, (total[r],), generator=gen).tolist()
        done = {r: rng.randint(1, total[r]) if rng.random() < 0.8 else total[r] for r in ids}
        need = max(need, sum((total[r] + 63) // 64 * 64 for r in ids))
        entries, keys = [], []
        for r in ids:
            w = wanted(done[r])
            entries.append({"id": r, "tokens": requests[r][:done[r]], "want": w})
            keys += [(r, p) for p in w]
        live = ids
        while True:
            ending = [r for r in live if done[r] == total[r]]
            steps.append({"step": s, "entries": entries, "end": ending})
            where[s] = keys
            s += 1
            live = [r for r in live if r not in ending]
            if not live:
                break
            entries, keys = [], []
            for r in live:
                w = [0] if rng.random() < 0.8 else []
                entries.append({"id": r, "tokens": [requests[r][done[r]]], "want": w})
                keys += [(r, done[r])] * len(w)
                done[r] += 1
    return steps, where, requests, need


@pytest.mark.parametrize("name,seed", [("A", 1), ("C", 2), ("D", 3)])
def test_a_drawn_trace_against_the_plain_implementation(name, seed, tmp_path):
    cfg = ALL[name]
    weights = P.random_weights(cfg, seed, std=0.05)
    for key in weights:                                  # sharper attention: a wrong key or position shows
        if "q_proj" in key or "k_proj" in key:
            weights[key] = (weights[key].float() * 2).to(weights[key].dtype)
    folder = tmp_path / "model"
    folder.mkdir()
    P.write_model(str(folder), cfg, weights)
    steps, where, requests, need = draw_trace(cfg, seed)
    assert any(not keys for keys in where.values()) and len(steps) > 50
    refs = {r: P.forward(weights, cfg, t, torch.float64).numpy() for r, t in requests.items()}
    own = {"float32": max(np.abs(P.forward(weights, cfg, t, torch.float32).numpy() - refs[r]).max()
                          for r, t in requests.items()),
           "bfloat16": max(np.abs(P.forward(weights, cfg, t, torch.float64, torch.bfloat16).numpy() - refs[r]).max()
                           for r, t in requests.items())}
    scale = np.mean([r.std() for r in refs.values()])
    for dtype in ("float32", "bfloat16"):
        out_dir = tmp_path / dtype
        out_dir.mkdir()
        got = TU.run_trace(str(folder), dtype, steps, where, cfg["vocab_size"], need, str(out_dir))
        assert len(got) == len({k for keys in where.values() for k in keys})
        tol = 3 * own[dtype] + 1e-6 * scale
        for (r, p), row in got.items():
            err = np.abs(row.astype(np.float64) - refs[r][p]).max()
            assert err < tol, (name, dtype, r, p, err, tol)
