"""The engine against the plain implementation, in 32-bit and in bfloat16: each request
alone and whole, with its last 32 tokens one by one, and in batches of unequal lengths whose
shorter requests end earlier, one batch after another so that slots and pages are used again.
The schedules run through bin/trace_run, i.e. through the engine's own step function."""
import os

import numpy as np
import pytest
import torch

import plain_llama as P
import trace_util as TU
from tiny_configs import ALL

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [40, 7, 100, 1, 64, 65, 33, 127], "B": [200, 1, 4, 9, 16, 31, 130, 255], "C": [300, 70, 5, 640, 129]}


def make_weights(cfg, seed):
    """Random weights with sharper attention than N(0, 0.02) gives: q and k projections are
    scaled up so that scores differ by a unit or two and a wrong key or position shows, yet
    bfloat16 rounding of the scores stays small."""
    w = P.random_weights(cfg, seed, std=0.05)
    for name in w:
        if "q_proj" in name or "k_proj" in name:
            w[name] = (w[name].float() * 2).to(w[name].dtype)
    return w


@pytest.fixture(scope="module", params=list(ALL))
def model(request, tmp_path_factory):
    name = request.param
    cfg = ALL[name]
    folder = str(tmp_path_factory.mktemp(f"tiny_{name}"))
    weights = make_weights(cfg, seed=ord(name))
    P.write_model(folder, cfg, weights)
    g = torch.Generator().manual_seed(7)
    requests = {f"r{i}": torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist()
                for i, n in enumerate(LENGTHS[name])}
    refs = {rid: P.forward(weights, cfg, toks, torch.float64).numpy() for rid, toks in requests.items()}
    # what 32-bit arithmetic itself costs on this model: the plain implementation in float32
    FP32_ERROR[name] = max(np.abs(P.forward(weights, cfg, toks, torch.float32).numpy() - refs[rid]).max()
                           for rid, toks in requests.items())
    # and what storing activations in bfloat16 between the kernels costs
    BF16_ERROR[name] = max(np.abs(P.forward(weights, cfg, toks, torch.float64, torch.bfloat16).numpy()
                                  - refs[rid]).max() for rid, toks in requests.items())
    return name, cfg, folder, requests, refs


FP32_ERROR = {}
BF16_ERROR = {}


def check(got, refs, dtype, what):
    """Within three times the error that the plain implementation itself has against float64 on
    the same model and requests: in float32 arithmetic, or with its activations rounded to
    bfloat16 at the places where a 16-bit engine stores them."""
    scale = np.mean([r.std() for r in refs.values()])
    own = FP32_ERROR if dtype == "float32" else BF16_ERROR
    tol = 3 * own[what.split()[0]] + 1e-6 * scale
    worst, worst_key = 0.0, None
    for (rid, p), row in got.items():
        e = np.abs(row.astype(np.float64) - refs[rid][p]).max()
        if e > worst:
            worst, worst_key = e, (rid, p)
    assert worst < tol, f"{what} {dtype}: first look at {worst_key}: error {worst:.3e}, allowed {tol:.3e}"
    return worst


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_three_schedules(model, dtype, tmp_path):
    name, cfg, folder, requests, refs = model
    vocab = cfg["vocab_size"]
    s1, w1 = TU.steps_whole(requests)
    s2, w2 = TU.steps_tail(requests, 32, first_step=1000)
    decoded = {rid: [0, 3, 32, 1, 17, 40, 9, 50][i % 8] for i, rid in enumerate(requests)}
    s3, w3 = TU.steps_batches(requests, 3, decoded, first_step=5000)
    need = sum(-(-len(t) // 64) * 64 for t in list(requests.values())[:3])
    max_tokens = max(need, max(-(-len(t) // 64) * 64 for t in requests.values()) * 3)
    got = TU.run_trace(folder, dtype, s1 + s2 + s3, {**w1, **w2, **w3}, vocab, max_tokens, str(tmp_path))
    assert got
    all_keys = set()
    for where, what in ((w1, "whole"), (w2, "tail"), (w3, "batches")):
        sub = {}
        for s, keys in where.items():
            data = np.fromfile(os.path.join(str(tmp_path), f"{s}.f32"), dtype="<f4").reshape(len(keys), vocab)
            for k, row in zip(keys, data):
                sub[k] = row
        assert set(sub) == {(r, p) for r, t in requests.items() for p in range(len(t))}, what
        check(sub, refs, dtype, f"{name} {what}")
        all_keys |= set(sub)
    assert len(all_keys) == sum(len(t) for t in requests.values())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_step_direct_and_generate(model, dtype):
    """Through the Python entry point: logits of a ragged batch, then greedy generation compared
    with the plain implementation token by token (where the plain logits leave no near tie)."""
    import llm_infer_amd
    name, cfg, folder, requests, refs = model
    weights = P.load_weights(folder)
    eng = llm_infer_amd.load(folder, dtype=dtype, max_tokens=4096)
    ids = list(requests)[:4]
    slots = [eng.alloc_slot() for _ in ids]
    logits = eng.step(slots, [requests[r] for r in ids]).cpu().numpy()
    got = {(r, len(requests[r]) - 1): logits[i] for i, r in enumerate(ids)}
    check(got, refs, dtype, f"{name} step")
    for s in slots:
        eng.free_slot(s)
    prompts = [requests[r][:20] for r in ids]
    n_new = 12
    for use_graph in (False, True):
        out = eng.generate(prompts, max_new_tokens=n_new, temperature=0.0, use_graph=use_graph)
        for p, o in zip(prompts, out):
            assert len(o) == n_new
            toks = list(p)
            for t in o:
                ref = P.forward(weights, cfg, toks, torch.float64)[-1]
                top2 = torch.topk(ref, 2).values
                margin = (top2[0] - top2[1]).item()
                if margin < (1e-4 if dtype == "float32" else 5e-2) * ref.std().item():
                    break                                     # a near tie: either token is right
                assert t == int(ref.argmax()), (name, dtype, use_graph)
                toks.append(t)
