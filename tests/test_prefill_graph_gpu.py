"""Short prompts run as recorded steps (engine/prefill.py): the same logits as the eager step, whatever the
padding, for whole prompts, chunks that continue a sequence and ragged batches, in 32-bit to the bit."""
import numpy as np
import pytest
import torch

import plain_llama as P
from tiny_configs import TINY_A, TINY_D

pytestmark = pytest.mark.gpu


def _model(tmp_path, cfg, stored):
    w = P.random_weights(cfg, 21, std=0.05, matrix_dtype=getattr(torch, stored))
    for name in w:
        if "q_proj" in name or "k_proj" in name:
            w[name] = (w[name].float() * 2).to(w[name].dtype)
    folder = str(tmp_path / f"m_{stored}")
    P.write_model(folder, dict(cfg, torch_dtype=stored), w)
    return folder, w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16"])
def test_recorded_prefill_steps_give_the_eager_logits(dtype, tmp_path):
    import llm_infer_amd
    cfg = dict(TINY_A, max_position_embeddings=1024)
    stored = "float16" if dtype == "float16" else "bfloat16"
    folder, weights = _model(tmp_path, cfg, stored)
    eager = llm_infer_amd.load(folder, dtype=dtype, max_tokens=8192)
    eager.record_prefill = False
    rec = llm_infer_amd.load(folder, dtype=dtype, max_tokens=8192)
    g = torch.Generator().manual_seed(5)
    act = None if dtype == "float32" else getattr(torch, dtype)

    def compare(steps, what):
        """``steps``: a list of (tokens of each sequence, wanted places) that continue the same sequences."""
        out = {}
        for eng, times in ((eager, 1), (rec, 3)):
            for _ in range(times):                               # first time eager, then recorded, then replayed
                slots = [eng.alloc_slot() for _ in steps[0][0]]
                got = [eng.step(slots[:len(toks)], toks, want).cpu() for toks, want in steps]
                for s in slots:
                    eng.free_slot(s)
                out.setdefault(eng, []).append(got)
        for run in out[rec]:
            for a, b in zip(out[eager][0], run):
                assert a.shape == b.shape
                if dtype == "float32":
                    assert torch.equal(a, b), what               # 32-bit: to the bit, whatever the padding
                else:
                    # other rows in the step, so other kernels: equal up to the rounding of 16-bit steps
                    assert (a - b).abs().max().item() < 0.05 * a.std().item(), what
        return out[rec][-1]

    for n in (1, 5, 16, 17, 100, 129, 300, 512):
        toks = torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist()
        got = compare([([toks], [list(range(n))])], f"one prompt of {n}")[0]
        ref = P.forward(weights, cfg, toks, torch.float64)
        own = (P.forward(weights, cfg, toks, torch.float64 if act else torch.float32, act).double() - ref).abs().max().item()
        assert (got.double() - ref).abs().max().item() < 3 * own + 1e-6 * ref.std().item(), n
    # a ragged batch, only the last places wanted; then the same sequences continued by chunks of unequal length
    lens = [7, 1, 13, 64, 30]
    seqs = [torch.randint(0, cfg["vocab_size"], (n + 40,), generator=g).tolist() for n in lens]
    first = ([s[:n] for s, n in zip(seqs, lens)], None)
    second = ([s[n:n + k] for s, n, k in zip(seqs, lens, (9, 40, 2, 17, 1))], [[0, k - 1] for k in (9, 40, 2, 17, 1)])
    got = compare([first, second], "a ragged batch and its continuation")
    for i, (s, n, k) in enumerate(zip(seqs, lens, (9, 40, 2, 17, 1))):
        ref = P.forward(weights, cfg, s[:n + k], torch.float64)
        own = (P.forward(weights, cfg, s[:n + k], torch.float64 if act else torch.float32, act).double() - ref).abs().max().item()
        tol = 3 * own + 1e-6 * ref.std().item()
        assert (got[0][i].double() - ref[n - 1]).abs().max().item() < tol
        assert (got[1][2 * i].double() - ref[n]).abs().max().item() < tol
        assert (got[1][2 * i + 1].double() - ref[n + k - 1]).abs().max().item() < tol
    assert rec._prefill.counts["replayed"] >= 9 and rec._prefill.counts["recorded"] >= 9
    assert eager._prefill is None or eager._prefill.counts["recorded"] == 0
    # a step of more than 512 tokens, or one that wants nothing, is not recorded
    before = dict(rec._prefill.counts)
    s = rec.alloc_slot()
    for _ in range(3):
        rec.step([s], [[1] * 10], [[]])
    long = torch.randint(0, cfg["vocab_size"], (513,), generator=g).tolist()
    rec.step([s], [long])
    assert rec._prefill.counts == before


def test_generation_through_recorded_prompts_and_steps(tmp_path):
    """Greedy generation, twice through the same engine (the second time every prompt step and decode step is a
    replay), against the plain implementation, at a head size that runs padded."""
    import llm_infer_amd
    folder, weights = _model(tmp_path, TINY_D, "bfloat16")
    eng = llm_infer_amd.load(folder, dtype="float32", max_tokens=2048)
    prompts = [[3, 1, 4, 1, 5, 9, 2, 6, 5, 3], [8, 9, 7], [2] * 33]
    want = [P.generate_greedy(weights, TINY_D, p, 6) for p in prompts]
    for _ in range(3):
        assert eng.generate(prompts, max_new_tokens=6, temperature=0.0) == want
        for p, w in zip(prompts, want):
            assert eng.generate([p], max_new_tokens=6, temperature=0.0) == [w]
    assert eng._prefill.counts["replayed"] >= 4
