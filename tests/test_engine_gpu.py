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

LENGTHS = {"A": [40, 7, 100, 1, 64, 65, 33, 127], "B": [200, 1, 4, 9, 16, 31, 130, 255], "C": [300, 70, 5, 640, 129],
           "D": [150, 2, 64, 33, 190], "E": [90, 1, 65, 300], "F": [120, 3, 64, 159, 31]}


def make_weights(cfg, seed, matrix_dtype=torch.bfloat16):
    """Random weights with sharper attention than N(0, 0.02) gives: q and k projections are
    scaled up so that scores differ by a unit or two and a wrong key or position shows, yet
    16-bit rounding of the scores stays small."""
    w = P.random_weights(cfg, seed, std=0.05, matrix_dtype=matrix_dtype)
    for name in w:
        if "q_proj" in name or "k_proj" in name:
            w[name] = (w[name].float() * 2).to(w[name].dtype)
    return w


DTYPES = ["float32", "bfloat16", "float16"]
STORED = {"float32": "bfloat16", "bfloat16": "bfloat16", "float16": "float16"}    # the folder a run opens
TORCH = {"bfloat16": torch.bfloat16, "float16": torch.float16}


class Model:
    """A tiny configuration with its requests and, for each storage type of the matrices, a model folder,
    the float64 logits of the plain implementation and that implementation's own error."""

    def __init__(self, name, tmp_path_factory):
        self.name, self.cfg = name, ALL[name]
        g = torch.Generator().manual_seed(7)
        self.requests = {f"r{i}": torch.randint(0, self.cfg["vocab_size"], (n,), generator=g).tolist()
                         for i, n in enumerate(LENGTHS[name])}
        self.folder, self.refs, self.own_error = {}, {}, {}
        for stored, dt in TORCH.items():
            folder = str(tmp_path_factory.mktemp(f"tiny_{name}_{stored}"))
            weights = make_weights(self.cfg, seed=ord(name), matrix_dtype=dt)
            P.write_model(folder, dict(self.cfg, torch_dtype=stored), weights)
            refs = {rid: P.forward(weights, self.cfg, toks, torch.float64).numpy()
                    for rid, toks in self.requests.items()}
            self.folder[stored], self.refs[stored] = folder, refs
            # what storing activations in this 16-bit type between the kernels costs
            self.own_error[stored] = max(
                np.abs(P.forward(weights, self.cfg, toks, torch.float64, dt).numpy() - refs[rid]).max()
                for rid, toks in self.requests.items())
            if stored == STORED["float32"]:
                # what 32-bit arithmetic itself costs on this model: the plain implementation in float32
                self.own_error["float32"] = max(
                    np.abs(P.forward(weights, self.cfg, toks, torch.float32).numpy() - refs[rid]).max()
                    for rid, toks in self.requests.items())


@pytest.fixture(scope="module", params=list(ALL))
def model(request, tmp_path_factory):
    return Model(request.param, tmp_path_factory)


def check(got, model, dtype, what):
    """Within three times the error that the plain implementation itself has against float64 on
    the same model and requests: in float32 arithmetic, or with its activations rounded to the
    16-bit type at the places where a 16-bit engine stores them."""
    refs = model.refs[STORED[dtype]]
    scale = np.mean([r.std() for r in refs.values()])
    tol = 3 * model.own_error[dtype] + 1e-6 * scale
    worst, worst_key = 0.0, None
    for (rid, p), row in got.items():
        e = np.abs(row.astype(np.float64) - refs[rid][p]).max()
        if e > worst:
            worst, worst_key = e, (rid, p)
    assert worst < tol, f"{model.name} {what} {dtype}: first look at {worst_key}: error {worst:.3e}, allowed {tol:.3e}"
    return worst


@pytest.mark.parametrize("dtype", DTYPES)
def test_replay_three_schedules(model, dtype, tmp_path):
    cfg, requests = model.cfg, model.requests
    vocab = cfg["vocab_size"]
    s1, w1 = TU.steps_whole(requests)
    s2, w2 = TU.steps_tail(requests, 32, first_step=1000)
    decoded = {rid: [0, 3, 32, 1, 17, 40, 9, 50][i % 8] for i, rid in enumerate(requests)}
    s3, w3 = TU.steps_batches(requests, 3, decoded, first_step=5000)
    need = sum(-(-len(t) // 64) * 64 for t in list(requests.values())[:3])
    max_tokens = max(need, max(-(-len(t) // 64) * 64 for t in requests.values()) * 3)
    got = TU.run_trace(model.folder[STORED[dtype]], dtype, s1 + s2 + s3, {**w1, **w2, **w3}, vocab, max_tokens,
                       str(tmp_path))
    assert got
    all_keys = set()
    for where, what in ((w1, "whole"), (w2, "tail"), (w3, "batches")):
        sub = {}
        for s, keys in where.items():
            data = np.fromfile(os.path.join(str(tmp_path), f"{s}.f32"), dtype="<f4").reshape(len(keys), vocab)
            for k, row in zip(keys, data):
                sub[k] = row
        assert set(sub) == {(r, p) for r, t in requests.items() for p in range(len(t))}, what
        check(sub, model, dtype, what)
        all_keys |= set(sub)
    assert len(all_keys) == sum(len(t) for t in requests.values())


@pytest.mark.parametrize("dtype", DTYPES)
def test_step_direct_and_generate(model, dtype):
    """Through the Python entry point: logits of a ragged batch, then greedy generation compared
    with the plain implementation token by token (where the plain logits leave no near tie)."""
    import llm_infer_amd
    cfg, requests, folder = model.cfg, model.requests, model.folder[STORED[dtype]]
    weights = P.load_weights(folder)
    eng = llm_infer_amd.load(folder, dtype=dtype, max_tokens=4096)
    ids = list(requests)[:4]
    slots = [eng.alloc_slot() for _ in ids]
    logits = eng.step(slots, [requests[r] for r in ids]).cpu().numpy()
    got = {(r, len(requests[r]) - 1): logits[i] for i, r in enumerate(ids)}
    check(got, model, dtype, "step")
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
                assert t == int(ref.argmax()), (model.name, dtype, use_graph)
                toks.append(t)


@pytest.mark.parametrize("dtype", DTYPES)
def test_half_paired_model_is_the_adjacent_model_with_dealt_out_rows(dtype, tmp_path):
    """"rope_pairing": "half" is served by ordering the rows of every q and k head when the weights are bound:
    the same checkpoint with those rows dealt out by hand (j -> 2j, j + rotary/2 -> 2j+1) and adjacent pairing
    gives the same logits to the bit, prompt and decoded tokens, and both run the fused kernels."""
    import llm_infer_amd
    cfg = dict(ALL["F"], torch_dtype=STORED[dtype])
    s = P.sizes(cfg)
    weights = make_weights(cfg, seed=11, matrix_dtype=TORCH[STORED[dtype]])
    order = list(range(s["hd"]))
    for j in range(s["rotary"] // 2):
        order[2 * j], order[2 * j + 1] = j, j + s["rotary"] // 2
    dealt = dict(weights)
    for name, w in weights.items():
        if "q_proj" in name or "k_proj" in name:
            heads = w.shape[0] // s["hd"]
            dealt[name] = w.view(heads, s["hd"], -1)[:, order].reshape(w.shape).contiguous()
    P.write_model(str(tmp_path / "half"), cfg, weights)
    P.write_model(str(tmp_path / "adjacent"), dict(cfg, rope_pairing="adjacent"), dealt)
    tokens = [[5, 300, 17, 2, 250, 99, 1], [8] * 70]
    out = []
    for folder in ("half", "adjacent"):
        eng = llm_infer_amd.load(str(tmp_path / folder), dtype=dtype, max_tokens=512)
        slots = [eng.alloc_slot() for _ in tokens]
        first = eng.step(slots, tokens, [list(range(len(t))) for t in tokens])
        second = eng.step(slots, [[3], [4]])
        out.append(torch.cat([first, second]).cpu())
    assert torch.equal(out[0], out[1])
    # and they are the plain implementation's, which pairs (j, j + rotary/2) itself
    ref = P.forward(weights, cfg, tokens[0], torch.float64)
    err = (out[0][:len(tokens[0])].double() - ref).abs().max().item()
    own = (P.forward(weights, cfg, tokens[0], torch.float64, None if dtype == "float32" else TORCH[dtype]) - ref).abs().max().item()
    own = max(own, (P.forward(weights, cfg, tokens[0], torch.float32).double() - ref).abs().max().item())
    assert err < 3 * own + 1e-6 * ref.std().item(), (err, own)
    wrong = P.forward(weights, dict(cfg, rope_pairing="adjacent"), tokens[0], torch.float64)
    assert (wrong - ref).abs().max().item() > 10 * (3 * own + 1e-6)       # the pairing matters on this model


def test_a_model_runs_in_its_own_dtype_unless_told_otherwise(model, capfd):
    """A folder opened with no dtype runs in the type its files say; a dtype that narrows or swaps the
    stored 16-bit type is said in one line."""
    import llm_infer_amd
    for stored, dt in TORCH.items():
        eng = llm_infer_amd.load(model.folder[stored], max_tokens=256)
        assert eng.dtype == dt and eng.model.layers[0].mixer.wo.dtype == dt
        assert eng.model.final_norm.weight.dtype == torch.float32
        assert "stored" not in capfd.readouterr().err
    eng = llm_infer_amd.load(model.folder["float16"], dtype="bfloat16", max_tokens=256)
    assert eng.dtype == torch.bfloat16 and "three bits" in capfd.readouterr().err
    eng = llm_infer_amd.load(model.folder["float16"], dtype="float32", max_tokens=256)
    assert eng.dtype == torch.float32 and "stored" not in capfd.readouterr().err


@pytest.mark.parametrize("dtype", DTYPES)
def test_random_weights_without_a_folder_are_the_folders(dtype, tmp_path):
    """An engine made from a configuration and a seed holds what write_random_model writes for them: the same
    logits to the bit as the engine that opens that folder.  With the device's generator they are other values."""
    import llm_infer_amd
    cfg = llm_infer_amd.config_from_dict(ALL["D"])
    llm_infer_amd.write_random_model(str(tmp_path), cfg, seed=5, dtype=STORED[dtype])
    tokens = [[3, 1, 4, 1, 5, 9, 2, 6], [5, 3]]
    want = [[7], [0, 1]]
    logits = []
    for eng in (llm_infer_amd.load(str(tmp_path), dtype=dtype, max_tokens=256),
                llm_infer_amd.random_model(cfg, seed=5, dtype=dtype, max_tokens=256),
                llm_infer_amd.random_model(cfg, seed=5, dtype=dtype, max_tokens=256, same_as_folder=False)):
        slots = [eng.alloc_slot() for _ in tokens]
        logits.append(eng.step(slots, tokens, want).float().cpu())
    assert torch.equal(logits[0], logits[1])
    assert not torch.equal(logits[0], logits[2])
