"""Each part alone against the plain implementation; long decoding; the first tokens; slots and
pages used again; batch composition; sampling through the entry points; and a toy architecture
(a mixer with state of its own, a layer named twice, a layer that reads another's cache) that is
registered, built and stepped without touching the framework's files."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama as P
from tiny_configs import TINY_A, TINY_B, TINY_C

pytestmark = pytest.mark.gpu
DEV = "cuda"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def sharp_weights(cfg, seed, matrix_dtype=torch.bfloat16):
    w = P.random_weights(cfg, seed, std=0.05, matrix_dtype=matrix_dtype)
    for name in w:
        if "q_proj" in name or "k_proj" in name:
            w[name] = (w[name].float() * 2).to(w[name].dtype)
    return w


@pytest.fixture(scope="module")
def lib():
    import llm_infer_amd
    return llm_infer_amd


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name, cfg in (("A", TINY_A), ("B", TINY_B), ("C", TINY_C)):
        d = str(tmp_path_factory.mktemp(f"gen_{name}"))
        P.write_model(d, cfg, sharp_weights(cfg, 11 + ord(name)))
        out[name] = d
        d = str(tmp_path_factory.mktemp(f"gen_{name}_float16"))          # the same model stored in float16
        P.write_model(d, dict(cfg, torch_dtype="float16"), sharp_weights(cfg, 11 + ord(name), torch.float16))
        out[name, "float16"] = d
    return out


DTYPES = ["float32", "bfloat16", "float16"]
ACT = {"bfloat16": torch.bfloat16, "float16": torch.float16}


def folder_for(folders, name, dtype):
    """The folder a run in ``dtype`` opens: matrices stored in float16 for float16, in bfloat16 otherwise."""
    return folders[name, "float16"] if dtype == "float16" else folders[name]


def _ctx(lens_before, tokens):
    from llm_infer_amd.engine.step import StepContext
    return StepContext(DEV, list(range(len(tokens))), tokens, lens_before, [[] for _ in tokens])


# ---------------------------------------------------------------------------
# the parts, each alone, at sizes of their own
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
def test_parts_alone(lib, dt):
    from llm_infer_amd.cache import Cache
    from llm_infer_amd.parts import Attention, Embedding, GatedMLP, LMHead, PreNormBlock, RMSNorm, RotaryPosition, SubLayer
    d, H, K, hd, F, V, eps, theta, rot = 112, 6, 3, 32, 200, 77, 1e-3, 777.0, 16
    g = torch.Generator().manual_seed(4)
    tol = 2e-5 if dt == torch.float32 else 3e-2

    def mat(*shape, s=0.1):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)

    w = {"n1.weight": 1 + 0.1 * torch.randn(d, generator=g), "n2.weight": 1 + 0.1 * torch.randn(d, generator=g),
         "a.q_proj.weight": mat(H * hd, d), "a.k_proj.weight": mat(K * hd, d), "a.v_proj.weight": mat(K * hd, d),
         "a.o_proj.weight": mat(d, H * hd), "f.gate_proj.weight": mat(F, d), "f.up_proj.weight": mat(F, d),
         "f.down_proj.weight": mat(d, F), "e.weight": mat(V, d, s=1.0)}
    dev = {k: v.to(DEV).to(torch.float32 if (v.dim() == 1 or dt == torch.float32) else dt) for k, v in w.items()}
    w64 = {k: v.double() for k, v in w.items()}
    norm1 = RMSNorm(size=d, eps=eps, prefix="n1.", dtype=dt, device=DEV)
    norm2 = RMSNorm(size=d, eps=eps, prefix="n2.", dtype=dt, device=DEV)
    pos = RotaryPosition(theta=theta, rotary_dim=rot, head_dim=hd, dtype=dt, device=DEV)
    attn = Attention(hidden_size=d, n_heads=H, n_kv_heads=K, head_dim=hd, scale=hd ** -0.5, position=pos,
                     prefix="a.", dtype=dt, device=DEV)
    ffn = GatedMLP(hidden_size=d, intermediate_size=F, prefix="f.", dtype=dt, device=DEV)
    emb = Embedding(vocab_size=V, hidden_size=d, prefix="e.", dtype=dt, device=DEV)
    head = LMHead(vocab_size=V, hidden_size=d, tied=True, prefix="h.", dtype=dt, device=DEV)
    for part in (norm1, norm2, attn, ffn, emb):
        assert all(tuple(dev[part.prefix + n].shape) == tuple(s.shape) for n, s in part.params().items())
        part.bind({n: dev[part.prefix + n] for n in part.params()})
    head.tie(emb.weight)
    assert head.params() == {} and head.ignorable() == ["h.weight"]

    lens = [70, 3]
    toks = [torch.randint(0, V, (n,), generator=g).tolist() for n in lens]
    ctx = _ctx([0, 0], toks)
    # embedding
    x = emb.forward(ctx)
    x_ref = torch.cat([w64["e.weight"][t] for t in toks])
    assert torch.equal(x.double().cpu(), x_ref)
    # norm
    h = norm1.forward(x)
    h_ref = P.rmsnorm(x_ref, w64["n1.weight"], eps)
    assert h.dtype == dt and (h.double().cpu() - h_ref).abs().max() < tol * 4
    # feed-forward (adds into the residual)
    res = x.clone()
    ffn.forward(h, res)
    f_ref = P.swiglu(h.double().cpu(), w64["f.gate_proj.weight"], w64["f.up_proj.weight"], w64["f.down_proj.weight"])
    assert (res.double().cpu() - (x_ref + f_ref)).abs().max() < tol * (1 + f_ref.abs().max())
    # the same feed-forward with the gate's other activation
    ffn_g = GatedMLP(hidden_size=d, intermediate_size=F, activation="gelu", prefix="f.", dtype=dt, device=DEV)
    ffn_g.bind({n: dev["f." + n] for n in ffn_g.params()})
    res = x.clone()
    ffn_g.forward(h, res)
    g_ref = P.swiglu(h.double().cpu(), w64["f.gate_proj.weight"], w64["f.up_proj.weight"], w64["f.down_proj.weight"],
                     act="gelu")
    assert (res.double().cpu() - (x_ref + g_ref)).abs().max() < tol * (1 + g_ref.abs().max())
    assert (g_ref - f_ref).abs().max() > 100 * tol * (1 + f_ref.abs().max()) or dt != torch.float32
    with pytest.raises(ValueError, match="silu and gelu"):
        GatedMLP(hidden_size=d, intermediate_size=F, activation="relu", prefix="f.", dtype=dt, device=DEV)
    # attention over a fresh cache, two sequences of unequal length in one step
    cache = Cache([attn.cache_spec()], 256, 128, dt, DEV, 2)
    slots = [cache.alloc_slot(), cache.alloc_slot()]
    cache.grow(slots, lens)
    res = x.clone()
    attn.forward(h, ctx, cache.view(0), res)
    s = dict(n_heads=H, n_kv=K, hd=hd, theta=theta, rotary=rot)
    wa = {k: v for k, v in w64.items()}
    off, a_ref = 0, []
    for n in lens:
        a_ref.append(P.attention_part(h.double().cpu()[off:off + n], wa, "a.", s, torch.arange(n)))
        off += n
    a_ref = torch.cat(a_ref)
    assert (res.double().cpu() - (x_ref + a_ref)).abs().max() < tol * (1 + a_ref.abs().max())
    # the whole block on fresh slots equals norm -> attention -> norm -> feed-forward
    for sl in slots:
        cache.free_slot(sl)
    slots = [cache.alloc_slot(), cache.alloc_slot()]
    cache.grow(slots, lens)
    blk = PreNormBlock([SubLayer("mixer", attn, norm1), SubLayer("feed_forward", ffn, norm2)])
    xb = x.clone()
    blk.forward(xb, ctx, [cache.view(0)])
    wb = {"model.layers.0.input_layernorm.weight": w64["n1.weight"],
          "model.layers.0.post_attention_layernorm.weight": w64["n2.weight"]}
    for k in ("q_proj", "k_proj", "v_proj", "o_proj"):
        wb[f"model.layers.0.self_attn.{k}.weight"] = w64[f"a.{k}.weight"]
    for k in ("gate_proj", "up_proj", "down_proj"):
        wb[f"model.layers.0.mlp.{k}.weight"] = w64[f"f.{k}.weight"]
    s.update(eps=eps)
    off, b_ref = 0, []
    for n in lens:
        b_ref.append(P.block(x_ref[off:off + n], wb, 0, s, torch.arange(n)))
        off += n
    b_ref = torch.cat(b_ref)
    assert (xb.double().cpu() - b_ref).abs().max() < tol * (1 + b_ref.abs().max()) * 2
    # head on chosen rows
    rows = torch.tensor([69, 72, 0], dtype=torch.int32, device=DEV)
    logits = head.forward(norm2.forward(xb, rows))
    l_ref = P.linear(P.rmsnorm(xb.double().cpu()[rows.long().cpu()], w64["n2.weight"], eps), w64["e.weight"])
    assert logits.dtype == torch.float32 and (logits.double().cpu() - l_ref).abs().max() < tol * (1 + l_ref.abs().max())


@pytest.mark.parametrize("dt", [torch.float32, torch.float16])
@pytest.mark.parametrize("hd,H,K,rot", [(72, 3, 1, 72), (20, 4, 2, 10), (100, 2, 2, 50), (250, 1, 1, 250)])
def test_attention_part_with_head_sizes_that_are_no_multiple_of_16(dt, hd, H, K, rot):
    """The attention part alone at head sizes that the kernels do not take as they are: it runs them as
    the next multiple of 16 with zero rows and columns in its matrices, and the plain implementation at
    the true head size (scale 1/sqrt(hd), rotation of the first ``rot`` dimensions) is what it must match,
    for whole prompts and for decoded tokens.  Above 256 it refuses."""
    from llm_infer_amd.cache import Cache
    from llm_infer_amd.parts import Attention, RotaryPosition
    d, theta = 64, 3000.0
    g = torch.Generator().manual_seed(hd)
    w = {n: (torch.randn(*shape, generator=g) * s).to(torch.float16) for n, shape, s in (
        ("q_proj.weight", (H * hd, d), 0.3), ("k_proj.weight", (K * hd, d), 0.3), ("v_proj.weight", (K * hd, d), 0.2),
        ("o_proj.weight", (d, H * hd), 0.1))}
    pos = RotaryPosition(theta=theta, rotary_dim=rot, head_dim=hd, dtype=dt, device=DEV)
    attn = Attention(hidden_size=d, n_heads=H, n_kv_heads=K, head_dim=hd, scale=hd ** -0.5, position=pos,
                     prefix="a.", dtype=dt, device=DEV)
    assert attn.padded_head_dim == -(-hd // 16) * 16 and attn.cache_spec().head_dim == attn.padded_head_dim
    attn.bind({n: t.to(DEV).to(dt if dt != torch.float32 else torch.float32) for n, t in w.items()})
    lens = [70, 3]
    x = (torch.randn(sum(lens), d, generator=g)).to(dt)
    w64 = {"a." + n: t.double() for n, t in w.items()}
    s = dict(n_heads=H, n_kv=K, hd=hd, theta=theta, rotary=rot)
    ref, off = [], 0
    for n in lens:
        ref.append(P.attention_part(x.double()[off:off + n], w64, "a.", s, torch.arange(n)))
        off += n
    ref = torch.cat(ref)
    tol = (2e-5 if dt == torch.float32 else 6e-3) * (1 + ref.abs().max().item())
    cache = Cache([attn.cache_spec()], 256, 128, dt, DEV, 2)
    slots = [cache.alloc_slot(), cache.alloc_slot()]
    # whole prompts
    cache.grow(slots, lens)
    res = torch.zeros((sum(lens), d), dtype=torch.float32, device=DEV)
    attn.forward(x.to(DEV), _ctx([0, 0], [[0] * n for n in lens]), cache.view(0), res)
    assert (res.double().cpu() - ref).abs().max().item() < tol
    # the last token of each again, as a decode step over what the prompts left (positions n - 1 rewritten)
    for sl in slots:
        cache.free_slot(sl)
    slots = [cache.alloc_slot(), cache.alloc_slot()]
    cache.grow(slots, [n - 1 for n in lens])
    head = torch.cat([x[:lens[0] - 1], x[lens[0]:lens[0] + lens[1] - 1]])
    attn.forward(head.to(DEV), _ctx([0, 0], [[0] * (n - 1) for n in lens]), cache.view(0),
                 torch.zeros((head.shape[0], d), dtype=torch.float32, device=DEV))
    cache.grow(slots, lens)
    last = torch.stack([x[lens[0] - 1], x[-1]])
    res = torch.zeros((2, d), dtype=torch.float32, device=DEV)
    attn.forward(last.to(DEV), _ctx([n - 1 for n in lens], [[0], [0]]), cache.view(0), res)
    assert (res.double().cpu() - torch.stack([ref[lens[0] - 1], ref[-1]])).abs().max().item() < tol
    with pytest.raises(ValueError, match="up to 256"):
        Attention(hidden_size=d, n_heads=1, n_kv_heads=1, head_dim=272, scale=1.0, position=pos, prefix="a.",
                  dtype=dt, device=DEV)


# ---------------------------------------------------------------------------
# long decoding, the first tokens, graph replay
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_and_first_tokens(lib, folders, dtype):
    cfg, folder = TINY_C, folder_for(folders, "C", dtype)
    weights = P.load_weights(folder)
    n = 700
    toks = torch.randint(0, cfg["vocab_size"], (n,), generator=torch.Generator().manual_seed(2)).tolist()
    ref = P.forward(weights, cfg, toks, torch.float64)
    own = (P.forward(weights, cfg, toks, torch.float32) if dtype == "float32"
           else P.forward(weights, cfg, toks, torch.float64, ACT[dtype]))
    tol = 3 * (own.double() - ref).abs().max().item() + 1e-6
    eng = lib.load(folder, dtype=dtype, max_tokens=2048)
    s = eng.alloc_slot()
    got = [eng.step([s], [toks[:1]])[0]]                       # the very first token alone
    for p in range(1, n):                                      # then 699 tokens one by one, across 11 pages
        got.append(eng.step([s], [[toks[p]]])[0])
    got = torch.stack(got).double().cpu()
    err = (got - ref).abs().max(dim=1).values
    assert err.max().item() < tol, f"first wrong place: {int((err >= tol).nonzero()[0])}"
    assert err[:4].max().item() < tol                          # positions 0..3
    eng.free_slot(s)
    # a 2-token prompt in one step: both places
    s = eng.alloc_slot()
    two = eng.step([s], [toks[:2]], [[0, 1]]).double().cpu()
    assert (two - ref[:2]).abs().max().item() < tol
    eng.free_slot(s)


@pytest.mark.parametrize("name,cfg", [("A", TINY_A), ("B", TINY_B)])
def test_float32_with_the_references_float16_cache(lib, folders, name, cfg):
    """float32 activations with keys and values rounded to float16 on their way into the cache is the
    reference's own mix (src/model/block.cpp:145-148).  Rounding is not continuous: two correct
    implementations whose float32 sums differ in the last bit round a few elements to different
    neighbours, each a whole float16 step apart, so the largest difference of the logits is that of
    one unlucky element.  What is exact is checked exactly (the first layer's pages, whose inputs do
    not depend on the cache, and the result however the tokens are cut); the logits are compared by
    their root mean square, with the measure that the other tests use."""
    folder = folders[name]
    weights = P.load_weights(folder)
    n = 90
    toks = torch.randint(0, cfg["vocab_size"], (n,), generator=torch.Generator().manual_seed(4)).tolist()
    ref = P.forward(weights, cfg, toks, torch.float64, kv_dtype=torch.float16)
    own = P.forward(weights, cfg, toks, torch.float32, kv_dtype=torch.float16)
    unrounded = P.forward(weights, cfg, toks, torch.float64)
    rms = lambda a, b: (a.double() - b.double()).pow(2).mean().sqrt().item()
    eng = lib.load(folder, dtype="float32", max_tokens=256, kv_round="float16")
    s = eng.alloc_slot()
    got = [eng.step([s], [toks[:n - 8]], [list(range(n - 8))])]
    for t in toks[n - 8:]:
        got.append(eng.step([s], [[t]]))
    got = torch.cat(got).cpu()
    assert rms(got, ref) < 3 * rms(own, ref) + 1e-7
    # the rounding is there: an engine that did not round would fail the line above
    assert rms(got, unrounded) > 0.5 * rms(ref, unrounded) and rms(got, unrounded) > 2 * (3 * rms(own, ref) + 1e-7)
    whole = lib.load(folder, dtype="float32", max_tokens=256, kv_round="float16")
    assert whole.alloc_slot() == s
    assert torch.equal(whole.step([s], [toks], [list(range(n))]).cpu(), got)       # however it is cut
    # the first layer's keys and values: exactly the float16 neighbours of what an engine without the
    # option stores (round to nearest even, as f32_to_f16 of include/kernels_cpu.hpp:17)
    plain_cache = lib.load(folder, dtype="float32", max_tokens=256)
    assert plain_cache.alloc_slot() == s
    plain_cache.step([s], [toks], [[n - 1]])
    def first_layer(e):
        g = e.cache.groups[0]
        return g.storage.view(g.storage.shape[0], len(g.entries), g.layer_elems)[:, g.entries.index(0)]
    a, b = first_layer(whole), first_layer(plain_cache)
    assert torch.equal(a, b.half().float()) and not torch.equal(a, b) and int((b != 0).sum()) > n
    with pytest.raises(Exception, match="kv_round"):
        lib.load(folder, dtype="bfloat16", max_tokens=256, kv_round="float16")


@pytest.mark.parametrize("dtype", DTYPES)
def test_recorded_steps_replay_like_eager_steps(lib, folders, dtype):
    """Greedy generation of 150 tokens for a ragged batch whose sequences end at different times:
    the recorded (graph) runner and the eager runner must give the same tokens, replay after replay."""
    eng = lib.load(folder_for(folders, "C", dtype), dtype=dtype, max_tokens=8192)
    g = torch.Generator().manual_seed(3)
    prompts = [torch.randint(0, 331, (n,), generator=g).tolist() for n in (5, 90, 33, 64)]
    plain_tokens = eng.generate(prompts, max_new_tokens=150, temperature=0.0, use_graph=False)
    stop = {plain_tokens[1][40], plain_tokens[2][100]}          # make two sequences end early
    a = eng.generate(prompts, max_new_tokens=150, temperature=0.0, use_graph=False, stop_token_ids=stop)
    b = eng.generate(prompts, max_new_tokens=150, temperature=0.0, use_graph=True, stop_token_ids=stop)
    c = eng.generate(prompts, max_new_tokens=150, temperature=0.0, use_graph=True, stop_token_ids=stop)
    assert a == b == c
    assert len(a[1]) <= 40 and len(a[2]) <= 100 and len(a[0]) <= 150
    assert all(t not in stop for o in a for t in o)
    t1 = eng.generate(prompts, max_new_tokens=40, temperature=0.7, seed=5, use_graph=False)
    t2 = eng.generate(prompts, max_new_tokens=40, temperature=0.7, seed=5, use_graph=True)
    assert t1 == t2
    assert eng.cache.slots.n_free == eng.cache.n_slots and eng.cache.tokens_free() == (eng.cache.n_pages - 1) * 64


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_recorded_steps_at_bucket_edges_other_temperatures_and_after_eviction(lib, folders, dtype, monkeypatch):
    """What a recorded step is keyed by, each edge crossed: the bucket of context lengths (193 and 449 tokens
    are where the split count may change), the rows of the step (a batch that shrinks through the sizes 8,
    4, 2, 1 with idle rows in between), the temperature (read from the device: one recorded step, two
    temperatures), and a table of recorded steps so small that a step is dropped and recorded again."""
    from llm_infer_amd.engine import decode
    eng = lib.load(folder_for(folders, "C", dtype), dtype=dtype, max_tokens=16384)
    g = torch.Generator().manual_seed(11)
    prompts = [torch.randint(0, 331, (n,), generator=g).tolist() for n in (185, 440, 60, 189, 7, 445, 100, 3)]
    budgets = [16, 14, 3, 12, 5, 9, 7, 2]                       # the batch shrinks 8 -> 1, crossing both edges on the way
    eager = eng.generate(prompts, max_new_tokens=budgets, temperature=0.0, use_graph=False)
    assert [len(o) for o in eager] == budgets
    assert eng.decode_counts == {"eager": 0, "recorded": 0, "replayed": 0}
    first = eng.generate(prompts, max_new_tokens=budgets, temperature=0.0, use_graph=True)
    counts = dict(eng.decode_counts)
    again = eng.generate(prompts, max_new_tokens=budgets, temperature=0.0, use_graph=True)
    assert first == eager and again == eager
    assert counts["eager"] == 1 and counts["recorded"] >= 4 and counts["replayed"] >= 1
    assert eng.decode_counts["recorded"] == counts["recorded"]            # the second time every step was there
    rows = sorted({k[0] for k in eng._graphs})
    assert rows == [1, 2, 4, 8], rows                                     # 7, 6, 5 and 3 live sequences ran as 8, 8, 8 and 4 rows
    # two temperatures through the same recorded steps, against the eager runner with the same seeds
    for temperature in (0.7, 1.6):
        cold = eng.generate(prompts, max_new_tokens=budgets, temperature=temperature, seed=3, use_graph=False)
        warm = eng.generate(prompts, max_new_tokens=budgets, temperature=temperature, seed=3, use_graph=True)
        assert cold == warm, temperature
    recorded_hot = eng.decode_counts["recorded"]
    assert eng.generate(prompts, max_new_tokens=budgets, temperature=0.9, seed=3, use_graph=True) == \
        eng.generate(prompts, max_new_tokens=budgets, temperature=0.9, seed=3, use_graph=False)
    assert eng.decode_counts["recorded"] == recorded_hot                 # a third temperature recorded nothing
    # a table of two: steps are dropped while the batch shrinks and recorded again when they come back
    monkeypatch.setattr(decode, "MAX_RECORDED_STEPS", 2)
    before = eng.decode_counts["recorded"]
    for _ in range(2):
        assert eng.generate(prompts, max_new_tokens=budgets, temperature=0.0, use_graph=True) == eager
    assert len(eng._graphs) <= 2 and eng.decode_counts["recorded"] >= before + 6
    assert eng.cache.slots.n_free == eng.cache.n_slots and eng.cache.tokens_free() == (eng.cache.n_pages - 1) * 64


# ---------------------------------------------------------------------------
# slots and pages used again, batch composition
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_reused_slots_and_batch_composition(lib, folders, dtype):
    cfg, folder = TINY_B, folder_for(folders, "B", dtype)
    eng = lib.load(folder, dtype=dtype, max_tokens=64 * 6, n_slots=3)
    g = torch.Generator().manual_seed(9)
    reqs = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (100, 17, 64, 65, 1, 30)]

    def alone(toks):
        s = eng.alloc_slot()
        out = eng.step([s], [toks], [list(range(len(toks)))]).clone()
        eng.free_slot(s)
        return out

    base = [alone(t) for t in reqs]
    # poison everything that is free: a sequence that starts in a used slot and used pages sees none of it
    for grp in eng.cache.groups:
        grp.storage.fill_(float("nan"))
    again = [alone(t) for t in reqs]
    for x, y in zip(base, again):
        assert torch.equal(x, y)
    # batches of three with unequal lengths, in two orders: same logits for every request
    for order in ([0, 1, 2, 3, 4, 5], [4, 3, 5, 2, 0, 1]):
        for b in range(0, 6, 3):
            ids = order[b:b + 3]
            slots = [eng.alloc_slot() for _ in ids]
            out = eng.step(slots, [reqs[i] for i in ids], [list(range(len(reqs[i]))) for i in ids])
            off = 0
            for i in ids:
                part = out[off:off + len(reqs[i])]
                off += len(reqs[i])
                if dtype == "float32":
                    assert torch.equal(part, base[i]), "32-bit results do not depend on the batch"
                else:
                    assert (part - base[i]).abs().max().item() < 2e-2 * base[i].std().item()
            for s in slots:
                eng.free_slot(s)
    with pytest.raises(Exception, match="cache is full|in use"):
        slots = [eng.alloc_slot() for _ in range(3)]
        eng.step(slots, [reqs[0] + reqs[0], reqs[0] + reqs[0], reqs[0] + reqs[0]])


def test_many_sequences_in_one_batch(lib, folders):
    """150 sequences of unequal lengths as one batch (more rows than the decode kernels' small-batch
    paths take, page tables of many slots): in float32 every sequence's logits and greedy tokens are
    bit-equal to those it has alone."""
    import random
    cfg, folder = TINY_C, folders["C"]
    rng = random.Random(3)
    prompts = [[rng.randrange(cfg["vocab_size"]) for _ in range(rng.choice([1, 2, 5, 17, 40, 63, 64, 65]))]
               for _ in range(150)]
    eng = lib.load(folder, dtype="float32", max_tokens=150 * 128)
    out = eng.generate(prompts, max_new_tokens=12, temperature=0.0)
    slots = [eng.alloc_slot() for _ in prompts]
    together = eng.step(slots, prompts).cpu()
    one = lib.load(folder, dtype="float32", max_tokens=1024)
    for i in range(0, 150, 11):
        assert one.generate([prompts[i]], max_new_tokens=12, temperature=0.0)[0] == out[i], i
        s = one.alloc_slot()
        assert torch.equal(one.step([s], [prompts[i]]).cpu()[0], together[i]), i
        one.free_slot(s)


@pytest.mark.parametrize("dtype", DTYPES)
def test_prompt_in_several_chunks(lib, folders, dtype):
    """A prompt fed in chunks of several tokens (each chunk attends to the cache of the chunks before
    it and causally to itself), next to a sequence that is decoding: same logits as the whole prompt."""
    cfg, folder = TINY_A, folder_for(folders, "A", dtype)
    weights = P.load_weights(folder)
    eng = lib.load(folder, dtype=dtype, max_tokens=1024)
    g = torch.Generator().manual_seed(4)
    a = torch.randint(0, 256, (120,), generator=g).tolist()
    b = torch.randint(0, 256, (90,), generator=g).tolist()
    ref_a, ref_b = (P.forward(weights, cfg, t, torch.float64) for t in (a, b))
    own = (P.forward(weights, cfg, a, torch.float32) if dtype == "float32"
           else P.forward(weights, cfg, a, torch.float64, ACT[dtype]))
    tol = 3 * (own.double() - ref_a).abs().max().item() + 1e-6
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    eng.step([sb], [b[:60]])
    cuts = [0, 5, 64, 65, 100, 120]
    got = []
    for i, (lo, hi) in enumerate(zip(cuts, cuts[1:])):
        out = eng.step([sa, sb], [a[lo:hi], [b[60 + i]]], [list(range(hi - lo)), [0]])
        got.append(out[:hi - lo])
        assert (out[hi - lo].double().cpu() - ref_b[60 + i]).abs().max().item() < tol
    got = torch.cat(got).double().cpu()
    assert (got - ref_a).abs().max().item() < tol


def test_requests_are_checked(lib, folders):
    eng = lib.load(folders["A"], dtype="bfloat16", max_tokens=256)
    s = eng.alloc_slot()
    with pytest.raises(ValueError, match="token id outside"):
        eng.step([s], [[1, 256]])
    with pytest.raises(ValueError, match="brings no token"):
        eng.step([s], [[]])
    with pytest.raises(ValueError, match="wanted place"):
        eng.step([s], [[1, 2]], [[2]])
    with pytest.raises(Exception, match="exceeds the model's 128 positions"):
        eng.step([s], [list(range(129))])
    from llm_infer_amd.engine.generate import RequestError
    with pytest.raises(RequestError, match="Prompt too long: 128 tokens \\(max: 128\\)"):
        eng.generate([list(range(128))], max_new_tokens=1)


# ---------------------------------------------------------------------------
# sampling through the entry points
# ---------------------------------------------------------------------------
def test_temperature_sampling_follows_the_plain_sampler(lib, folders):
    """float32 engine, T = 0.8: every token equals the plain sampler's choice for the same uniform
    number, unless that number falls within rounding of a boundary of the cumulative distribution."""
    from llm_infer_amd.sampling import Sampler
    cfg, folder = TINY_B, folders["B"]
    weights = P.load_weights(folder)
    eng = lib.load(folder, dtype="float32", max_tokens=1024)
    prompts = [[5], [1, 2, 3, 4], list(range(10, 19)), list(range(40, 56)), list(range(100, 131))]
    T, seed, n_new = 0.8, 1, 12
    out = eng.generate(prompts, max_new_tokens=n_new, temperature=T, seed=seed, stop_token_ids=())
    sampler = Sampler(T, seed)
    for r_idx, (p, o) in enumerate(zip(prompts, out)):
        assert len(o) == n_new
        toks = list(p)
        for k, t in enumerate(o):
            logits = P.forward(weights, cfg, toks, torch.float64)[-1]
            r = sampler.uniform(r_idx, k)
            c = torch.cumsum(P.probabilities(logits, T), 0)
            if (c - r).abs().min().item() > 1e-5:
                assert t == P.sample_temperature(logits, T, r), (r_idx, k)
            toks.append(t)
    # a request's tokens do not depend on the batch it runs in, only on (seed, request index)
    alone = eng.generate([prompts[0]], max_new_tokens=n_new, temperature=T, seed=seed, stop_token_ids=())
    assert alone[0] == out[0]
    other = eng.generate(prompts, max_new_tokens=n_new, temperature=T, seed=seed + 1, stop_token_ids=())
    assert other != out
    # one batch after another: a single slot serves all five requests
    small = lib.load(folder, dtype="float32", max_tokens=64, n_slots=1)
    serial, stats = small.generate(prompts, max_new_tokens=n_new, temperature=T, seed=seed, stop_token_ids=(),
                                   return_stats=True)
    assert serial == out and stats.batches == 5


def test_command_line_generates_greedily(folders):
    cfg, folder = TINY_A, folders["A"]
    weights = P.load_weights(folder)
    prompts = [[3, 14, 15, 92, 65, 35, 89], [7], list(range(20, 33))]
    cmd = [sys.executable, os.path.join(ROOT, "bin", "infer"), folder, "-n", "8", "-t", "0", "--dtype", "float32"]
    for p in prompts:
        cmd += ["--tokens", ",".join(map(str, p))]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr
    got = [json.loads(line.split("tokens: ", 1)[1]) for line in res.stdout.splitlines() if " tokens: [" in line]
    assert got == [P.generate_greedy(weights, cfg, p, 8) for p in prompts]
    for word in ("Loading model:", "Layers: 2", "KV Heads: 2", "Prefilling...", "Generation Statistics:",
                 "Prompt tokens: 21", "Generated tokens: 24", "Temperature: 0.00"):
        assert word in res.stdout
    bad = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "infer"), folder + "_nope", "--tokens", "1"],
                         capture_output=True, text=True, timeout=300)
    assert bad.returncode == 1 and "Error:" in bad.stderr
    # two slots for three requests (two batches, the slots used again), random weights from a
    # configuration file alone: the same tokens as the library gives for that seed
    cmd = [sys.executable, os.path.join(ROOT, "bin", "infer"), "-", "--random-weights", "--seed-weights", "5",
           "--config", os.path.join(folder, "config.json"), "--slots", "2", "-n", "6", "-t", "0", "--dtype", "float32"]
    for p in prompts:
        cmd += ["--tokens", ",".join(map(str, p))]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr
    got = [json.loads(line.split("tokens: ", 1)[1]) for line in res.stdout.splitlines() if " tokens: [" in line]
    import llm_infer_amd
    eng = llm_infer_amd.random_model(llm_infer_amd.config_from_folder(folder), seed=5, dtype="float32", max_tokens=512)
    assert got == eng.generate(prompts, max_new_tokens=6, temperature=0.0)


def test_a_gguf_file_runs_like_the_folder(lib, folders, tmp_path):
    """The reference's own model format: the same weights as one GGUF file (its tensor names, its
    metadata keys, a vocabulary inside) give the same logits as the folder, through the library
    and through the command line with a text prompt."""
    from llm_infer_amd.weights import write_gguf
    cfg = lib.config_from_dict(TINY_B)
    weights = P.load_weights(folders["B"])
    path = str(tmp_path / "tiny.gguf")
    vocab = [f"<{i}>" for i in range(cfg.vocab_size)]
    vocab[65:91] = [chr(c) for c in range(65, 91)]                       # "A".."Z" are tokens 65..90
    md = dict(cfg.gguf_metadata(), **{"tokenizer.ggml.tokens": vocab})
    write_gguf(path, md, {cfg.gguf_tensor_name(n): (t.float() if t.dim() == 1 else t) for n, t in weights.items()})
    prompt = [72, 69, 76, 76, 79]                                         # "HELLO"
    a = lib.load(folders["B"], dtype="float32", max_tokens=256)
    b = lib.load(path, dtype="float32", max_tokens=256)
    la = a.step([a.alloc_slot()], [prompt], [list(range(5))])
    lb = b.step([b.alloc_slot()], [prompt], [list(range(5))])
    assert torch.equal(la, lb)
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "infer"), path, "-i", "HELLO", "-n", "6",
                          "-t", "0", "--dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr
    got = [json.loads(line.split("tokens: ", 1)[1]) for line in res.stdout.splitlines() if " tokens: [" in line]
    assert got == [P.generate_greedy(weights, TINY_B, prompt, 6)]
    assert "Prompt tokens: 5" in res.stdout


# ---------------------------------------------------------------------------
# a toy architecture, defined here
# ---------------------------------------------------------------------------
def test_toy_architecture_with_a_stateful_mixer(lib):
    from llm_infer_amd.cache import StateSpec
    from llm_infer_amd.config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from llm_infer_amd.engine import Engine
    from llm_infer_amd.parts.base import Part
    from llm_infer_amd.weights.loader import ParamSpec

    @lib.register_mixer("toy_decay")
    class DecayMixer(Part):
        """s <- decay * s + W_in h ;  out = W_out s, with s kept per sequence in the cache."""

        def __init__(self, *, hidden_size, state_size, decay, position=None, prefix, dtype, device):
            self.d, self.n, self.decay, self.prefix, self.dtype = hidden_size, state_size, decay, prefix, dtype

        def params(self):
            return {"in.weight": ParamSpec((self.n, self.d)), "out.weight": ParamSpec((self.d, self.n))}

        def bind(self, tensors):
            self.w_in, self.w_out = tensors["in.weight"].float(), tensors["out.weight"].float()

        def cache_spec(self):
            return StateSpec((self.n,), "float32")

        def forward(self, h, ctx, cache_view, residual, owns_cache=True):
            u = h.float() @ self.w_in.t()
            y = torch.empty_like(u)
            row = 0
            for slot, n in zip(ctx.host_slots, ctx.host_qlens):
                s = cache_view.state[slot].clone()
                for _ in range(n):
                    s = self.decay * s + u[row]
                    y[row] = s
                    row += 1
                cache_view.state[slot] = s
            residual += y @ self.w_out.t()

    class ToyConfig:
        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def model_spec(self):
            r = self.raw
            d, hd = r["width"], r["head"]
            norm = PartSpec("rmsnorm", {"size": d, "eps": r["eps"]})
            ffn = PartSpec("gated_mlp", {"hidden_size": d, "intermediate_size": r["ffn"]})
            toy = LayerSpec.mixer_then_feed_forward("pre_norm", PartSpec("toy_decay", {"hidden_size": d, "state_size": r["state"],
                                                               "decay": r["decay"]}, "l0.mix."),
                            ffn.with_prefix("l0.ffn."), norm.with_prefix("l0.n1."), norm.with_prefix("l0.n2."))
            att = LayerSpec.mixer_then_feed_forward("pre_norm", PartSpec("attention", {"hidden_size": d, "n_heads": 2, "n_kv_heads": 1,
                                                               "head_dim": hd, "scale": hd ** -0.5}, "l1.mix."),
                            ffn.with_prefix("l1.ffn."), norm.with_prefix("l1.n1."), norm.with_prefix("l1.n2."),
                            PartSpec("rope", {"theta": 100.0, "rotary_dim": hd, "head_dim": hd}))
            # the toy layer runs twice (two states), the attention layer runs twice, its second run
            # reading the keys and values that its first run stored
            schedule = (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1, cache_from=1))
            return ModelSpec(d, r["vocab"], r["positions"],
                             PartSpec("embedding", {"vocab_size": r["vocab"], "hidden_size": d}, "emb."),
                             (toy, att), schedule, norm.with_prefix("final."),
                             PartSpec("lm_head", {"vocab_size": r["vocab"], "hidden_size": d, "tied": True}, "head."))

    lib.register_architecture("ToyForCausalLM", ToyConfig)
    raw = {"architectures": ["ToyForCausalLM"], "width": 48, "head": 16, "ffn": 40, "state": 24, "decay": 0.9,
           "eps": 1e-5, "vocab": 50, "positions": 256}
    cfg = lib.config_from_dict(raw)
    eng = Engine.from_random(cfg, seed=1, dtype="float32", max_tokens=512, stored_dtype="float32")
    model = eng.model
    assert sorted(type(g).__name__ for g in eng.cache.groups) == ["KVGroup", "StateGroup"]
    assert [s is None for s in model.cache_specs()] == [False, False, False, True]

    # plain float64 reference of this toy model, whole sequence
    W = {}
    for layer, p in zip(model.layers, ("l0.", "l1.")):
        W[p + "n1"], W[p + "n2"] = layer.mixer_norm.weight.double().cpu(), layer.feed_forward_norm.weight.double().cpu()
        gu = layer.feed_forward.w_gate_up.double().cpu()
        W[p + "gate"], W[p + "up"], W[p + "down"] = gu[0::2], gu[1::2], layer.feed_forward.w_down.double().cpu()
    toy, att = model.layers[0].mixer, model.layers[1].mixer
    wq, wk, wv = att.wqkv.double().cpu().split([32, 16, 16])
    wo = att.wo.double().cpu()

    def ref_forward(toks):
        n = len(toks)
        x = model.embedding.weight.double().cpu()[toks]
        posn = torch.arange(n)
        kv = None
        for entry in (0, 1, 2, 3):
            p = "l0." if entry in (0, 2) else "l1."
            h = P.rmsnorm(x, W[p + "n1"], 1e-5)
            if p == "l0.":
                u = h @ toy.w_in.double().cpu().t()
                s, ys = torch.zeros(24, dtype=torch.float64), []
                for t in range(n):
                    s = 0.9 * s + u[t]
                    ys.append(s)
                x = x + torch.stack(ys) @ toy.w_out.double().cpu().t()
            else:
                q = P.rope((h @ wq.t()).view(n, 2, 16), posn, 100.0, 16)
                if entry == 1:
                    kv = (P.rope((h @ wk.t()).view(n, 1, 16), posn, 100.0, 16), (h @ wv.t()).view(n, 1, 16))
                x = x + P.attention(q, kv[0], kv[1]).reshape(n, 32) @ wo.t()
            x = x + P.swiglu(P.rmsnorm(x, W[p + "n2"], 1e-5), W[p + "gate"], W[p + "up"], W[p + "down"])
        return P.rmsnorm(x, model.final_norm.weight.double().cpu(), 1e-5) @ model.embedding.weight.double().cpu().t()

    g = torch.Generator().manual_seed(0)
    seqs = [torch.randint(0, 50, (n,), generator=g).tolist() for n in (70, 9, 130)]
    refs = [ref_forward(t) for t in seqs]
    # whole, in one ragged batch
    slots = [eng.alloc_slot() for _ in seqs]
    out = eng.step(slots, seqs, [list(range(len(t))) for t in seqs]).double().cpu()
    assert (out - torch.cat(refs)).abs().max().item() < 2e-5
    for s in slots:
        eng.free_slot(s)
    # cut: a first part, then token by token; the state is carried from step to step and reset on reuse
    slots = [eng.alloc_slot() for _ in seqs]
    heads = [len(t) - 5 for t in seqs]
    out = eng.step(slots, [t[:h] for t, h in zip(seqs, heads)]).double().cpu()
    for i, (r, h) in enumerate(zip(refs, heads)):
        assert (out[i] - r[h - 1]).abs().max().item() < 2e-5
    for k in range(5):
        out = eng.step(slots, [[t[h + k]] for t, h in zip(seqs, heads)]).double().cpu()
        for i, (r, h) in enumerate(zip(refs, heads)):
            assert (out[i] - r[h + k]).abs().max().item() < 2e-5
    for s in slots:
        eng.free_slot(s)
    toks = eng.generate([seqs[1]], max_new_tokens=4, temperature=0.0, use_graph=False)[0]
    assert toks[0] == int(refs[1][-1].argmax())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_with_a_window_group(lib, dtype):
    """Two attention layers with different needs, all keys and a window of 70: two cache groups with
    pools and page tables of their own; the window group gives pages back while a sequence grows."""
    from llm_infer_amd.config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from llm_infer_amd.engine import Engine

    class WindowConfig:
        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def model_spec(self):
            d, hd = 64, 32
            norm = PartSpec("rmsnorm", {"size": d, "eps": 1e-5})
            ffn = PartSpec("gated_mlp", {"hidden_size": d, "intermediate_size": 96})
            rope = PartSpec("rope", {"theta": 1000.0, "rotary_dim": hd, "head_dim": hd})
            layers = []
            for i, window in enumerate((None, 70)):
                att = PartSpec("attention", {"hidden_size": d, "n_heads": 2, "n_kv_heads": 2, "head_dim": hd,
                                             "scale": hd ** -0.5, "window": window}, f"l{i}.mix.")
                layers.append(LayerSpec.mixer_then_feed_forward("pre_norm", att, ffn.with_prefix(f"l{i}.ffn."), norm.with_prefix(f"l{i}.n1."),
                                        norm.with_prefix(f"l{i}.n2."), rope))
            return ModelSpec(d, 40, 512, PartSpec("embedding", {"vocab_size": 40, "hidden_size": d}, "emb."),
                             tuple(layers), (ScheduleEntry(0), ScheduleEntry(1)), norm.with_prefix("final."),
                             PartSpec("lm_head", {"vocab_size": 40, "hidden_size": d, "tied": True}, "head."))

    lib.register_architecture("WindowToyForCausalLM", WindowConfig)
    cfg = lib.config_from_dict({"architectures": ["WindowToyForCausalLM"]})
    eng = Engine.from_random(cfg, seed=2, dtype=dtype, max_tokens=1024, stored_dtype="bfloat16")
    model, cache = eng.model, eng.cache
    groups = {g.spec.window: g for g in cache.groups}
    assert set(groups) == {None, 70}

    emb = model.embedding.weight.double().cpu()
    fin = model.final_norm.weight.double().cpu()

    def rows(w):                                     # a weight back in plain row order, whatever its layout
        from llm_infer_amd.kernels import ops
        if ops.is_tiled(w):
            eye = torch.eye(w.logical[1], dtype=w.dtype, device=DEV)
            return ops.linear(eye, w, out_dtype=torch.float32).t().double().cpu()
        return w.double().cpu()

    def ref_forward(toks):
        n = len(toks)
        x = emb[toks]
        posn = torch.arange(n)
        for layer, window in zip(model.layers, (None, 70)):
            att, ffn = layer.mixer, layer.feed_forward
            wq, wk, wv = rows(att.wqkv).split([64, 64, 64])
            h = P.rmsnorm(x, layer.mixer_norm.weight.double().cpu(), 1e-5)
            q = P.rope((h @ wq.t()).view(n, 2, 32), posn, 1000.0, 32)
            k = P.rope((h @ wk.t()).view(n, 2, 32), posn, 1000.0, 32)
            v = (h @ wv.t()).view(n, 2, 32)
            x = x + P.attention(q, k, v, window).reshape(n, 64) @ rows(att.wo).t()
            gu = rows(ffn.w_gate_up)
            x = x + P.swiglu(P.rmsnorm(x, layer.feed_forward_norm.weight.double().cpu(), 1e-5), gu[0::2], gu[1::2],
                             rows(ffn.w_down))
        return P.rmsnorm(x, fin, 1e-5) @ emb.t()

    toks = torch.randint(0, 40, (300,), generator=torch.Generator().manual_seed(1)).tolist()
    ref = ref_forward(toks)
    tol = 1e-5 if dtype == "float32" else 4e-2 * ref.std().item()
    s = eng.alloc_slot()
    got = [eng.step([s], [toks[:150]], [list(range(150))])]
    assert sorted(groups[70].pages_of[s]) == [1, 2] and sorted(groups[None].pages_of[s]) == [0, 1, 2]
    for p in range(150, 300):
        got.append(eng.step([s], [[toks[p]]]))
    assert sorted(groups[70].pages_of[s]) == [3, 4] and sorted(groups[None].pages_of[s]) == [0, 1, 2, 3, 4]
    got = torch.cat(got).double().cpu()
    err = (got - ref).abs().max(dim=1).values
    assert err.max().item() < tol, f"first wrong place: {int((err >= tol).nonzero()[0])}"
    eng.free_slot(s)
    assert groups[70].pool.n_free == groups[None].pool.n_free == cache.n_pages - 1


# ---------------------------------------------------------------------------
# a toy feed-forward with routing and a toy position encoding, both defined here
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_routed_feed_forward_and_another_position_encoding(lib, dtype):
    """A feed-forward that sends every token to one of three experts (router logits and weights in
    float32) and a rotation whose angles are those of position / 4: registered from the test, built
    by the registry from a config, run by the engine whole, cut and in a ragged batch.  Nothing in
    the framework's files names either."""
    from llm_infer_amd.config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from llm_infer_amd.engine import Engine
    from llm_infer_amd.kernels import ops
    from llm_infer_amd.parts.base import Part
    from llm_infer_amd.parts.position import RotaryPosition
    from llm_infer_amd.weights.loader import ParamSpec

    @lib.register_feed_forward("toy_top1")
    class Top1Experts(Part):
        recordable = False            # the rows of an expert are counted on the host

        def __init__(self, *, hidden_size, expert_size, n_experts, prefix, dtype, device):
            self.d, self.f, self.e, self.prefix, self.dtype = hidden_size, expert_size, n_experts, prefix, dtype

        def params(self):
            p = {"router.weight": ParamSpec((self.e, self.d))}
            for i in range(self.e):
                p[f"experts.{i}.up.weight"] = ParamSpec((self.f, self.d))
                p[f"experts.{i}.down.weight"] = ParamSpec((self.d, self.f))
            return p

        def bind(self, tensors):
            self.router = tensors["router.weight"].float()
            self.up = [tensors[f"experts.{i}.up.weight"] for i in range(self.e)]
            self.down = [tensors[f"experts.{i}.down.weight"] for i in range(self.e)]

        def forward(self, h, residual):
            logits = ops.linear(h.float(), self.router, out_dtype=torch.float32)       # float32 router
            weight, pick = torch.softmax(logits, dim=-1).max(dim=-1)
            for i in range(self.e):
                rows = (pick == i).nonzero().flatten()
                if rows.numel() == 0:
                    continue
                a = torch.relu(ops.linear(h[rows].contiguous(), self.up[i], out_dtype=torch.float32))
                y = ops.linear(a.to(self.dtype), self.down[i], out_dtype=torch.float32)
                residual.index_add_(0, rows, y * weight[rows, None])

    @lib.register_position("toy_slow_rope")
    class SlowRotary(RotaryPosition):
        """The rotation of position / slowdown: only the table of frequencies differs."""

        def __init__(self, *, slowdown, **kw):
            super().__init__(**kw)
            self.inv_freq = self.inv_freq / float(slowdown)

    class RoutedConfig:
        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def model_spec(self):
            r = self.raw
            d, hd = r["width"], r["head"]
            norm = PartSpec("rmsnorm", {"size": d, "eps": r["eps"]})
            layers = []
            for i in range(2):
                mix = PartSpec("attention", {"hidden_size": d, "n_heads": 3, "n_kv_heads": 3, "head_dim": hd,
                                             "scale": hd ** -0.5}, f"l{i}.mix.")
                ffn = PartSpec("toy_top1", {"hidden_size": d, "expert_size": r["expert"], "n_experts": 3}, f"l{i}.moe.")
                pos = PartSpec("toy_slow_rope", {"theta": 50.0, "rotary_dim": hd, "head_dim": hd, "slowdown": 4.0})
                layers.append(LayerSpec.mixer_then_feed_forward("pre_norm", mix, ffn, norm.with_prefix(f"l{i}.n1."),
                                        norm.with_prefix(f"l{i}.n2."), pos))
            return ModelSpec(d, r["vocab"], r["positions"],
                             PartSpec("embedding", {"vocab_size": r["vocab"], "hidden_size": d}, "emb."),
                             tuple(layers), (ScheduleEntry(0), ScheduleEntry(1)), norm.with_prefix("final."),
                             PartSpec("lm_head", {"vocab_size": r["vocab"], "hidden_size": d, "tied": False}, "head."))

    lib.register_architecture("RoutedToyForCausalLM", RoutedConfig)
    raw = {"architectures": ["RoutedToyForCausalLM"], "width": 64, "head": 16, "expert": 40, "eps": 1e-6,
           "vocab": 70, "positions": 256}
    eng = Engine.from_random(lib.config_from_dict(raw), seed=4, dtype=dtype, max_tokens=512)
    # the same weights (values that bfloat16 holds) as plain float32 tensors, for the reference
    model = Engine.from_random(lib.config_from_dict(raw), seed=4, dtype="float32", max_tokens=64).model

    # random routers are indifferent; scaled up they decide, so that a wrong choice would show
    for m_ in (eng.model, model):
        for layer in m_.layers:
            layer.feed_forward.router *= 30.0

    def dbl(t):
        return t.double().cpu()

    def ref_forward(toks):
        """float64, whole sequence; the expert of a token is taken from the engine's own choice only
        where the two best router logits are closer than rounding could decide."""
        n = len(toks)
        x = dbl(model.embedding.weight)[toks]
        posn = torch.arange(n, dtype=torch.float64) / 4.0
        for layer in model.layers:
            att, moe = layer.mixer, layer.feed_forward
            h = P.rmsnorm(x, dbl(layer.mixer_norm.weight), 1e-6)
            wq, wk, wv = dbl(att.wqkv).split([48, 48, 48])
            q = P.rope((h @ wq.t()).view(n, 3, 16), posn, 50.0, 16)
            k = P.rope((h @ wk.t()).view(n, 3, 16), posn, 50.0, 16)
            x = x + P.attention(q, k, (h @ wv.t()).view(n, 3, 16)).reshape(n, 48) @ dbl(att.wo).t()
            h = P.rmsnorm(x, dbl(layer.feed_forward_norm.weight), 1e-6)
            prob = torch.softmax(h @ moe.router.double().cpu().t(), dim=-1)
            weight, pick = prob.max(dim=-1)
            top2 = prob.topk(2, dim=-1).values
            sure = (top2[:, 0] - top2[:, 1]) > 0.05
            y = torch.zeros_like(x)
            for t in range(n):
                e = int(pick[t])
                y[t] = weight[t] * (torch.relu(h[t] @ dbl(moe.up[e]).t()) @ dbl(moe.down[e]).t())
            x = x + y
        return P.rmsnorm(x, dbl(model.final_norm.weight), 1e-6) @ dbl(model.head.weight).t(), sure

    g = torch.Generator().manual_seed(11)
    seqs = [torch.randint(0, 70, (n,), generator=g).tolist() for n in (40, 7, 90)]
    tol = 3e-5 if dtype == "float32" else 3e-2
    slots = [eng.alloc_slot() for _ in seqs]
    whole = eng.step(slots, seqs, [list(range(len(t))) for t in seqs]).double().cpu()
    for s in slots:
        eng.free_slot(s)
    off = 0
    for toks in seqs:
        ref, sure = ref_forward(toks)
        # a token whose router was too close to call may differ from there on: compare up to it
        upto = len(toks) if bool(sure.all()) else int((~sure).nonzero()[0])
        scale = ref.abs().max().item()
        assert upto >= min(5, len(toks))
        assert (whole[off:off + upto] - ref[:upto]).abs().max().item() < tol * (1 + scale)
        off += len(toks)
    # cut: a first part, then one token at a time, against the engine's own whole run
    slots = [eng.alloc_slot() for _ in seqs]
    heads = [len(t) - 4 for t in seqs]
    eng.step(slots, [t[:h] for t, h in zip(seqs, heads)])
    starts = [0, len(seqs[0]), len(seqs[0]) + len(seqs[1])]
    for kk in range(4):
        out = eng.step(slots, [[t[h + kk]] for t, h in zip(seqs, heads)]).double().cpu()
        for i, (h, st) in enumerate(zip(heads, starts)):
            assert (out[i] - whole[st + h + kk]).abs().max().item() < tol * (1 + whole.abs().max().item())
    for s in slots:
        eng.free_slot(s)
    a = eng.generate([seqs[1], seqs[0]], max_new_tokens=6, temperature=0.0, use_graph=True)
    b = eng.generate([seqs[1], seqs[0]], max_new_tokens=6, temperature=0.0, use_graph=False)
    assert a == b and all(len(o) == 6 for o in a)


# ---------------------------------------------------------------------------
# a toy norm and a toy arrangement of a block, both defined here
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_norm_and_parallel_block(lib, dtype):
    """A norm with mean and bias (LayerNorm) and a block whose mixer and feed-forward both read the
    same normed input (parallel residual): registered from here, chosen by a configuration, run
    whole, cut and through generation, against a float64 reference of the same toy model."""
    from llm_infer_amd.config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
    from llm_infer_amd.engine import Engine
    from llm_infer_amd.parts.base import Part
    from llm_infer_amd.weights.loader import ParamSpec

    @lib.register_norm("toy_layernorm")
    class LayerNorm(Part):
        def __init__(self, *, size, eps, prefix, dtype, device):
            self.size, self.eps, self.prefix, self.dtype = size, eps, prefix, dtype

        def params(self):
            return {"weight": ParamSpec((self.size,), "vector", "ones"), "bias": ParamSpec((self.size,), "vector")}

        def bind(self, tensors):
            self.weight, self.bias = tensors["weight"], tensors["bias"]

        def forward(self, x, rows=None):
            if rows is not None:
                x = x[rows.long()]
            y = torch.nn.functional.layer_norm(x, (self.size,), self.weight, self.bias, self.eps)   # float32
            return y.to(self.dtype)

    @lib.register_block("toy_parallel")
    class ParallelBlock(Part):
        """x += mixer(n(x)) + feed_forward(n(x)) with one norm; the second norm of the spec is unused."""

        def __init__(self, sublayers):
            mix, ffn = sublayers
            self.norm, self.mixer, self.feed_forward = mix.norm, mix.part, ffn.part

        def children(self):
            return [self.norm, self.mixer, self.feed_forward]

        def forward(self, x, ctx, cache_views, owns_cache=True):
            h = self.norm.forward(x)
            self.mixer.forward(h, ctx, cache_views[0], x, owns_cache)
            self.feed_forward.forward(h, x)

    class ParallelConfig:
        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def model_spec(self):
            r = self.raw
            d, hd = r["width"], r["head"]
            layers = []
            for i in range(r["layers"]):
                norm = PartSpec("toy_layernorm", {"size": d, "eps": r["eps"]}, f"h.{i}.ln.")
                mix = PartSpec("attention", {"hidden_size": d, "n_heads": 4, "n_kv_heads": 2, "head_dim": hd,
                                             "scale": hd ** -0.5}, f"h.{i}.attn.")
                ffn = PartSpec("gated_mlp", {"hidden_size": d, "intermediate_size": r["ffn"]}, f"h.{i}.mlp.")
                pos = PartSpec("rope", {"theta": 777.0, "rotary_dim": hd // 2, "head_dim": hd})
                layers.append(LayerSpec.mixer_then_feed_forward("toy_parallel", mix, ffn, norm, norm, pos))
            return ModelSpec(d, r["vocab"], r["positions"],
                             PartSpec("embedding", {"vocab_size": r["vocab"], "hidden_size": d}, "wte."),
                             tuple(layers), tuple(ScheduleEntry(i) for i in range(r["layers"])),
                             PartSpec("toy_layernorm", {"size": d, "eps": r["eps"]}, "ln_f."),
                             PartSpec("lm_head", {"vocab_size": r["vocab"], "hidden_size": d, "tied": True}, "head."))

    lib.register_architecture("ParallelToyForCausalLM", ParallelConfig)
    raw = {"architectures": ["ParallelToyForCausalLM"], "width": 96, "head": 32, "ffn": 120, "eps": 1e-5,
           "vocab": 90, "positions": 512, "layers": 2}
    eng = Engine.from_random(lib.config_from_dict(raw), seed=8, dtype=dtype, max_tokens=1024)
    model = Engine.from_random(lib.config_from_dict(raw), seed=8, dtype="float32", max_tokens=64).model
    for m_ in (eng.model, model):                       # biases that matter
        for part in [b.norm for b in m_.layers] + [m_.final_norm]:
            part.bias += 0.1 * torch.arange(96, device=part.bias.device, dtype=torch.float32).cos()

    def dbl(t):
        return t.double().cpu()

    def layernorm(x, part):
        mu = x.mean(-1, keepdim=True)
        var = ((x - mu) ** 2).mean(-1, keepdim=True)
        return (x - mu) / torch.sqrt(var + 1e-5) * dbl(part.weight) + dbl(part.bias)

    def ref_forward(toks):
        n = len(toks)
        x = dbl(model.embedding.weight)[toks]
        posn = torch.arange(n)
        for layer in model.layers:
            att, ffn = layer.mixer, layer.feed_forward
            h = layernorm(x, layer.norm)
            wq, wk, wv = dbl(att.wqkv).split([128, 64, 64])
            q = P.rope((h @ wq.t()).view(n, 4, 32), posn, 777.0, 16)
            k = P.rope((h @ wk.t()).view(n, 2, 32), posn, 777.0, 16)
            a = P.attention(q, k, (h @ wv.t()).view(n, 2, 32)).reshape(n, 128) @ dbl(att.wo).t()
            gu = dbl(ffn.w_gate_up)
            x = x + a + P.swiglu(h, gu[0::2], gu[1::2], dbl(ffn.w_down))
        return layernorm(x, model.final_norm) @ dbl(model.embedding.weight).t()

    g = torch.Generator().manual_seed(2)
    seqs = [torch.randint(0, 90, (n,), generator=g).tolist() for n in (150, 3, 66)]
    refs = [ref_forward(t) for t in seqs]
    tol = 3e-5 if dtype == "float32" else 4e-2
    scale = 1 + max(r.abs().max().item() for r in refs)
    slots = [eng.alloc_slot() for _ in seqs]
    whole = eng.step(slots, seqs, [list(range(len(t))) for t in seqs]).double().cpu()
    assert (whole - torch.cat(refs)).abs().max().item() < tol * scale
    for s in slots:
        eng.free_slot(s)
    slots = [eng.alloc_slot() for _ in seqs]
    heads = [len(t) - 2 for t in seqs]
    eng.step(slots, [t[:h] for t, h in zip(seqs, heads)])
    for kk in range(2):
        out = eng.step(slots, [[t[h + kk]] for t, h in zip(seqs, heads)]).double().cpu()
        for i, (r, h) in enumerate(zip(refs, heads)):
            assert (out[i] - r[h + kk]).abs().max().item() < tol * scale
    for s in slots:
        eng.free_slot(s)
    a = eng.generate(seqs, max_new_tokens=5, temperature=0.0, use_graph=True)
    b = eng.generate(seqs, max_new_tokens=5, temperature=0.0, use_graph=False)
    assert a == b
    if dtype == "float32":
        assert a[1][0] == int(refs[1][-1].argmax())


# ---------------------------------------------------------------------------
# layers of other shapes: norms after the parts, three sub-layers, no feed-forward; a position
# encoding that owns a tensor
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_layers_of_other_shapes_and_a_position_part_with_a_tensor(lib, dtype):
    """A block with a norm before and after each part (four norms a layer), a layer of three sub-layers
    (two attention mixers with caches of their own, then a feed-forward), a layer without feed-forward,
    and a rotation whose frequencies are divided by factors that it owns as a tensor, shared by all
    layers: all registered from here, described by a configuration, built and stepped by the engine
    whole, cut and through generation, against a float64 reference of the same toy model."""
    from llm_infer_amd.config.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry, SubLayerSpec
    from llm_infer_amd.engine import Engine
    from llm_infer_amd.parts.block import Block
    from llm_infer_amd.parts.position import RotaryPosition
    from llm_infer_amd.weights.loader import ParamSpec

    @lib.register_block("toy_sandwich")
    class SandwichBlock(Block):
        """x += post_norm(part(norm(x))) for each sub-layer; a sub-layer without a post norm adds directly."""

        def forward(self, x, ctx, cache_views, owns_cache=True):
            views = iter(cache_views)
            for s in self.sublayers:
                h = s.norm.forward(x)
                out = x if s.post_norm is None else torch.zeros_like(x)
                if s.role == "mixer":
                    s.part.forward(h, ctx, next(views), out, owns_cache)
                else:
                    s.part.forward(h, out)
                if s.post_norm is not None:
                    x += s.post_norm.forward(out).float()

    @lib.register_position("toy_factor_rope")
    class FactorRotary(RotaryPosition):
        """Rotation with each frequency divided by a factor; the factors are a tensor of the model."""

        def params(self):
            return {"weight": ParamSpec((self.rotary_dim // 2,), "vector", "ones")}

        def bind(self, tensors):
            self.factors = tensors["weight"]
            self.inv_freq = self.inv_freq / self.factors

    D, HD, F, V = 64, 16, 72, 60

    class ShapesConfig:
        def __init__(self, raw):
            self.raw = raw

        @classmethod
        def from_dict(cls, raw):
            return cls(raw)

        def model_spec(self):
            norm = PartSpec("rmsnorm", {"size": D, "eps": 1e-5})
            pos = PartSpec("toy_factor_rope", {"theta": 300.0, "rotary_dim": HD, "head_dim": HD}, "rope_freqs.")

            def att(prefix, n_heads, n_kv):
                return PartSpec("attention", {"hidden_size": D, "n_heads": n_heads, "n_kv_heads": n_kv, "head_dim": HD,
                                              "scale": HD ** -0.5}, prefix)
            ffn = PartSpec("gated_mlp", {"hidden_size": D, "intermediate_size": F})
            l0 = LayerSpec("toy_sandwich", (
                SubLayerSpec("mixer", att("l0.a.", 4, 2), norm.with_prefix("l0.n1."), norm.with_prefix("l0.p1.")),
                SubLayerSpec("feed_forward", ffn.with_prefix("l0.f."), norm.with_prefix("l0.n2."), norm.with_prefix("l0.p2."))), pos)
            l1 = LayerSpec("pre_norm", (
                SubLayerSpec("mixer", att("l1.a.", 4, 2), norm.with_prefix("l1.n1.")),
                SubLayerSpec("mixer", att("l1.b.", 2, 1), norm.with_prefix("l1.n2.")),
                SubLayerSpec("feed_forward", ffn.with_prefix("l1.f."), norm.with_prefix("l1.n3."))), pos)
            l2 = LayerSpec("pre_norm", (SubLayerSpec("mixer", att("l2.a.", 2, 1), norm.with_prefix("l2.n1.")),), pos)
            return ModelSpec(D, V, 256, PartSpec("embedding", {"vocab_size": V, "hidden_size": D}, "emb."),
                             (l0, l1, l2), (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(2)),
                             norm.with_prefix("final."),
                             PartSpec("lm_head", {"vocab_size": V, "hidden_size": D, "tied": True}, "head."))

    lib.register_architecture("ShapesToyForCausalLM", ShapesConfig)
    cfg = lib.config_from_dict({"architectures": ["ShapesToyForCausalLM"]})
    eng = Engine.from_random(cfg, seed=6, dtype=dtype, max_tokens=1024)
    model = Engine.from_random(cfg, seed=6, dtype="float32", max_tokens=64).model      # the same values as plain tensors
    # one position part for all three layers, and its tensor is in the model's table once
    assert len(eng.model.positions) == 1 and "rope_freqs.weight" in eng.model.params()
    assert all(m.position is next(iter(eng.model.positions.values())) for ms in eng.model.layer_mixers for m in ms)
    # four units of cache: two groups (2 KV heads: l0.a and l1.a; 1 KV head: l1.b and l2.a)
    assert len(eng.model.cache_specs()) == 4 and len(eng.cache.groups) == 2
    assert sorted(len(g.entries) for g in eng.cache.groups) == [2, 2]
    factors = next(iter(model.positions.values())).factors.double().cpu()
    assert (factors - 1).abs().max() > 1e-3              # they matter: angles differ by a radian at position 100

    def dbl(t):
        return t.double().cpu()

    def rotate(v, posn):
        i = torch.arange(0, HD, 2, dtype=torch.float64)
        ang = posn.double()[:, None] * (1.0 / torch.pow(torch.tensor(300.0, dtype=torch.float64), i / HD) / factors)[None, :]
        cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        out = v.clone()
        out[..., 0::2] = v[..., 0::2] * cos - v[..., 1::2] * sin
        out[..., 1::2] = v[..., 0::2] * sin + v[..., 1::2] * cos
        return out

    def ref_forward(toks):
        n = len(toks)
        x = dbl(model.embedding.weight)[toks]
        posn = torch.arange(n)
        for layer in model.layers:
            for s in layer.sublayers:
                h = P.rmsnorm(x, dbl(s.norm.weight), 1e-5)
                if s.role == "mixer":
                    a = s.part
                    wq, wk, wv = dbl(a.wqkv).split([a.n_heads * HD, a.n_kv_heads * HD, a.n_kv_heads * HD])
                    q = rotate((h @ wq.t()).view(n, a.n_heads, HD), posn)
                    k = rotate((h @ wk.t()).view(n, a.n_kv_heads, HD), posn)
                    y = P.attention(q, k, (h @ wv.t()).view(n, a.n_kv_heads, HD)).reshape(n, -1) @ dbl(a.wo).t()
                else:
                    gu = dbl(s.part.w_gate_up)
                    y = P.swiglu(h, gu[0::2], gu[1::2], dbl(s.part.w_down))
                if s.post_norm is not None:
                    y = P.rmsnorm(y, dbl(s.post_norm.weight), 1e-5)
                x = x + y
        return P.rmsnorm(x, dbl(model.final_norm.weight), 1e-5) @ dbl(model.embedding.weight).t()

    g = torch.Generator().manual_seed(12)
    seqs = [torch.randint(0, V, (n,), generator=g).tolist() for n in (130, 4, 70)]
    refs = [ref_forward(t) for t in seqs]
    tol = 3e-5 if dtype == "float32" else 4e-2
    scale = 1 + max(r.abs().max().item() for r in refs)
    slots = [eng.alloc_slot() for _ in seqs]
    whole = eng.step(slots, seqs, [list(range(len(t))) for t in seqs]).double().cpu()
    assert (whole - torch.cat(refs)).abs().max().item() < tol * scale
    for s in slots:
        eng.free_slot(s)
    slots = [eng.alloc_slot() for _ in seqs]
    heads = [len(t) - 3 for t in seqs]
    eng.step(slots, [t[:h] for t, h in zip(seqs, heads)])
    for kk in range(3):
        out = eng.step(slots, [[t[h + kk]] for t, h in zip(seqs, heads)]).double().cpu()
        for i, (r, h) in enumerate(zip(refs, heads)):
            assert (out[i] - r[h + kk]).abs().max().item() < tol * scale
    for s in slots:
        eng.free_slot(s)
    a = eng.generate(seqs, max_new_tokens=5, temperature=0.0, use_graph=True)
    b = eng.generate(seqs, max_new_tokens=5, temperature=0.0, use_graph=False)
    assert a == b
    assert eng.cache.slots.n_free == eng.cache.n_slots and eng.cache.tokens_free() == (eng.cache.n_pages - 1) * 64
