"""The engine against the plain implementation at the layer sizes the benchmark runs and at a long
context, in 32-bit and in float16, under the three ways of cutting requests into steps.

The tiny configurations never reach the code that serves real sizes: head size 128 with four query
heads a KV head, a down projection with K = 14,336, products of 17 to 300 rows that split K, the
prefill product's tiles (256, 192 and 128 rows of W, a last tile of rows that is partly empty, the
kernels whose epilogue is the residual sum or the rotation alone), page tables beyond 128 pages, 64 splits of the decode attention, rotation angles at
positions in the thousands.  Here they lie on a tested path: two layers of the Llama-3.1-8B layer
shape, one layer of the Llama-2-7B shape (32 KV heads), and a small model with a request of 9,000
tokens."""
import os

import numpy as np
import pytest
import torch

import plain_llama as P
import trace_util as TU

pytestmark = pytest.mark.gpu

CONFIGS = {
    # the Llama-3.1-8B layer: 4 query heads a KV head, head size 128, K = 14,336 in the down projection
    "8b": {"architectures": ["LlamaForCausalLM"], "num_hidden_layers": 2, "hidden_size": 4096,
           "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 14336,
           "vocab_size": 2048, "rope_theta": 500000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 512,
           "tie_word_embeddings": False, "hidden_act": "silu", "torch_dtype": "float16"},
    # the Llama-2-7B layer: as many KV heads as heads, another intermediate size and theta
    "7b": {"architectures": ["LlamaForCausalLM"], "num_hidden_layers": 1, "hidden_size": 4096,
           "num_attention_heads": 32, "num_key_value_heads": 32, "intermediate_size": 11008,
           "vocab_size": 1000, "rope_theta": 10000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 2048,
           "tie_word_embeddings": False, "hidden_act": "silu", "torch_dtype": "float16"},
    # small layers, long context
    "long": {"architectures": ["LlamaForCausalLM"], "num_hidden_layers": 2, "hidden_size": 128,
             "num_attention_heads": 4, "num_key_value_heads": 1, "head_dim": 32, "intermediate_size": 200,
             "vocab_size": 300, "rope_theta": 500000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 16384,
             "tie_word_embeddings": True, "hidden_act": "silu", "torch_dtype": "float16"},
}
# 1,300 rows: eleven tiles of rows, the last a fifth full; the 7B layer's q/k/v product takes the 192-row tile
LENGTHS = {"8b": [1, 17, 64, 65, 300], "7b": [1, 17, 64, 65, 300, 1300], "long": [9000]}


def make_weights(name, cfg):
    if name != "long":
        return P.random_weights(cfg, seed=len(name) + 40, std=0.02, matrix_dtype=torch.float16)
    # few dimensions: sharper queries and keys, so that a far key among thousands carries weight
    w = P.random_weights(cfg, seed=3, std=0.05, matrix_dtype=torch.float16)
    for n in w:
        if "q_proj" in n or "k_proj" in n:
            w[n] = (w[n].float() * 2).to(w[n].dtype)
    return w


class Case:
    def __init__(self, name, tmp_path_factory):
        self.name, self.cfg = name, CONFIGS[name]
        self.folder = str(tmp_path_factory.mktemp(f"real_{name}"))
        weights = make_weights(name, self.cfg)
        P.write_model(self.folder, self.cfg, weights)
        g = torch.Generator().manual_seed(17)
        self.requests = {f"r{i}": torch.randint(0, self.cfg["vocab_size"], (n,), generator=g).tolist()
                         for i, n in enumerate(LENGTHS[name])}
        self.refs, self.own = {}, {"float32": 0.0, "float16": 0.0}
        for rid, toks in self.requests.items():
            ref = P.forward(weights, self.cfg, toks, torch.float64)
            self.refs[rid] = ref.numpy()
            # the plain implementation's own error: in float32 arithmetic, and with its activations
            # rounded to float16 where a 16-bit engine stores them
            self.own["float32"] = max(self.own["float32"], (P.forward(weights, self.cfg, toks, torch.float32).double()
                                                            - ref).abs().max().item())
            self.own["float16"] = max(self.own["float16"], (P.forward(weights, self.cfg, toks, torch.float64,
                                                                      torch.float16) - ref).abs().max().item())


@pytest.fixture(scope="module", params=list(CONFIGS))
def case(request, tmp_path_factory):
    return Case(request.param, tmp_path_factory)


@pytest.mark.parametrize("dtype", ["float32", "float16"])
def test_three_schedules_at_real_sizes(case, dtype, tmp_path):
    cfg, requests = case.cfg, case.requests
    vocab = cfg["vocab_size"]
    s1, w1 = TU.steps_whole(requests)
    s2, w2 = TU.steps_tail(requests, 32, first_step=100_000)
    # batches of three that start together: the first step of the first batch has 1 + 17 + 32 rows, the
    # second batch's 64 + 260 (+ 1,290); shorter requests end earlier
    decoded = {rid: [3, 0, 32, 1, 40, 10][i % 6] for i, rid in enumerate(requests)}
    s3, w3 = TU.steps_batches(requests, 3, decoded, first_step=200_000)
    page = lambda n: -(-n // 64) * 64
    max_tokens = sum(sorted((page(len(t)) for t in requests.values()), reverse=True)[:3])
    TU.run_trace(case.folder, dtype, s1 + s2 + s3, {**w1, **w2, **w3}, vocab, max_tokens, str(tmp_path), timeout=900)
    scale = np.mean([r.std() for r in case.refs.values()])
    tol = 3 * case.own[dtype] + 1e-6 * scale
    for where, what in ((w1, "whole"), (w2, "tail"), (w3, "batches")):
        seen, worst, worst_key = set(), 0.0, None
        for s, keys in where.items():
            data = np.fromfile(os.path.join(str(tmp_path), f"{s}.f32"), dtype="<f4").reshape(len(keys), vocab)
            for (rid, p), row in zip(keys, data):
                seen.add((rid, p))
                e = np.abs(row.astype(np.float64) - case.refs[rid][p]).max()
                if e > worst:
                    worst, worst_key = e, (rid, p)
        assert seen == {(r, p) for r, t in requests.items() for p in range(len(t))}, what
        assert worst < tol, f"{case.name} {what} {dtype}: first look at {worst_key}: error {worst:.3e}, allowed {tol:.3e}"


def test_recorded_decode_steps_at_real_sizes(tmp_path):
    """Greedy generation through recorded steps at the 8B layer's sizes: twenty sequences that end at different
    times, so the recorded steps run 24, 16, 12, 8, 4, 2 and 1 rows (idle rows on the scratch slot) through the
    kernels for 17 to 128 rows and for up to 16, the prompts through recorded prefill steps the second time.
    The tokens are those of the eager steps, and where the plain implementation's two best logits lie further
    apart than the engine may err, they are the plain implementation's choice."""
    import llm_infer_amd as lib
    cfg = CONFIGS["8b"]
    weights = make_weights("8b", cfg)
    folder = str(tmp_path / "m")
    P.write_model(folder, cfg, weights)
    eng = lib.load(folder, dtype="float16", max_tokens=20 * 192, n_slots=24)     # 20 live rows run as 24
    g = torch.Generator().manual_seed(5)
    lengths = [3, 70, 17, 64, 33, 5, 48, 65, 9, 100, 2, 31, 80, 12, 57, 24, 6, 90, 40, 1]
    budgets = [40, 6, 22, 9, 35, 14, 4, 28, 11, 19, 38, 7, 25, 16, 3, 31, 13, 21, 5, 36]
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in lengths]
    eager = eng.generate(prompts, max_new_tokens=budgets, temperature=0.0, use_graph=False, stop_token_ids=())
    assert [len(o) for o in eager] == budgets
    first = eng.generate(prompts, max_new_tokens=budgets, temperature=0.0, use_graph=True, stop_token_ids=())
    again = eng.generate(prompts, max_new_tokens=budgets, temperature=0.0, use_graph=True, stop_token_ids=())
    assert first == eager and again == eager
    assert sorted({k[0] for k in eng._graphs}) == [1, 2, 4, 8, 12, 16, 24]
    assert eng.decode_counts["replayed"] > eng.decode_counts["recorded"] > 0
    checked = 0
    for i in (0, 4, 10):                                   # the three that decode longest, from short prompts
        whole = prompts[i] + eager[i]
        ref = P.forward(weights, cfg, whole, torch.float64)
        own = (P.forward(weights, cfg, whole, torch.float64, torch.float16) - ref).abs().max().item()
        tol = 3 * own + 1e-6 * ref.std().item()
        for j, tok in enumerate(eager[i]):
            top = torch.topk(ref[len(prompts[i]) + j - 1], 2)
            if (top.values[0] - top.values[1]).item() > 2 * tol:
                assert tok == top.indices[0].item(), (i, j)
                checked += 1
    assert checked >= 60, checked
    assert eng.cache.slots.n_free == eng.cache.n_slots
