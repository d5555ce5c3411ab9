"""Configurations drawn at random from the sizes the architecture allows (seeded, so every run
draws the same ones): one step of four unequal prompts with every position wanted, then six
tokens each, against the plain implementation in float64. What the fixed tiny configurations
do not reach shows here: a width of the attention output shorter than a product's tile, many
groups on few key heads, a vocabulary and a width that are no multiple of anything."""
import random

import numpy as np
import pytest
import torch

import plain_llama as P

pytestmark = pytest.mark.gpu

DTYPES = {"float32": None, "bfloat16": torch.bfloat16, "float16": torch.float16}
PROMPT_LENGTHS = [1, 5, 17, 40, 64, 65, 97, 130, 200, 300, 513]
DECODED = 6


def draw(seed):
    """A configuration and four prompt lengths. Two families of sizes: the common ones, and
    those that sit beside a kernel's tile (head sizes of 96 to 256, 5 and 7 and 33 query heads
    on a key head)."""
    rng = random.Random(seed)
    if seed % 2 == 0:
        hd, kvh, g = rng.choice([16, 32, 48, 64, 80, 128]), rng.choice([1, 2, 3, 4]), rng.choice([1, 2, 3, 4, 8])
    else:
        hd, kvh, g = rng.choice([16, 96, 112, 144, 160, 256]), rng.choice([1, 2, 5]), rng.choice([1, 5, 7, 33])
    cfg = {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "num_hidden_layers": rng.choice([1, 2, 3]),
           "hidden_size": rng.choice([64, 72, 96, 100, 128, 200, 256, 320, 512]),
           "num_attention_heads": kvh * g, "num_key_value_heads": kvh, "head_dim": hd,
           "intermediate_size": rng.choice([96, 136, 172, 256, 344, 1000]),
           "vocab_size": rng.choice([100, 331, 512, 1000, 5003]),
           "rope_theta": rng.choice([100.0, 10000.0, 500000.0]), "rms_norm_eps": rng.choice([1e-6, 1e-5, 1e-4]),
           "partial_rotary_factor": rng.choice([1.0, 1.0, 0.5, 0.25]),
           "max_position_embeddings": 1024, "tie_word_embeddings": rng.choice([True, False]),
           "hidden_act": rng.choice(["silu", "silu", "gelu"])}
    return cfg, [rng.choice(PROMPT_LENGTHS) for _ in range(4)]


def one_head_of_16():
    """The attention output is 16 wide: shorter than the depth of any tile of the product that follows it,
    with more rows than the small products' kernels take."""
    cfg, _ = draw(0)
    cfg.update(num_attention_heads=1, num_key_value_heads=1, head_dim=16, hidden_size=96, num_hidden_layers=2)
    return cfg, [300, 513, 97, 17]


CASES = {f"seed{seed}": draw(seed) for seed in range(14)}
CASES["one_head_of_16"] = one_head_of_16()


@pytest.mark.parametrize("name", list(CASES))
def test_a_drawn_configuration_against_the_plain_implementation(name, tmp_path):
    import llm_infer_amd
    cfg, lens = CASES[name]
    seed = sorted(CASES).index(name)
    gen = torch.Generator().manual_seed(seed)
    requests = [torch.randint(0, cfg["vocab_size"], (n + DECODED,), generator=gen).tolist() for n in lens]
    for dtype, stored in DTYPES.items():
        weights = P.random_weights(cfg, seed, std=0.05, matrix_dtype=stored or torch.bfloat16)
        for key in weights:                              # sharper attention: a wrong key or position shows
            if "q_proj" in key or "k_proj" in key:
                weights[key] = (weights[key].float() * 2).to(weights[key].dtype)
        folder = tmp_path / dtype
        folder.mkdir()
        P.write_model(str(folder), cfg, weights)
        refs = [P.forward(weights, cfg, t, torch.float64).numpy() for t in requests]
        if stored is None:
            own = max(np.abs(P.forward(weights, cfg, t, torch.float32).numpy() - r).max() for t, r in zip(requests, refs))
        else:
            own = max(np.abs(P.forward(weights, cfg, t, torch.float64, stored).numpy() - r).max()
                      for t, r in zip(requests, refs))
        tol = 3 * own + 1e-6 * np.mean([r.std() for r in refs])

        engine = llm_infer_amd.load(str(folder), dtype=dtype, max_tokens=4096)
        slots = [engine.alloc_slot() for _ in requests]
        got = engine.step(slots, [t[:n] for t, n in zip(requests, lens)], [list(range(n)) for n in lens]).double().cpu().numpy()
        at = 0
        for i, (ref, n) in enumerate(zip(refs, lens)):
            err = np.abs(got[at:at + n] - ref[:n]).max(axis=1)
            assert err.max() < tol, (dtype, "prompt", i, "position", int(err.argmax()), err.max(), tol, cfg, lens)
            at += n
        for k in range(DECODED):
            got = engine.step(slots, [[t[n + k]] for t, n in zip(requests, lens)]).double().cpu().numpy()
            for i, (ref, n) in enumerate(zip(refs, lens)):
                err = np.abs(got[i] - ref[n + k]).max()
                assert err < tol, (dtype, "request", i, "decoded", k, err, tol, cfg, lens)
        for slot in slots:
            engine.free_slot(slot)
