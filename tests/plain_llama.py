"""Plain, slow Llama decoder: whole sequences, no cache, one function per part.

Written from the formulas of the reference's CPU path and sharing no code with
the engine.  Every function cites the reference lines that fix it.  All
arithmetic is done in the dtype of the inputs (float32 by default, float64 when
the caller widens the weights), weights are used exactly as stored.

Weights are a dict of torch tensors under the checkpoint's tensor names
(``model.embed_tokens.weight`` ...), the configuration is the plain dict read
from ``config.json``.
"""
from __future__ import annotations

import json
import math
import os

import torch


# --------------------------------------------------------------------------
# configuration: defaults as in src/model/config.cpp:74-137
# --------------------------------------------------------------------------
def read_config(folder: str) -> dict:
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def sizes(cfg: dict) -> dict:
    """Sizes with the reference's defaults (src/model/config.cpp:77-93)."""
    d = cfg["hidden_size"]
    n_heads = cfg["num_attention_heads"]
    n_kv = cfg.get("num_key_value_heads", n_heads)          # config.cpp:81
    hd = cfg.get("head_dim", d // n_heads)                  # config.cpp:82
    rotary = int(hd * cfg.get("partial_rotary_factor", 1.0))  # config.cpp:89-90
    return dict(
        n_layers=cfg["num_hidden_layers"], d=d, n_heads=n_heads, n_kv=n_kv, hd=hd,
        ffn=cfg["intermediate_size"], vocab=cfg["vocab_size"],
        theta=float(cfg.get("rope_theta", 10000.0)),        # config.cpp:88
        rotary=rotary,
        eps=float(cfg.get("rms_norm_eps", 1e-5)),           # config.cpp:93
        tied=bool(cfg.get("tie_word_embeddings", False)),
        # absent: silu, the Llama decoder's activation and what the reference's GGUF constructor fixes
        # (config.cpp:163); its HF constructor would default to gelu (config.cpp:97), a departure on purpose
        act=cfg.get("hidden_act", "silu"),
        # which two dimensions of a head form a rotated pair: (2j, 2j+1) as the reference rotates them, or
        # (j, j + rotary/2) for checkpoints whose rows were not permuted for it (docs/gguf.md:487-493)
        pairing=cfg.get("rope_pairing", "adjacent"),
    )


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------
def embed(table: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
    """x = E[token, :], no scaling (src/model/model.cpp:101-118)."""
    return table[tokens.long()]


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """out_i = x_i / sqrt(mean(x^2) + eps) * w_i (include/kernels_cpu.hpp:43-54).

    eps is added to the mean inside the root; the weight multiplies (no 1+w).
    """
    ms = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x / torch.sqrt(ms + eps) * w


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """out_j = sum_i x_i W[j, i], no bias (include/kernels_cpu.hpp:69-80)."""
    return x @ w.t()


def rope(v: torch.Tensor, positions: torch.Tensor, theta: float, rotary_dim: int,
         pairing: str = "adjacent") -> torch.Tensor:
    """Rotate adjacent pairs (i, i+1), i even < rotary_dim, by pos * theta^(-i/rotary_dim).

    v is [n, heads, head_dim]; include/kernels_cpu.hpp:82-100.  Dimensions at or
    beyond rotary_dim stay as they are.  ``pairing`` "half" pairs dimension j with
    j + rotary_dim/2 instead, pair j keeping the angle of the adjacent pair j: the order of a
    checkpoint before the row permutation that the reference's files carry (docs/gguf.md:487-493,
    which maps row j of the first half to 2j and row j of the second half to 2j+1).
    """
    out = v.clone()
    i = torch.arange(0, rotary_dim, 2, dtype=v.dtype)
    freq = 1.0 / torch.pow(torch.tensor(theta, dtype=v.dtype), i / rotary_dim)   # hpp:87
    ang = positions.to(v.dtype)[:, None] * freq[None, :]                          # hpp:88
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    if pairing == "half":
        first, second = slice(0, rotary_dim // 2), slice(rotary_dim // 2, rotary_dim)
    else:
        first, second = slice(0, rotary_dim, 2), slice(1, rotary_dim, 2)
    v0 = v[..., first]
    v1 = v[..., second]
    out[..., first] = v0 * cos - v1 * sin                                         # hpp:96
    out[..., second] = v0 * sin + v1 * cos                                        # hpp:97
    return out


def _r(t: torch.Tensor, act_dtype) -> torch.Tensor:
    """Rounds an activation to the dtype an engine stores it in (None: no rounding).  Only used to
    measure what 16-bit storage of activations itself costs; the formulas are unchanged."""
    return t if act_dtype is None else t.to(act_dtype).to(t.dtype)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int | None = None,
              act_dtype=None) -> torch.Tensor:
    """Causal grouped-query attention over one whole sequence.

    q [n, H, hd], k and v [n, K, hd] -> [n, H, hd].  Query head h reads KV head
    h // (H // K) (src/model/block.cpp:158-164).  score = (q.k) / sqrt(hd), a
    token sees keys 0..pos, softmax subtracts the maximum, the values are mixed
    by the probabilities (include/kernels_cpu.hpp:122-167).  ``window`` (not in
    the reference, which has none) keeps only the last ``window`` keys.
    """
    n, n_heads, hd = q.shape
    n_kv = k.shape[1]
    group = n_heads // n_kv
    out = torch.empty_like(q)
    for h in range(n_heads):
        g = h // group
        for t in range(n):
            lo = 0 if window is None else max(0, t + 1 - window)
            keys = k[lo:t + 1, g, :]
            s = (keys @ q[t, h, :]) / math.sqrt(hd)          # hpp:146-154
            s = torch.exp(s - s.max())                        # hpp:122-133
            p = _r(s, act_dtype) / s.sum()                    # hpp:135-137
            out[t, h, :] = p @ v[lo:t + 1, g, :]             # hpp:159-166
    return out


def silu(x: torch.Tensor) -> torch.Tensor:
    """x / (1 + exp(-x)) (include/kernels_cpu.hpp:186)."""
    return x / (1.0 + torch.exp(-x))


def gelu(x: torch.Tensor) -> torch.Tensor:
    """The tanh form: 0.5 x (1 + tanh(sqrt(2 / pi) (x + 0.044715 x^3))) (include/kernels_cpu.hpp:179-184)."""
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x * x * x)))


def swiglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor,
           act_dtype=None, act: str = "silu") -> torch.Tensor:
    """down(act(gate(x)) * up(x)), act chosen by the configuration (src/model/block.cpp:200-217)."""
    fn = {"silu": silu, "gelu": gelu}[act]                     # block.cpp:203-214
    return linear(_r(fn(linear(x, w_gate)) * linear(x, w_up), act_dtype), w_down)


def attention_part(x, w, prefix, s, positions, window=None, act_dtype=None, kv_dtype=None):
    """Projections, rotation of q and k, attention, output projection (block.cpp:125-167)."""
    n = x.shape[0]
    q = linear(x, w[prefix + "q_proj.weight"]).view(n, s["n_heads"], s["hd"])
    k = linear(x, w[prefix + "k_proj.weight"]).view(n, s["n_kv"], s["hd"])
    v = linear(x, w[prefix + "v_proj.weight"]).view(n, s["n_kv"], s["hd"])
    pairing = s.get("pairing", "adjacent")
    q = _r(rope(q, positions, s["theta"], s["rotary"], pairing), act_dtype)          # block.cpp:141
    k = _r(rope(k, positions, s["theta"], s["rotary"], pairing), act_dtype)          # block.cpp:142
    k, v = _r(k, kv_dtype), _r(v, kv_dtype)               # the cache holds float16 (block.cpp:145-148)
    a = attention(q, k, _r(v, act_dtype), window, act_dtype).reshape(n, s["n_heads"] * s["hd"])
    return linear(_r(a, act_dtype), w[prefix + "o_proj.weight"])            # block.cpp:167


def block(x, w, i, s, positions, act_dtype=None, kv_dtype=None):
    """Pre-norm decoder layer: x += attn(norm(x)); x += ffn(norm(x)) (block.cpp:106-224)."""
    p = f"model.layers.{i}."
    h = _r(rmsnorm(x, w[p + "input_layernorm.weight"], s["eps"]), act_dtype)      # block.cpp:113-119
    x = x + attention_part(h, w, p + "self_attn.", s, positions, None, act_dtype, kv_dtype)  # block.cpp:170-172
    h = _r(rmsnorm(x, w[p + "post_attention_layernorm.weight"], s["eps"]), act_dtype)   # block.cpp:177-183
    x = x + swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                   w[p + "mlp.down_proj.weight"], act_dtype, s.get("act", "silu"))  # block.cpp:220-222
    return x


def forward(weights: dict, cfg: dict, tokens, dtype=torch.float32, act_dtype=None, kv_dtype=None) -> torch.Tensor:
    """Logits [n, vocab] at every position of one whole sequence (model.cpp:60-99).
    ``act_dtype`` rounds the activations that a 16-bit engine stores between its kernels; ``kv_dtype``
    rounds keys (after the rotation) and values as the reference's float16 cache does."""
    s = sizes(cfg)
    w = {k: v.to(dtype) for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.numel())
    x = embed(w["model.embed_tokens.weight"], tokens)
    for i in range(s["n_layers"]):
        x = block(x, w, i, s, positions, act_dtype, kv_dtype)
    x = _r(rmsnorm(x, w["model.norm.weight"], s["eps"]), act_dtype)                # model.cpp:79-90
    head = w["model.embed_tokens.weight"] if s["tied"] or "lm_head.weight" not in w else w["lm_head.weight"]
    return linear(x, head)                                                          # model.cpp:93-98


# --------------------------------------------------------------------------
# sampling (tools/infer.cpp:34-106)
# --------------------------------------------------------------------------
def sample_greedy(logits: torch.Tensor) -> int:
    """First maximum wins (strict >, tools/infer.cpp:64-74)."""
    best, best_i = logits[0].item(), 0
    for i in range(1, logits.numel()):
        if logits[i].item() > best:
            best, best_i = logits[i].item(), i
    return best_i


def probabilities(logits: torch.Tensor, temperature: float) -> torch.Tensor:
    """p_i = exp((l_i - max) / T) / sum (tools/infer.cpp:84-102)."""
    e = torch.exp((logits - logits.max()) / temperature)
    return e / e.sum()


def token_prob(logits: torch.Tensor, token: int) -> float:
    """Probability of one token at temperature 1; 0 outside the vocabulary (tools/infer.cpp:77-81)."""
    return probabilities(logits, 1.0)[token].item() if 0 <= token < logits.numel() else 0.0


def sample_temperature(logits: torch.Tensor, temperature: float, r: float) -> int:
    """argmax if T <= 0, else the first i with r < cumsum_i, fallback V-1 (infer.cpp:40-61)."""
    if temperature <= 0.0:
        return sample_greedy(logits)
    p = probabilities(logits.float(), temperature)
    c = 0.0
    for i in range(p.numel()):
        c += p[i].item()
        if r < c:
            return i
    return p.numel() - 1


def generate_greedy(weights, cfg, prompt, max_new_tokens, stop=(), dtype=torch.float32):
    """sample -> stop check (stop token not kept) -> append -> forward (infer.cpp:289-324)."""
    tokens = list(prompt)
    out = []
    for _ in range(max_new_tokens):
        logits = forward(weights, cfg, tokens, dtype)[-1]
        nxt = sample_greedy(logits)
        if nxt in stop:
            break
        out.append(nxt)
        tokens.append(nxt)
    return out


# --------------------------------------------------------------------------
# random weights for the tests, independent of the engine's generator
# --------------------------------------------------------------------------
def tensor_shapes(cfg: dict) -> dict:
    s = sizes(cfg)
    shapes = {"model.embed_tokens.weight": (s["vocab"], s["d"]), "model.norm.weight": (s["d"],)}
    if not s["tied"]:
        shapes["lm_head.weight"] = (s["vocab"], s["d"])
    for i in range(s["n_layers"]):
        p = f"model.layers.{i}."
        shapes[p + "input_layernorm.weight"] = (s["d"],)
        shapes[p + "post_attention_layernorm.weight"] = (s["d"],)
        shapes[p + "self_attn.q_proj.weight"] = (s["n_heads"] * s["hd"], s["d"])
        shapes[p + "self_attn.k_proj.weight"] = (s["n_kv"] * s["hd"], s["d"])
        shapes[p + "self_attn.v_proj.weight"] = (s["n_kv"] * s["hd"], s["d"])
        shapes[p + "self_attn.o_proj.weight"] = (s["d"], s["n_heads"] * s["hd"])
        shapes[p + "mlp.gate_proj.weight"] = (s["ffn"], s["d"])
        shapes[p + "mlp.up_proj.weight"] = (s["ffn"], s["d"])
        shapes[p + "mlp.down_proj.weight"] = (s["d"], s["ffn"])
    return shapes


def random_weights(cfg: dict, seed: int, std: float = 0.02, matrix_dtype=torch.bfloat16) -> dict:
    """Matrices N(0, std) in ``matrix_dtype``, norm weights 1 + N(0, 0.01) in float32."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if len(shape) == 1:
            out[name] = (1.0 + 0.01 * torch.randn(shape, generator=g)).float()
        else:
            out[name] = (std * torch.randn(shape, generator=g)).to(matrix_dtype)
    return out


def write_model(folder: str, cfg: dict, weights: dict) -> None:
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))


def load_weights(folder: str) -> dict:
    from safetensors.torch import load_file
    return load_file(os.path.join(folder, "model.safetensors"))
