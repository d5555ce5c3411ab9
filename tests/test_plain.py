"""Pins the plain implementation by what fixes it beside the reference's text.

The reference holds no test vectors, so each formula is pinned by special cases
that reduce to a library routine and by invariants, chosen so that a plausible
mistake (wrong sign or pairing, eps outside the root, swapped gate and up, a norm
in the wrong place) fails.
"""
import math

import pytest
import torch

import plain_llama as P
from tiny_configs import ALL, TINY_A, TINY_B, TINY_C

torch.manual_seed(0)
F64 = torch.float64


def test_rmsnorm_library_formula_and_eps_place():
    x = torch.randn(5, 96, dtype=F64)
    w = torch.randn(96, dtype=F64)
    ref = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w
    assert torch.allclose(P.rmsnorm(x, w, 1e-5), ref, rtol=1e-12, atol=0)
    # eps is added to the mean inside the root: at mean-square 1e-6, eps 1e-5 dominates
    x = torch.full((1, 64), 1e-3, dtype=F64)
    out = P.rmsnorm(x, torch.ones(64, dtype=F64), 1e-5)
    assert torch.allclose(out, torch.full_like(out, 1e-3 / math.sqrt(1e-6 + 1e-5)), rtol=1e-12)
    # the weight multiplies, it is not (1 + w)
    assert P.rmsnorm(torch.randn(3, 8, dtype=F64), torch.zeros(8, dtype=F64), 1e-5).abs().max() == 0
    # mean-square of the output with w=1
    x = torch.randn(4, 128, dtype=F64)
    ms = (x * x).mean(-1)
    out = P.rmsnorm(x, torch.ones(128, dtype=F64), 1e-5)
    assert torch.allclose((out * out).mean(-1), ms / (ms + 1e-5), rtol=1e-12)


def test_linear_is_x_wt():
    x, w = torch.randn(3, 7, dtype=F64), torch.randn(5, 7, dtype=F64)
    assert torch.allclose(P.linear(x, w), torch.nn.functional.linear(x, w))
    assert P.linear(x, w).shape == (3, 5)


def test_rope_identity_norm_pairing_theta_sign():
    v = torch.randn(6, 3, 32, dtype=F64)
    pos = torch.tensor([0, 1, 2, 50, 51, 1000])
    out = P.rope(v, pos, 10000.0, 32)
    assert torch.equal(out[0], v[0])                      # position 0 is the identity
    a = v.view(6, 3, 16, 2).norm(dim=-1)
    b = out.view(6, 3, 16, 2).norm(dim=-1)
    assert torch.allclose(a, b, rtol=1e-12)               # every adjacent pair keeps its norm
    # a one-hot at 2j moves mass only to 2j+1, with (cos a, +sin a)
    j = 3
    e = torch.zeros(1, 1, 32, dtype=F64)
    e[0, 0, 2 * j] = 1.0
    r = P.rope(e, torch.tensor([7]), 500000.0, 32)
    ang = 7.0 * 500000.0 ** (-(2 * j) / 32)
    want = torch.zeros(32, dtype=F64)
    want[2 * j], want[2 * j + 1] = math.cos(ang), math.sin(ang)
    assert torch.allclose(r[0, 0], want, atol=1e-12)
    # the exponent's denominator is rotary_dim, not head_dim
    e = torch.zeros(1, 1, 32, dtype=F64)
    e[0, 0, 2] = 1.0
    r = P.rope(e, torch.tensor([1]), 10000.0, 16)
    assert abs(r[0, 0, 2].item() - math.cos(10000.0 ** (-2 / 16))) < 1e-12
    # dimensions beyond rotary_dim are left alone
    out = P.rope(v, pos, 10000.0, 16)
    assert torch.equal(out[..., 16:], v[..., 16:])
    assert not torch.equal(out[1:, :, :16], v[1:, :, :16])


def test_rope_scores_depend_on_distance_only():
    q = torch.randn(1, 2, 16, dtype=F64)
    k = torch.randn(1, 2, 16, dtype=F64)
    def score(m, n):
        return (P.rope(q, torch.tensor([m]), 1e4, 16) * P.rope(k, torch.tensor([n]), 1e4, 16)).sum(-1)
    assert torch.allclose(score(5, 2), score(105, 102), atol=1e-10)
    assert not torch.allclose(score(5, 2), score(5, 3), atol=1e-6)


def test_rope_half_pairing_is_a_complex_product_and_a_permutation_of_the_adjacent_one():
    """Half pairing: dimension j and j + rotary/2 are the real and imaginary part of a number that is
    multiplied by exp(i pos theta^(-2j/rotary)) (a library routine), and the same rotation as the adjacent
    one on a head whose dimensions were dealt out (first half to the even places, second half to the odd
    ones: the permutation of docs/gguf.md:487-493).  A wrong sign, a pair (j, j+1) or frequencies counted
    over the half fail one of the two."""
    rot, hd = 24, 32
    v = torch.randn(5, 2, hd, dtype=F64)
    pos = torch.tensor([0, 1, 7, 300, 4097])
    out = P.rope(v, pos, 20000.0, rot, "half")
    z = torch.complex(v[..., :rot // 2], v[..., rot // 2:rot])
    ang = pos.to(F64)[:, None] * 20000.0 ** (-torch.arange(0, rot, 2, dtype=F64) / rot)[None, :]
    w = z * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    assert torch.allclose(out[..., :rot // 2], w.real, atol=1e-12)
    assert torch.allclose(out[..., rot // 2:rot], w.imag, atol=1e-12)
    assert torch.equal(out[..., rot:], v[..., rot:]) and torch.equal(out[0], v[0])
    # dealt out: new dimension 2j <- j, 2j+1 <- j + rot/2; the adjacent rotation of that is the half one, dealt out
    order = list(range(hd))
    for j in range(rot // 2):
        order[2 * j], order[2 * j + 1] = j, j + rot // 2
    assert torch.allclose(P.rope(v[..., order], pos, 20000.0, rot), out[..., order], atol=1e-12)
    assert not torch.allclose(P.rope(v, pos, 20000.0, rot), out, atol=1e-3)
    # scores depend on the distance alone here too
    q, k = v[:1], v[1:2]
    s = lambda m, n: (P.rope(q, torch.tensor([m]), 1e4, rot, "half") * P.rope(k, torch.tensor([n]), 1e4, rot, "half")).sum(-1)
    assert torch.allclose(s(9, 4), s(209, 204), atol=1e-10)


def _library_attention(q, k, v):
    n, H, hd = q.shape
    g = H // k.shape[1]
    kk = k.repeat_interleave(g, dim=1).transpose(0, 1)
    vv = v.repeat_interleave(g, dim=1).transpose(0, 1)
    o = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), kk, vv, is_causal=True)
    return o.transpose(0, 1)


@pytest.mark.parametrize("H,K,hd", [(4, 2, 16), (3, 1, 32), (5, 5, 48), (8, 2, 64)])
def test_attention_equals_library(H, K, hd):
    n = 11
    q, k, v = torch.randn(n, H, hd, dtype=F64), torch.randn(n, K, hd, dtype=F64), torch.randn(n, K, hd, dtype=F64)
    assert torch.allclose(P.attention(q, k, v), _library_attention(q, k, v), atol=1e-12)


def test_attention_special_cases():
    n, H, K, hd = 6, 4, 2, 16
    q, v = torch.randn(n, H, hd, dtype=F64), torch.randn(n, K, hd, dtype=F64)
    k = torch.randn(n, K, hd, dtype=F64)
    out = P.attention(q, k, v)
    # the first token sees only itself
    assert torch.allclose(out[0], v[0].repeat_interleave(2, dim=0))
    # equal keys: the output is the running mean of the values
    ku = torch.ones(n, K, hd, dtype=F64)
    out = P.attention(q, ku, v)
    means = torch.cumsum(v, 0) / torch.arange(1, n + 1, dtype=F64)[:, None, None]
    assert torch.allclose(out, means.repeat_interleave(2, dim=1), atol=1e-12)
    # consecutive query heads share a KV head: h // (H // K)
    q2 = q.clone()
    q2[:, 1] = q2[:, 0]
    out = P.attention(q2, k, v)
    assert torch.allclose(out[:, 0], out[:, 1])
    assert not torch.allclose(out[:, 1], P.attention(q2[:, [0, 2, 1, 3]], k, v)[:, 1])
    # the scale is 1/sqrt(hd): with one outstanding key the weights are known in closed form
    hd = 32
    q = torch.zeros(2, 1, hd, dtype=F64)
    q[1, 0, 0] = 3.0
    k = torch.zeros(2, 1, hd, dtype=F64)
    k[1, 0, 0] = 2.0
    v = torch.tensor([[[0.0] * hd], [[1.0] * hd]], dtype=F64)
    p1 = math.exp(6.0 / math.sqrt(hd)) / (1.0 + math.exp(6.0 / math.sqrt(hd)))
    assert abs(P.attention(q, k, v)[1, 0, 0].item() - p1) < 1e-12
    # window: only the last w keys
    n = 9
    q, k, v = (torch.randn(n, 2, 16, dtype=F64) for _ in range(3))
    w = P.attention(q, k, v, window=3)
    assert torch.allclose(w[:3], P.attention(q, k, v)[:3])
    assert torch.allclose(w[8], P.attention(q[6:9], k[6:9], v[6:9])[2])


def test_silu_and_swiglu():
    x = torch.tensor([0.0, 30.0, -2.0, 2.0], dtype=F64)
    s = P.silu(x)
    assert s[0] == 0 and abs(s[1] - 30.0) < 1e-9
    assert torch.allclose(s[2], -2.0 * torch.sigmoid(torch.tensor(-2.0, dtype=F64)))
    assert torch.allclose(s, torch.nn.functional.silu(x))
    d, f = 8, 12
    xx = torch.randn(3, d, dtype=F64)
    wg, wu, wd = torch.randn(f, d, dtype=F64), torch.randn(f, d, dtype=F64), torch.randn(d, f, dtype=F64)
    assert P.swiglu(xx, torch.zeros_like(wg), wu, wd).abs().max() == 0
    assert P.swiglu(xx, wg, torch.zeros_like(wu), wd).abs().max() == 0
    ref = torch.nn.functional.linear(torch.nn.functional.silu(xx @ wg.t()) * (xx @ wu.t()), wd)
    assert torch.allclose(P.swiglu(xx, wg, wu, wd), ref)
    assert not torch.allclose(P.swiglu(xx, wu, wg, wd), ref)       # gate and up are not interchangeable
    # the other activation of the gate: the library's tanh form, no other (the exact form differs by 1e-3),
    # zero at zero, the identity far out, and chosen by name
    g = P.gelu(x)
    assert torch.allclose(g, torch.nn.functional.gelu(x, approximate="tanh"))
    assert not torch.allclose(P.gelu(xx), torch.nn.functional.gelu(xx), atol=1e-5)
    assert g[0] == 0 and abs(g[1] - 30.0) < 1e-9 and g[2] < 0
    ref = torch.nn.functional.linear(torch.nn.functional.gelu(xx @ wg.t(), approximate="tanh") * (xx @ wu.t()), wd)
    assert torch.allclose(P.swiglu(xx, wg, wu, wd, act="gelu"), ref)
    assert not torch.allclose(P.swiglu(xx, wg, wu, wd, act="silu"), ref)


@pytest.mark.parametrize("name", list(ALL))
def test_block_is_identity_without_output_matrices(name):
    cfg = ALL[name]
    s = P.sizes(cfg)
    w = {k: v.double() for k, v in P.random_weights(cfg, 3).items()}
    w["model.layers.0.self_attn.o_proj.weight"].zero_()
    w["model.layers.0.mlp.down_proj.weight"].zero_()
    x = torch.randn(5, s["d"], dtype=F64)
    assert torch.equal(P.block(x, w, 0, s, torch.arange(5)), x)


def _block_weights(cfg, seed):
    return {k: v.double() for k, v in P.random_weights(cfg, seed, std=0.3).items()}


@pytest.mark.parametrize("name", list(ALL))
def test_block_arrangement_norm_before_each_part_and_sequential_residuals(name):
    """block.cpp:113-119, 170-183, 220-222: a norm feeds the mixer, its result is added, a second norm
    reads the sum, the feed-forward's result is added.  Each line fails for one plausible mistake: a
    missing norm, a norm after the part, a feed-forward that reads x instead of x + attention."""
    cfg = ALL[name]
    s = P.sizes(cfg)
    w = _block_weights(cfg, 4)
    p = "model.layers.0."
    pos = torch.arange(6)
    x = torch.randn(6, s["d"], dtype=F64)
    n1 = P.rmsnorm(x, w[p + "input_layernorm.weight"], s["eps"])
    a = P.attention_part(n1, w, p + "self_attn.", s, pos)
    # without the feed-forward's output matrix exactly x + attention(norm1(x)) is left
    w0 = dict(w)
    w0[p + "mlp.down_proj.weight"] = torch.zeros_like(w[p + "mlp.down_proj.weight"])
    assert torch.allclose(P.block(x, w0, 0, s, pos), x + a, atol=1e-12)
    assert not torch.allclose(P.block(x, w0, 0, s, pos), x + P.attention_part(x, w, p + "self_attn.", s, pos), atol=1e-3)
    # the feed-forward reads norm2(x + attention), not norm2(x) (a parallel residual) and not x + attention
    y = P.block(x, w, 0, s, pos)
    gate, up, down = (w[p + f"mlp.{m}_proj.weight"] for m in ("gate", "up", "down"))
    n2 = P.rmsnorm(x + a, w[p + "post_attention_layernorm.weight"], s["eps"])
    assert torch.allclose(y - x - a, P.swiglu(n2, gate, up, down, act=s["act"]), atol=1e-10)
    parallel = P.swiglu(P.rmsnorm(x, w[p + "post_attention_layernorm.weight"], s["eps"]), gate, up, down, act=s["act"])
    assert not torch.allclose(y - x - a, parallel, atol=1e-3)
    assert not torch.allclose(y - x - a, P.swiglu(x + a, gate, up, down, act=s["act"]), atol=1e-3)
    # what a layer adds does not depend on the scale of a large input: both parts see it only through a
    # norm (and norm2(c x + a) = norm2(x + a / c) -> norm2(x) as x grows).  Without either norm it does.
    big = 1e6 * x
    u1 = P.block(big, w, 0, s, pos) - big
    u3 = P.block(3 * big, w, 0, s, pos) - 3 * big
    assert (u1 - u3).abs().max() < 1e-3 * u1.abs().max()
    # and the norms' weights are the layer's own two vectors, each in its place
    w2 = dict(w)
    w2[p + "input_layernorm.weight"] = 2 * w[p + "input_layernorm.weight"]
    a2 = P.attention_part(2 * n1, w, p + "self_attn.", s, pos)
    assert torch.allclose(P.block(x, {**w2, p + "mlp.down_proj.weight": w0[p + "mlp.down_proj.weight"]}, 0, s, pos),
                          x + a2, atol=1e-12)


@pytest.mark.parametrize("name", list(ALL))
def test_final_norm_and_unscaled_embedding(name):
    """model.cpp:79-98, 101-118: the last layer's output goes through the final norm before the head, and a
    token's row of the table enters unscaled."""
    cfg = dict(ALL[name], num_hidden_layers=1)
    s = P.sizes(cfg)
    w = _block_weights(cfg, 6)
    toks = [3, 1, 4, 1, 5]
    full = P.forward(w, cfg, toks, F64)
    # the logits scale with the final norm's weight and vanish with it
    w2 = dict(w)
    w2["model.norm.weight"] = 2 * w["model.norm.weight"]
    assert torch.allclose(P.forward(w2, cfg, toks, F64), 2 * full, atol=1e-9)
    w2["model.norm.weight"] = torch.zeros_like(w["model.norm.weight"])
    assert P.forward(w2, cfg, toks, F64).abs().max() == 0
    # a weight that picks one channel: the logits see that channel of the normalised state alone
    e0 = torch.zeros_like(w["model.norm.weight"])
    e0[2] = 1.0
    w2["model.norm.weight"] = e0
    head = w["model.embed_tokens.weight"] if s["tied"] else w["lm_head.weight"]
    one = P.forward(w2, cfg, toks, F64)
    assert torch.allclose(one / head[:, 2][None, :], (one / head[:, 2][None, :])[:, :1].expand_as(one), atol=1e-9)
    # with a layer that adds nothing the logits are norm(E[token]) W^T, the norm taken from the library:
    # no factor on the embedding (sqrt(d) or any other would change what eps does to a small row)
    wz = dict(w)
    wz["model.layers.0.self_attn.o_proj.weight"] = torch.zeros_like(w["model.layers.0.self_attn.o_proj.weight"])
    wz["model.layers.0.mlp.down_proj.weight"] = torch.zeros_like(w["model.layers.0.mlp.down_proj.weight"])
    wz["model.embed_tokens.weight"] = w["model.embed_tokens.weight"] * 1e-2      # rows near sqrt(eps): a scale would show
    rows = wz["model.embed_tokens.weight"][torch.tensor(toks)]
    normed = torch.nn.functional.rms_norm(rows, (s["d"],), w["model.norm.weight"], s["eps"])
    headz = wz["model.embed_tokens.weight"] if s["tied"] else wz["lm_head.weight"]
    got = P.forward(wz, cfg, toks, F64)
    assert torch.allclose(got, normed @ headz.t(), atol=1e-12)
    scaled = torch.nn.functional.rms_norm(rows * s["d"] ** 0.5, (s["d"],), w["model.norm.weight"], s["eps"])
    assert not torch.allclose(got, scaled @ headz.t(), rtol=1e-3, atol=0)


def test_attention_part_shift_invariance():
    s = P.sizes(TINY_A)
    w = {k: v.double() for k, v in P.random_weights(TINY_A, 1, std=0.3).items()}
    x = torch.randn(7, s["d"], dtype=F64)
    a = P.attention_part(x, w, "model.layers.0.self_attn.", s, torch.arange(7))
    b = P.attention_part(x, w, "model.layers.0.self_attn.", s, torch.arange(7) + 40)
    assert torch.allclose(a, b, atol=1e-10)


def test_cache_rounding_touches_keys_after_rotation_and_values_only():
    """block.cpp:141-148: q and k are rotated, then k and v go into the cache as float16; q does not."""
    s = P.sizes(TINY_A)
    w = {k: v.double() for k, v in P.random_weights(TINY_A, 3, std=0.3).items()}
    x = torch.randn(6, s["d"], dtype=F64)
    pre = "model.layers.0.self_attn."
    pos = torch.arange(6) + 3
    got = P.attention_part(x, w, pre, s, pos, kv_dtype=torch.float16)
    q = P.rope(P.linear(x, w[pre + "q_proj.weight"]).view(6, s["n_heads"], s["hd"]), pos, s["theta"], s["rotary"])
    k = P.rope(P.linear(x, w[pre + "k_proj.weight"]).view(6, s["n_kv"], s["hd"]), pos, s["theta"], s["rotary"])
    v = P.linear(x, w[pre + "v_proj.weight"]).view(6, s["n_kv"], s["hd"])
    a = P.attention(q, k.half().double(), v.half().double()).reshape(6, -1)
    assert torch.equal(got, P.linear(a, w[pre + "o_proj.weight"]))
    assert not torch.equal(got, P.attention_part(x, w, pre, s, pos))
    # a single token: the output is its own value row, rounded
    one = P.attention_part(x[:1], w, pre, s, pos[:1], kv_dtype=torch.float16)
    v0 = v[:1].half().double().repeat_interleave(s["n_heads"] // s["n_kv"], dim=1).reshape(1, -1)
    assert torch.allclose(one, P.linear(v0, w[pre + "o_proj.weight"]), atol=1e-12)


def test_sizes_defaults():
    s = P.sizes({"hidden_size": 64, "num_attention_heads": 4, "num_hidden_layers": 1,
                 "intermediate_size": 8, "vocab_size": 10})
    assert s["n_kv"] == 4 and s["hd"] == 16 and s["theta"] == 10000.0 and s["eps"] == 1e-5
    assert s["rotary"] == 16 and not s["tied"]
    assert P.sizes(TINY_C)["rotary"] == 24 and P.sizes(TINY_C)["hd"] == 48


def test_head_tied_and_untied_and_prefix_property():
    for cfg in (TINY_A, TINY_B):
        w = P.random_weights(cfg, 5, std=0.2)
        toks = list(range(3, 14))
        full = P.forward(w, cfg, toks, F64)
        # causal: the logits of a prefix equal the prefix of the logits
        part = P.forward(w, cfg, toks[:6], F64)
        assert torch.allclose(full[:6], part, atol=1e-10)
        assert full.shape == (11, cfg["vocab_size"])
    assert "lm_head.weight" not in P.random_weights(TINY_B, 0)
    w = P.random_weights(TINY_A, 5, std=0.2)
    a = P.forward(w, TINY_A, [1, 2, 3], F64)
    w["lm_head.weight"] = w["lm_head.weight"] * 2
    assert torch.allclose(P.forward(w, TINY_A, [1, 2, 3], F64), 2 * a, atol=1e-10)


def test_sampling_rules():
    l = torch.tensor([1.0, 5.0, 5.0, 2.0])
    assert P.sample_greedy(l) == 1                                  # the first maximum wins
    assert P.sample_temperature(l, 0.0, 0.3) == 1
    assert P.sample_temperature(l, -1.0, 0.3) == 1
    p = P.probabilities(l, 0.8)
    assert torch.allclose(p, torch.softmax(l / 0.8, 0))
    assert P.sample_temperature(l, 0.8, 0.0) == 0
    assert P.sample_temperature(l, 0.8, float(p[0]) + 1e-4) == 1
    assert P.sample_temperature(l, 0.8, 0.99999999) == 3
    assert P.sample_temperature(l, 1e-4, 0.9) in (1, 2)
    assert abs(P.token_prob(l, 3) - torch.softmax(l, 0)[3].item()) < 1e-7       # temperature 1, whatever the sampler's
    assert P.token_prob(l, 4) == 0.0 and P.token_prob(l, -1) == 0.0


def test_generate_stops_before_keeping_the_stop_token():
    w = P.random_weights(TINY_A, 2, std=0.2)
    out = P.generate_greedy(w, TINY_A, [4, 5, 6], 6)
    assert len(out) == 6
    cut = P.generate_greedy(w, TINY_A, [4, 5, 6], 6, stop=(out[2],))
    first = out.index(out[2])
    assert cut == out[:first]
