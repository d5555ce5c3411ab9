#!/usr/bin/env python3
"""Decode and prefill throughput of the Llama-3.1-8B shape with random weights on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one decode step of the generation loop's own runner (bookkeeping, the
model's forward pass from the cache, sampling, tokens back to the host) for a
batch of 8 sequences whose contexts end at the benchmark's context length.  The
runner replays recorded steps; the window of positions is walked once untimed
first, so that no step is recorded inside the timed ones (`warmup` counts all
untimed steps).  The
line printed also holds the prefill of one 2,048-token prompt, the decode step's
share of the HBM roofline, and decode throughput at batch 1 and 64.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published peaks
HBM_BYTES_S = 8.0e12
# what a kernel that only reads memory reaches on this chip (16 bytes a lane, 8 loads in flight, 8 GB): the
# achievable ceiling beside the nominal one
HBM_MEASURED_BYTES_S = 6.3e12
PEAK_FLOPS = {"fp16": 2.5e15, "bf16": 2.5e15, "fp32": 157.3e12}

# the shapes of the benchmark configurations; the default run is the Llama-3.1-8B shape
SHAPES = {
    "llama-3.1-8b": dict(num_hidden_layers=32, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8,
                         head_dim=128, intermediate_size=14336, vocab_size=128256, rope_theta=500000.0,
                         rms_norm_eps=1e-5, max_position_embeddings=8192, tie_word_embeddings=False),
    "llama-3.2-1b": dict(num_hidden_layers=16, hidden_size=2048, num_attention_heads=32, num_key_value_heads=8,
                         head_dim=64, intermediate_size=8192, vocab_size=128256, rope_theta=500000.0,
                         rms_norm_eps=1e-5, max_position_embeddings=8192, tie_word_embeddings=True),
    "llama-2-7b": dict(num_hidden_layers=32, hidden_size=4096, num_attention_heads=32, num_key_value_heads=32,
                       head_dim=128, intermediate_size=11008, vocab_size=32000, rope_theta=10000.0,
                       rms_norm_eps=1e-5, max_position_embeddings=4096, tie_word_embeddings=False),
}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--shape", default="llama-3.1-8b", choices=sorted(SHAPES))
    ap.add_argument("--context", type=int, default=0, help="context length (default: the shape's)")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the shape has (named in config)")
    ap.add_argument("--ragged-prefill", type=int, default=0,
                    help="also time one step of this many prompts with lengths uniform in 16..2048")
    ap.add_argument("--dtype", default="fp16", choices=["fp16", "bf16"])
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--points", default="1,16,64", help="further decode batch sizes, comma separated ('' for none)")
    ap.add_argument("--no-other-shapes", action="store_true",
                    help="leave out the 1B ragged step and the 7B batch-64 decode that the default run adds to points")
    ap.add_argument("--no-further-sizes", action="store_true",
                    help="leave out the long contexts, batch 128 and the generation run that the default run adds to points")
    ap.add_argument("--generate", type=int, default=0,
                    help="also generate for this many 128-token prompts with budgets drawn from 16..512 tokens")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this library runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    if args.shape == "llama-3.1-8b" and not args.no_further_sizes and args.prefill_tokens == 2048:
        args.also_prefill = [16, 128]                      # short prompts, which run as recorded steps
    line = measure(args)
    for n, r in line.pop("also_prefill", {}).items():
        line["points"][f"prefill_{n}_ms"] = r["ms"]
    if args.shape == "llama-3.1-8b" and not args.no_other_shapes and not args.ragged_prefill:
        # the other two benchmark shapes, each in an engine of its own, into the same line
        import copy
        a1 = copy.copy(args)
        a1.shape, a1.batch, a1.points, a1.ragged_prefill, a1.context, a1.layers = "llama-3.2-1b", 8, "", 32, 0, 0
        a1.steps, a1.warmup, a1.prefill_tokens = 8, 2, 0
        r1 = measure(a1)["ragged_prefill"]
        a7 = copy.copy(args)
        a7.shape, a7.batch, a7.points, a7.ragged_prefill, a7.context, a7.layers = "llama-2-7b", 64, "", 0, 0, 0
        a7.steps, a7.warmup, a7.prefill_tokens = 24, 4, 0
        r7 = measure(a7)
        line["points"].update({
            "ragged_1b_32prompts_ms": r1["ms"], "ragged_1b_32prompts_tokens": r1["tokens"],
            "ragged_1b_32prompts_frac_of_peak": r1["frac"],
            "decode_7b_b64_ctx4096_ms": r7["ms_per_step"], "decode_7b_b64_ctx4096_tokens_s": r7["value"],
            "decode_7b_b64_ctx4096_frac_of_hbm": r7["roofline"]["frac"]})
        line["config"]["also_in_points"] = ("llama-3.2-1b shape (16 layers, hidden 2048, 32/8 heads of 64, intermediate "
                                            "8192, tied): one step of 32 prompts of 16..2048 tokens; llama-2-7b shape (32 "
                                            "layers, hidden 4096, 32/32 heads of 128, intermediate 11008, vocab 32000): "
                                            "decode batch 64 at context 4096")
    if args.shape == "llama-3.1-8b" and not args.no_further_sizes and not args.ragged_prefill and not args.generate:
        # further sizes of the headline shape, in engines of their own: a long context, a large batch, and
        # generation whose batch shrinks
        import copy
        al = copy.copy(args)
        al.batch, al.points, al.context, al.layers, al.steps, al.warmup = 8, "", 32768, 0, 16, 3
        al.prefill_tokens, al.also_prefill = 32768, [8192]
        rl = measure(al)
        ag = copy.copy(args)
        ag.batch, ag.points, ag.context, ag.layers, ag.steps, ag.warmup = 128, "", 2048, 0, 24, 4
        ag.prefill_tokens, ag.generate = 0, 64
        rg = measure(ag)
        gen = rg["generation"]
        line["points"].update({
            "decode_b8_ctx32768_ms": rl["ms_per_step"], "decode_b8_ctx32768_tokens_s": rl["value"],
            "decode_b8_ctx32768_frac_of_hbm": rl["roofline"]["frac"],
            "prefill_32768_ms": rl["prefill"]["ms"], "prefill_32768_frac_of_peak": rl["prefill"]["frac"],
            "prefill_8192_ms": rl["also_prefill"]["8192"]["ms"],
            "prefill_8192_frac_of_peak": rl["also_prefill"]["8192"]["frac"],
            "decode_b128_ctx2048_ms": rg["ms_per_step"], "decode_b128_ctx2048_tokens_s": rg["value"],
            "decode_b128_ctx2048_frac_of_hbm": rg["roofline"]["frac"],
            "generate_64x128_tokens_s": gen["tokens_s"], "generate_64x128_new_tokens": gen["new_tokens"],
            "generate_64x128_decode_s": gen["decode_s"], "generate_64x128_steps_eager": gen["steps_eager"],
            "generate_64x128_steps_recorded": gen["steps_recorded"], "generate_64x128_steps_replayed": gen["steps_replayed"],
            "generate_64x128_replayed_frac": gen["replayed_frac"]})
        line["config"]["also_in_points"] = (line["config"].get("also_in_points", "") + "; the headline shape again: decode "
                                            "batch 8 at context 32768, prompts of 8192 and 32768 tokens, decode batch 128 at "
                                            "context 2048, and generation for 64 prompts of 128 tokens with budgets uniform "
                                            "in 16..512 (greedy, no stop token; tokens/s of the decode phase)").lstrip("; ")
    print(json.dumps(line))
    return 0


def measure(args) -> dict:
    """One engine of one shape: decode at the given batch sizes, the prefill of one prompt, optionally a
    ragged step of many prompts; returns the benchmark line."""
    import gc

    import torch

    import llm_infer_amd
    from llm_infer_amd.sampling import Sampler

    SHAPE = dict(SHAPES[args.shape], hidden_act="silu", architectures=["LlamaForCausalLM"])
    args.context = args.context or SHAPE["max_position_embeddings"]
    args.layers = args.layers or SHAPE["num_hidden_layers"]
    raw = dict(SHAPE, num_hidden_layers=args.layers, max_position_embeddings=args.context)
    cfg = llm_infer_amd.config_from_dict(raw)
    points = [int(p) for p in args.points.split(",") if p]
    batches = [args.batch] + [p for p in points if p != args.batch]
    also_prefill = list(getattr(args, "also_prefill", None) or [])
    max_tokens = max(max(batches) * args.context, args.prefill_tokens, args.ragged_prefill * 2048,
                     args.generate * 640, *also_prefill) + 64 * max(batches)
    t0 = time.time()
    engine = llm_infer_amd.random_model(cfg, seed=0, dtype=args.dtype, max_tokens=max_tokens,
                                        n_slots=max(max(batches), args.ragged_prefill, args.generate))
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    model, cache = engine.model, engine.cache
    elem = 2

    # bytes a decode step has to read: every matrix once, the norms, and the cache of the live requests
    weight_bytes = 0
    for name, spec in model.params().items():
        n = 1
        for s in spec.shape:
            n *= s
        if name.startswith("model.embed_tokens"):
            if cfg.tie_word_embeddings:
                weight_bytes += n * elem               # the tied head reads the whole table
            continue                                   # else only the batch's rows are read
        weight_bytes += n * (4 if spec.kind == "vector" else elem)
    kv_bytes_per_token = cache.bytes_per_token()

    def decode_run(batch, steps, warmup, timed=True):
        """Fills `batch` sequences to just below the context length with random keys and values,
        then times `steps` decode steps.  The runner records a step the first time it meets its size and its
        bucket of context lengths, and the window of positions crosses a bucket's edge (8,128 tokens at a
        context of 8,192); `timed=False` walks the window once beforehand so that the timed steps are all
        replays, as every step of a long generation is."""
        start = args.context - steps - warmup - 2            # warm-up enqueues one step more than it returns
        slots = [engine.alloc_slot() for _ in range(batch)]
        cache.grow(slots, [start] * batch)
        for g in cache.groups:
            g.storage.normal_(0.0, 1.0)
        sampler = Sampler(temperature=0.0, seed=0)
        sampler.start(cache, slots, list(range(batch)))
        runner = engine.decode_runner(sampler, use_graph=True)
        gen = torch.Generator().manual_seed(batch)
        toks = torch.randint(0, cfg.vocab_size, (batch,), generator=gen).tolist()
        # as in the generation loop: the next step is enqueued before this one's tokens are read
        for _ in range(warmup):
            toks = runner.run(slots, toks, may_follow=True)
        runner.drain()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for i in range(steps):
            toks = runner.run(slots, toks, may_follow=i + 1 < steps)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        ctx_mid = start + warmup + 1 + steps // 2
        for s in slots:
            engine.free_slot(s)
        return dt, ctx_mid

    results = {}
    for b in batches:
        decode_run(b, args.steps, args.warmup, timed=False)
        recorded = engine.decode_counts["recorded"]
        dt, ctx_mid = decode_run(b, args.steps, args.warmup)
        assert engine.decode_counts["recorded"] == recorded, "a step was recorded inside the timed steps"
        results[b] = (dt, ctx_mid)
        print(f"[bench] decode batch {b}: {dt / args.steps * 1e3:.3f} ms/step, "
              f"{b * args.steps / dt:.1f} tok/s", file=sys.stderr, flush=True)

    # prefill of one prompt
    L, d, H, K, hd, F, V = (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads,
                            cfg.num_key_value_heads, cfg.head_dim, cfg.intermediate_size, cfg.vocab_size)

    def prefill_run(T, repeats):
        gen = torch.Generator().manual_seed(1)
        prompt = torch.randint(0, cfg.vocab_size, (T,), generator=gen).tolist()
        times = []
        for i in range(repeats):
            slot = engine.alloc_slot()
            torch.cuda.synchronize()
            t = time.perf_counter()
            engine.step([slot], [prompt])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t)
            engine.free_slot(slot)
        flops = 2 * T * (d * (H + 2 * K) * hd + H * hd * d + 3 * d * F) * L + 2 * V * d + 2 * H * hd * T * (T + 1) * L
        return min(times[1:]), flops

    T = max(1, args.prefill_tokens)
    prefill_s, prefill_flops = prefill_run(T, (4 if T <= 4096 else 3) if args.prefill_tokens > 0 else 2)
    more_prefills = {}
    for n in also_prefill:
        s_, f_ = prefill_run(n, 5 if n <= 512 else 3)      # (a short prompt is run eagerly, recorded, then replayed)
        more_prefills[str(n)] = {"value": round(n / s_, 1), "tokens": n, "ms": round(s_ * 1e3, 3),
                                 "frac": round(f_ / s_ / PEAK_FLOPS[args.dtype], 4)}

    generation = None
    if args.generate:
        # the generation loop itself on a batch whose sequences end at different times: prompts of 128 tokens,
        # a budget for each request drawn from 16..512, greedy, no stop token
        gen = torch.Generator().manual_seed(3)
        prompts = [torch.randint(0, cfg.vocab_size, (128,), generator=gen).tolist() for _ in range(args.generate)]
        budgets = torch.randint(16, 513, (args.generate,), generator=gen).tolist()
        engine.generate(prompts[:2], max_new_tokens=4, temperature=0.0, stop_token_ids=())       # first-use work
        before = dict(engine.decode_counts)
        _, stats = engine.generate(prompts, max_new_tokens=budgets, temperature=0.0, stop_token_ids=(), return_stats=True)
        did = {k: engine.decode_counts[k] - before[k] for k in before}
        steps = max(1, sum(did.values()))
        # the first token of every request comes out of the prefill step; the decode phase makes the others
        decoded = stats.generated_tokens - len(prompts)
        generation = {"prompts": len(prompts), "new_tokens": stats.generated_tokens, "decode_s": round(stats.decode_s, 4),
                      "prefill_s": round(stats.prefill_s, 4), "tokens_s": round(decoded / stats.decode_s, 1),
                      "steps_eager": did["eager"], "steps_recorded": did["recorded"], "steps_replayed": did["replayed"],
                      "replayed_frac": round(did["replayed"] / steps, 4), "mean_batch": round(decoded / steps, 2)}
        print(f"[bench] generation: {generation}", file=sys.stderr, flush=True)

    ragged = None
    if args.ragged_prefill:
        gen = torch.Generator().manual_seed(2)
        lens = torch.randint(16, 2049, (args.ragged_prefill,), generator=gen).tolist()
        prompts = [torch.randint(0, cfg.vocab_size, (n,), generator=gen).tolist() for n in lens]
        best = None
        for i in range(3):
            slots = [engine.alloc_slot() for _ in prompts]
            torch.cuda.synchronize()
            t = time.perf_counter()
            engine.step(slots, prompts)
            torch.cuda.synchronize()
            t = time.perf_counter() - t
            best = t if best is None or (i > 0 and t < best) else best
            for sl in slots:
                engine.free_slot(sl)
        flop = sum(2 * n * (d * (H + 2 * K) * hd + H * hd * d + 3 * d * F) * L + 2 * H * hd * n * (n + 1) * L
                   for n in lens) + 2 * V * d * len(lens)
        ragged = {"prompts": len(lens), "tokens": sum(lens), "ms": round(best * 1e3, 3),
                  "value": round(sum(lens) / best, 1), "frac": round(flop / best / PEAK_FLOPS[args.dtype], 4)}

    dt, ctx_mid = results[args.batch]
    ms = dt / args.steps * 1e3
    step_bytes = weight_bytes + args.batch * d * elem + kv_bytes_per_token * ctx_mid * args.batch
    achieved = step_bytes / (dt / args.steps)
    line = {
        "metric": f"decode tokens/s, {args.shape} shape, batch {args.batch}, context {args.context}",
        "value": round(args.batch * args.steps / dt, 2), "unit": "tokens/s", "n_gpus": 1,
        # (untimed: a first walk over the same positions, in which the steps are recorded, then the warm-up)
        "steps": args.steps, "warmup": 2 * args.warmup + args.steps, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: random weights N(0, 0.02), uniform random token ids, cache filled with random "
                "keys and values up to the context length",
        "config": {
            "model": f"{args.shape} shape", "layers": L, "layers_of_shape": SHAPE["num_hidden_layers"],
            "hidden": d, "heads": H, "kv_heads": K, "head_dim": hd, "intermediate": F, "vocab": V,
            "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_norm_eps, "tied": cfg.tie_word_embeddings,
            "global_batch": args.batch, "seq_len": args.context, "context": args.context,
            "prefill_tokens": T, "parallelism": "1 GPU", "sampling": "greedy",
        },
        "prefill": {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
                    "frac": round(prefill_flops / prefill_s / PEAK_FLOPS[args.dtype], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_BYTES_S / 1e9,
                     "unit": "GB/s", "frac": round(achieved / HBM_BYTES_S, 4),
                     "measured_peak": HBM_MEASURED_BYTES_S / 1e9,
                     "frac_of_measured": round(achieved / HBM_MEASURED_BYTES_S, 4)},
        "points": {f"decode_b{b}": round(b * args.steps / results[b][0], 2) for b in batches if b != args.batch},
    }
    if ragged:
        line["ragged_prefill"] = ragged
    if more_prefills:
        line["also_prefill"] = more_prefills
    if generation:
        line["generation"] = generation
    del engine, model, cache
    gc.collect()
    torch.cuda.empty_cache()
    return line


if __name__ == "__main__":
    sys.exit(main())
