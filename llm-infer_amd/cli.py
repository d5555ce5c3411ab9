"""``infer``: the command line, in the manner of the reference's tool (tools/infer.cpp:112-349).

    infer <model_dir> [-i <prompt> | -f <file> | --tokens 1,2,3 | --tokens-file F]
          [-n 256] [-t 1.0] [--seed 0] [-T <context>] [-d hip] [--dtype <name>]

Options the reference has keep their names and meanings: -i, -f, -n (tokens to generate,
256), -t (temperature, 1.0; <= 0 is greedy), --seed, -T (context length override), -d (device;
here only "hip": there is no CPU path), -h.  The model is a folder with config.json and
model.safetensors, or, as for the reference, a GGUF file (F32/F16/BF16 tensors; its metadata
is the configuration and holds the vocabulary).  Differences: prompts may be given as token ids (one --tokens or one
line of --tokens-file for each request of a batch); seed 0 is a fixed seed, not a random one.
"""
from __future__ import annotations

import json
import sys
import time

USAGE = """Usage: infer <model_dir | model.gguf> [options]
Example: infer model_dir -i "Hello, world!"

Options:
  -h                    Display this help message
  -d <device>           Device to use: hip (default: hip)
  -i <string>           Input prompt (needs tokenizer.json in the folder or a GGUF vocabulary)
  -f <file>             Input prompt from file
  --tokens <ids>        Input prompt as comma separated token ids (repeat for a batch)
  --tokens-file <file>  One prompt a line, token ids separated by commas or blanks
  -n <int>              Number of tokens to generate (default: 256)
  -t <float>            Temperature for sampling (default: 1.0)
  -T <int>              Context length override (default: model max)
  --seed <int>          Random seed (default: 0)
  --dtype <name>        bfloat16, float16 or float32 (default: the model's own)
  --kv-round <name>     With --dtype float32: keys and values rounded to float16 (the reference's cache) or bfloat16
  --slots <int>         Most sequences that run as one batch (default: all requests given)
  --random-weights      Ignore the model's tensors: random weights from --seed-weights
  --seed-weights <int>  Seed of the random weights (default: 0)
  --config <json>       With --random-weights: the configuration file (the model argument is not opened)
  --no-graph            Launch every decode step kernel by kernel

A folder whose q and k rows are in the original Hugging Face order (rotated pairs j and j + rotary_dim/2,
never permuted for adjacent pairs as GGUF files are) needs "rope_pairing": "half" in its config.json."""


def parse_ids(text: str) -> list:
    return [int(t) for t in text.replace(",", " ").split()]


def parse_args(argv):
    cfg = dict(model=None, device="hip", prompt=None, prompt_file=None, tokens=[], tokens_file=None,
               max_tokens=256, temperature=1.0, seed=0, context=None, dtype=None, random=False,
               seed_weights=0, graph=True, help=False, slots=None, config=None, kv_round=None)
    if any(a in ("-h", "--help") for a in argv):
        cfg["help"] = True
        return cfg
    if not argv:
        return None
    cfg["model"] = argv[0]
    takes = {"-d": ("device", str), "-i": ("prompt", str), "-f": ("prompt_file", str), "-n": ("max_tokens", int),
             "-t": ("temperature", float), "-T": ("context", int), "--seed": ("seed", int),
             "--dtype": ("dtype", str), "--tokens-file": ("tokens_file", str), "--seed-weights": ("seed_weights", int),
             "--slots": ("slots", int), "--config": ("config", str), "--kv-round": ("kv_round", str)}
    i = 1
    while i < len(argv):
        a = argv[i]
        if a in takes:
            if i + 1 >= len(argv):
                return None
            key, conv = takes[a]
            try:
                cfg[key] = conv(argv[i + 1])
            except ValueError:
                print(f"Invalid value for {a}: {argv[i + 1]}", file=sys.stderr)
                return None
            i += 2
        elif a == "--tokens":
            if i + 1 >= len(argv):
                return None
            cfg["tokens"].append(parse_ids(argv[i + 1]))
            i += 2
        elif a == "--random-weights":
            cfg["random"] = True
            i += 1
        elif a == "--no-graph":
            cfg["graph"] = False
            i += 1
        else:
            print(f"Unknown argument: {a}", file=sys.stderr)
            return None
    if cfg["device"] != "hip":
        print(f"Invalid device: {cfg['device']}. Must be 'hip'", file=sys.stderr)
        return None
    given = sum(bool(x) for x in (cfg["prompt"], cfg["prompt_file"], cfg["tokens"], cfg["tokens_file"]))
    if given == 0:
        print("Must specify one of -i <prompt>, -f <file>, --tokens <ids>, --tokens-file <file>", file=sys.stderr)
        return None
    if given > 1:
        print("Cannot specify more than one of -i, -f, --tokens, --tokens-file", file=sys.stderr)
        return None
    return cfg


def run(cfg) -> int:
    import llm_infer_amd
    from llm_infer_amd.engine import Engine
    from llm_infer_amd.tokenizer import Tokenizer
    print(f"Loading model: {cfg['model']}")
    if cfg["config"]:
        if not cfg["random"]:
            raise RuntimeError("--config goes with --random-weights")
        try:
            with open(cfg["config"]) as f:
                config = llm_infer_amd.config_from_dict(json.load(f))
        except OSError:
            raise RuntimeError(f"Failed to open configuration file: {cfg['config']}")
    else:
        config = llm_infer_amd.config_from_folder(cfg["model"])
    if cfg["context"]:
        raw = config.to_dict()
        raw["max_position_embeddings"] = cfg["context"]
        raw["eos_token_id"] = list(config.eos_token_ids) or None
        config = llm_infer_amd.config_from_dict(raw)
    tok = None if cfg["config"] else Tokenizer.from_model(
        cfg["model"], config.bos_token_id, config.eos_token_ids[0] if config.eos_token_ids else None)
    if cfg["prompt_file"]:
        try:
            with open(cfg["prompt_file"], encoding="utf-8") as f:
                cfg["prompt"] = f.read()
        except OSError:
            raise RuntimeError(f"Failed to open prompt file: {cfg['prompt_file']}")
    if cfg["prompt"] is not None:
        if tok is None:
            raise RuntimeError("the model has no tokenizer (tokenizer.json in the folder, or tokenizer.ggml.tokens "
                               "in a GGUF file): give the prompt as token ids (--tokens)")
        prompts = [tok.encode(cfg["prompt"], True)]
    elif cfg["tokens_file"]:
        with open(cfg["tokens_file"]) as f:
            prompts = [parse_ids(line) for line in f if line.strip()]
    else:
        prompts = cfg["tokens"]
    if cfg["slots"] is not None and cfg["slots"] <= 0:
        raise RuntimeError("--slots must be positive")
    n_slots = min(cfg["slots"] or len(prompts), len(prompts)) or 1
    each = sorted((-(-min(len(p) + cfg["max_tokens"], config.max_position_embeddings) // 64) * 64 for p in prompts),
                  reverse=True)
    need = sum(each[:n_slots])                       # the largest batch that can be live at once
    if cfg["random"]:
        engine = Engine.from_random(config, seed=cfg["seed_weights"], dtype=cfg["dtype"], max_tokens=need,
                                    n_slots=n_slots, kv_round=cfg["kv_round"])
    else:
        engine = Engine.from_folder(cfg["model"], dtype=cfg["dtype"], max_tokens=need, n_slots=n_slots,
                                    kv_round=cfg["kv_round"])
        engine.config = config
        if cfg["context"]:
            engine.max_positions = min(engine.max_positions, cfg["context"])
    print("Model load successful")
    print(f"  Layers: {config.num_hidden_layers}")
    print(f"  Dimensions: {config.hidden_size}")
    print(f"  Heads: {config.num_attention_heads}")
    print(f"  KV Heads: {config.num_key_value_heads}")
    print(f"  Vocab size: {config.vocab_size}")
    print(f"  Max seq len: {engine.max_positions}")
    print(f"  Device: {cfg['device']}")
    print()
    for p in prompts:
        print(f"Encoded {len(p)} tokens")
    stop = set(config.eos_token_ids)
    if tok is not None and tok.eot_id is not None:
        stop.add(tok.eot_id)
    print("Warming up...")
    engine.generate([prompts[0][:1]], max_new_tokens=2, temperature=0.0, stop_token_ids=())
    print("Prefilling...")
    t0 = time.perf_counter()
    outputs, stats = engine.generate(prompts, max_new_tokens=cfg["max_tokens"], temperature=cfg["temperature"],
                                     seed=cfg["seed"], stop_token_ids=stop, return_stats=True,
                                     use_graph=cfg["graph"])
    total_s = time.perf_counter() - t0
    print(f"Prefill completed in {stats.prefill_s:.3f}s ({stats.prompt_tokens / max(stats.prefill_s, 1e-9):.1f} tok/s)")
    print()
    print("Generating...")
    for i, out in enumerate(outputs):
        label = "Output" if len(outputs) == 1 else f"Output {i}"
        if tok is not None:
            print(f"{label}: {tok.decode(out)}")
        print(f"{label} tokens: {json.dumps(out)}")
    print()
    n_prompt, n_gen = stats.prompt_tokens, stats.generated_tokens
    print("Generation Statistics:")
    print(f"  Prompt tokens: {n_prompt}")
    print(f"  Generated tokens: {n_gen}")
    print(f"  Total tokens: {n_prompt + n_gen}")
    print(f"  Prefill time: {stats.prefill_s:.3f}s ({n_prompt / max(stats.prefill_s, 1e-9):.1f} tok/s)")
    print(f"  Generation time: {stats.decode_s:.3f}s ({n_gen / max(stats.decode_s, 1e-9):.1f} tok/s)")
    print(f"  Total time: {total_s:.3f}s ({(n_prompt + n_gen) / max(total_s, 1e-9):.1f} tok/s)")
    print(f"  Temperature: {cfg['temperature']:.2f}")
    return 0


def main(argv=None) -> int:
    cfg = parse_args(list(sys.argv[1:] if argv is None else argv))
    if cfg is None:
        print(USAGE)
        return 1
    if cfg["help"]:
        print(USAGE)
        return 0
    try:
        return run(cfg)
    except Exception as e:                      # tools/infer.cpp:345-348
        print(f"Error: {e}", file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(main())
