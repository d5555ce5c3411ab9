"""``model_info``: what a model folder or GGUF file holds, without a GPU, in the manner of the
reference's gguf_info and hf_info tools (tools/gguf_info.cpp:98-226, tools/hf_info.cpp): the
configuration as parsed, the tensors and whether they fit the model, and the tokenizer.

    model_info <model_dir | model.gguf> [-n <tensors to list, default 12>]
"""
from __future__ import annotations

import sys

USAGE = "Usage: model_info <model_dir | model.gguf> [-n <tensors to list>]"


def describe(path: str, n_list: int = 12, out=sys.stdout) -> int:
    import torch

    import llm_infer_amd
    from llm_infer_amd.engine.model import DecoderModel
    from llm_infer_amd.registry import find_gguf
    from llm_infer_amd.tokenizer import Tokenizer
    from llm_infer_amd.weights.loader import WeightError, check_tensors, read_checkpoint

    def say(text=""):
        print(text, file=out)

    say(f"Loading model: {path}")
    gguf = find_gguf(path)
    config = llm_infer_amd.config_from_folder(path)
    say(f"Format: {'GGUF (' + gguf + ')' if gguf else 'config.json + safetensors'}")
    say(f"Architecture: {getattr(config, 'architecture', type(config).__name__)}")
    say("Configuration:")
    fields = getattr(config, "__dataclass_fields__", None)
    for key in (fields or sorted(vars(config))):
        say(f"  {key}: {getattr(config, key)}")
    model = DecoderModel(config.model_spec(), dtype=torch.float32, device="cpu", allocate=False)
    needed = model.params()
    n_params = 0
    for spec in needed.values():
        c = 1
        for s in spec.shape:
            c *= s
        n_params += c
    say(f"Parameters the model needs: {len(needed)} tensors, {n_params:,} elements")
    ckpt = read_checkpoint(path, needed, config)
    names = ckpt.names()
    say(f"Tensor count: {len(names)}")
    for name in names[:n_list]:
        try:
            dtype, shape = ckpt.info(name)
            say(f"  {name}: {str(dtype).replace('torch.', '')} {list(shape)}")
        except ValueError as e:
            say(f"  {name}: {e}")
    if len(names) > n_list:
        say(f"  ... and {len(names) - n_list} more")
    status = 0
    try:
        check_tensors(needed, ckpt, model.ignorable_names() + list(getattr(config, "gguf_ignorable", ())))
        say("The tensors fit the model.")
    except (WeightError, ValueError) as e:
        say(str(e))
        status = 1
    eos = config.eos_token_ids[0] if getattr(config, "eos_token_ids", ()) else None
    tok = Tokenizer.from_model(path, getattr(config, "bos_token_id", None), eos)
    if tok is None:
        say("Tokenizer: none (requests are token ids)")
    else:
        say(f"Tokenizer vocab size: {len(tok.piece)}")
        say(f"BOS token ID: {tok.bos_id}")
        say(f"EOS token ID: {tok.eos_id}")
        if tok.eot_id is not None:
            say(f"EOT token ID: {tok.eot_id}")
        if len(tok.piece) != config.vocab_size:
            say(f"Warning: Vocab size mismatch - Tokenizer: {len(tok.piece)}, model: {config.vocab_size}")
    return status


def main(argv=None) -> int:
    argv = sys.argv[1:] if argv is None else argv
    if not argv or argv[0] in ("-h", "--help"):
        print(USAGE)
        return 0 if argv else 1
    n = 12
    if len(argv) >= 3 and argv[1] == "-n":
        try:
            n = int(argv[2])
        except ValueError:
            print(USAGE, file=sys.stderr)
            return 1
    elif len(argv) != 1:
        print(USAGE, file=sys.stderr)
        return 1
    try:
        return describe(argv[0], n)
    except (OSError, ValueError) as e:
        print(f"Error: {e}", file=sys.stderr)
        return 1
