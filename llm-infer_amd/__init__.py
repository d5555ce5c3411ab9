"""llm_infer_amd: a small, whole Llama generation library for one MI355X.

    engine = llm_infer_amd.load("model_dir", max_tokens=65536)
    new_tokens = engine.generate([[1, 2, 3], [4, 5]], max_new_tokens=16, temperature=0.0)
"""
from .config import ConfigError, LlamaConfig
from .tensor import Tensor
from .registry import (config_from_dict, config_from_folder, register_architecture, register_block,
                       register_embedding, register_feed_forward, register_head, register_mixer,
                       register_norm, register_position)

__version__ = "0.1.0"

register_architecture("LlamaForCausalLM", LlamaConfig)


def load(folder: str, dtype: str | None = None, max_tokens: int = 8192, n_slots=None, kv_round=None):
    """Open a model on the GPU: a folder with config.json and model.safetensors, or a GGUF file
    with unquantized tensors (the reference's own format) or the folder that holds one.
    ``dtype`` None runs the model in its own type: ``torch_dtype`` of config.json, else the type its
    matrices are stored in (float32 files run the 32-bit path).
    ``kv_round="float16"`` with ``dtype="float32"`` rounds keys and values as the reference's cache does."""
    from .engine import Engine
    return Engine.from_folder(folder, dtype=dtype, max_tokens=max_tokens, n_slots=n_slots, kv_round=kv_round)


def random_model(config, seed: int = 0, dtype: str | None = None, max_tokens: int = 8192, n_slots=None, kv_round=None,
                 same_as_folder=None):
    """An engine with random weights from a configuration and a seed, without a folder.  Up to half a billion
    parameters (or with ``same_as_folder=True``) the weights are those that ``write_random_model`` writes for
    the same seed and dtype; larger models draw theirs with the GPU's generator, which is other values."""
    from .engine import Engine
    return Engine.from_random(config, seed=seed, dtype=dtype, max_tokens=max_tokens, n_slots=n_slots, kv_round=kv_round,
                              same_as_folder=same_as_folder)


def write_random_model(folder: str, config, seed: int = 0, dtype: str = "bfloat16") -> None:
    """Write config.json and model.safetensors for a configuration and a seed."""
    from .weights import write_random_model as _w
    _w(folder, config, seed, dtype)
