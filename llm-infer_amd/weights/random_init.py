"""Random-weights mode: tensors from a parameter table and a seed.

Matrices and tables are N(0, 0.02), norm vectors 1 + N(0, 0.01).  Every tensor
has a generator of its own, seeded by (seed, tensor name), so a tensor's values
depend on neither the order nor the presence of the others.  The reference has
no such mode.
"""
from __future__ import annotations

import hashlib
import json
import os

import torch

from .safetensors_io import write_safetensors

MATRIX_STD = 0.02
VECTOR_STD = 0.01


def _seed_for(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & 0x7FFF_FFFF_FFFF_FFFF


def random_tensor(name: str, spec, seed: int, matrix_dtype: torch.dtype, device="cpu") -> torch.Tensor:
    g = torch.Generator(device=device).manual_seed(_seed_for(seed, name))
    if spec.kind == "int":
        raise ValueError(f"{name}: integer tables have no random initialisation")
    if spec.kind == "vector" or spec.init == "ones":
        return 1.0 + VECTOR_STD * torch.randn(spec.shape, generator=g, device=device, dtype=torch.float32)
    n = 1
    for s in spec.shape:
        n *= s
    if str(device) == "cpu" or n < (1 << 26):
        return (MATRIX_STD * torch.randn(spec.shape, generator=g, device=device, dtype=torch.float32)).to(matrix_dtype)
    # large tensors on the device: fill row blocks so that the float32 staging stays small
    out = torch.empty(spec.shape, device=device, dtype=matrix_dtype)
    rows = max(1, (1 << 26) // max(1, n // spec.shape[0]))
    for lo in range(0, spec.shape[0], rows):
        hi = min(spec.shape[0], lo + rows)
        block = torch.randn((hi - lo,) + tuple(spec.shape[1:]), generator=g, device=device, dtype=torch.float32)
        out[lo:hi] = (MATRIX_STD * block).to(matrix_dtype)
    return out


def random_tensors(params: dict, seed: int, matrix_dtype=torch.bfloat16, device="cpu") -> dict:
    return {name: random_tensor(name, spec, seed, matrix_dtype, device) for name, spec in params.items()}


def write_random_model(folder: str, config, seed: int, dtype: str = "bfloat16") -> None:
    """Write ``config.json`` and ``model.safetensors`` for a configuration and a seed."""
    from ..engine.model import DecoderModel
    matrix_dtype = {"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32}[dtype]
    model = DecoderModel(config.model_spec(), dtype=torch.float32, device="cpu", allocate=False)
    os.makedirs(folder, exist_ok=True)
    raw = config.to_dict()
    raw["torch_dtype"] = dtype
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(raw, f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      random_tensors(model.params(), seed, matrix_dtype), {"format": "pt", "seed": seed})


def write_random_gguf(path: str, config, seed: int, dtype: str = "float16", vocabulary=None) -> None:
    """The same random model as one GGUF file (matrices float16 by default, norms float32), under
    the tensor names and metadata keys the reference reads; ``vocabulary``: optional list of token
    strings for ``tokenizer.ggml.tokens``."""
    from ..engine.model import DecoderModel
    from .gguf_io import write_gguf
    matrix_dtype = {"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32}[dtype]
    model = DecoderModel(config.model_spec(), dtype=torch.float32, device="cpu", allocate=False)
    md = config.gguf_metadata()
    if vocabulary is not None:
        md["tokenizer.ggml.tokens"] = list(vocabulary)
    tensors = random_tensors(model.params(), seed, matrix_dtype)
    write_gguf(path, md, {config.gguf_tensor_name(n): t for n, t in tensors.items()})
