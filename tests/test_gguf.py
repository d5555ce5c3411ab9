"""GGUF files with unquantized tensors, the reference's own model format (src/gguf.cpp,
docs/gguf.md): metadata and tensors written and read back, the configuration taken from the
metadata keys the reference requires, tensor names mapped to the ones the model asks for, and the
errors."""
import os
import struct

import pytest
import torch

import llm_infer_amd
from llm_infer_amd.config.spec import ConfigError
from llm_infer_amd.tokenizer import Tokenizer
from llm_infer_amd.weights import (GGUFError, GGUFFile, WeightError, read_checkpoint, write_gguf, write_random_gguf,
                                   write_random_model)
from llm_infer_amd.weights.loader import check_tensors
from tiny_configs import TINY_A, TINY_B, TINY_C


def test_metadata_and_tensors_come_back(tmp_path):
    path = str(tmp_path / "x.gguf")
    g = torch.Generator().manual_seed(0)
    tensors = {"a.weight": torch.randn(5, 12, generator=g).to(torch.float16), "b": torch.randn(7, generator=g),
               "c": torch.randn(3, 2, 4, generator=g).to(torch.bfloat16)}
    md = {"general.architecture": "llama", "llama.block_count": 3, "big": 1 << 40, "neg": -5, "eps": 1e-5,
          "flag": True, "name": "tiny", "tokens": ["a", "b c", "é"], "ids": [1, 2, 3], "scores": [0.5, -1.0]}
    for align in (32, 64):
        write_gguf(path, md, tensors, alignment=align)
        f = GGUFFile(path)
        assert f.version == 3 and f.names() == list(tensors)
        assert f.metadata["llama.block_count"] == 3 and f.metadata["big"] == 1 << 40 and f.metadata["neg"] == -5
        assert abs(f.metadata["eps"] - 1e-5) < 1e-12 and f.metadata["flag"] is True and f.metadata["name"] == "tiny"
        assert f.metadata["tokens"] == ["a", "b c", "é"] and list(f.metadata["ids"]) == [1, 2, 3]
        assert [round(float(x), 3) for x in f.metadata["scores"]] == [0.5, -1.0]
        for name, t in tensors.items():
            dtype, shape = f.info(name)
            assert dtype == t.dtype and shape == tuple(t.shape)       # slowest dimension first
            assert torch.equal(f.tensor(name), t)
    # the dimensions lie fastest first in the file (docs/gguf.md): [12, 5] for the [5, 12] matrix
    raw = open(path, "rb").read()
    at = raw.index(b"a.weight") + len(b"a.weight")
    assert struct.unpack_from("<IQQ", raw, at) == (2, 12, 5)


def test_errors(tmp_path):
    path = str(tmp_path / "bad.gguf")
    open(path, "wb").write(b"GGML" + b"\0" * 40)
    with pytest.raises(GGUFError, match="not a GGUF file"):
        GGUFFile(path)
    open(path, "wb").close()
    with pytest.raises(GGUFError, match="not a GGUF file"):
        GGUFFile(path)
    open(path, "wb").write(b"GGUF" + struct.pack("<I", 1) + b"\0" * 40)
    with pytest.raises(GGUFError, match="version 1"):
        GGUFFile(path)
    open(path, "wb").write(b"GGUF" + struct.pack("<IQQ", 3, 1, 0) + struct.pack("<Q", 1000) + b"ab")
    with pytest.raises(GGUFError, match="past the end"):
        GGUFFile(path)
    write_gguf(path, {}, {"w": torch.zeros(4, 32, dtype=torch.float16)})
    data = bytearray(open(path, "rb").read())
    at = data.index(b"w") + 1 + 4 + 16                      # name, n_dims, two dimensions -> the tensor type
    struct.pack_into("<I", data, at, 12)                    # Q4_K
    open(path, "wb").write(bytes(data))
    with pytest.raises(GGUFError, match="Q4_K.*quantized weights are not supported"):
        GGUFFile(path).info("w")
    write_gguf(path, {}, {"w": torch.zeros(4, 32, dtype=torch.float16)})
    whole = open(path, "rb").read()
    open(path, "wb").write(whole[:-10])
    with pytest.raises(GGUFError, match="does not lie inside the file"):
        GGUFFile(path)


@pytest.mark.parametrize("raw", [TINY_A, TINY_B, TINY_C])
def test_random_model_as_gguf_reads_back_like_the_folder(raw, tmp_path):
    """The same seed written as a folder and as a GGUF file: the same configuration (but for what
    GGUF does not say) and the same tensors under the model's names."""
    cfg = llm_infer_amd.config_from_dict(raw)
    folder, path = str(tmp_path / "m"), str(tmp_path / "model.gguf")
    write_random_model(folder, cfg, seed=3, dtype="float16")
    write_random_gguf(path, cfg, seed=3, dtype="float16", vocabulary=[f"t{i}" for i in range(cfg.vocab_size)])
    for where in (path, str(tmp_path)):                      # the file, or the folder that holds it
        if where != path:
            os.rename(folder, str(tmp_path / "elsewhere"))   # so that the folder holds only the GGUF file
            folder = str(tmp_path / "elsewhere")
        got = llm_infer_amd.config_from_folder(where)
        for key in ("num_hidden_layers", "hidden_size", "intermediate_size", "num_attention_heads",
                    "num_key_value_heads", "head_dim", "vocab_size", "max_position_embeddings", "rotary_dim",
                    "tie_word_embeddings", "rope_pairing"):
            assert getattr(got, key) == getattr(cfg, key), key
        assert abs(got.rope_theta - cfg.rope_theta) < 1e-3 * cfg.rope_theta
        assert abs(got.rms_norm_eps - cfg.rms_norm_eps) < 1e-3 * cfg.rms_norm_eps
    from llm_infer_amd.engine.model import DecoderModel
    model = DecoderModel(cfg.model_spec(), dtype=torch.float32, device="cpu", allocate=False)
    needed = model.params()
    a = read_checkpoint(folder)
    b = read_checkpoint(path, needed, cfg)
    check_tensors(needed, b, model.ignorable_names())
    assert sorted(b.names()) == sorted(a.names())
    for name in needed:
        assert b.info(name) == a.info(name)
        assert torch.equal(b.tensor(name), a.tensor(name))
    names = set(GGUFFile(path).names())
    assert {"token_embd.weight", "output_norm.weight", "blk.0.attn_q.weight", "blk.0.ffn_down.weight",
            "blk.0.attn_norm.weight"} <= names
    assert ("output.weight" in names) == (not cfg.tie_word_embeddings)
    tok = Tokenizer.from_model(path)
    assert tok is not None and tok.encode("t7t1", add_bos=False) == [7, 1]


def test_a_gguf_file_that_does_not_fit(tmp_path):
    cfg = llm_infer_amd.config_from_dict(TINY_A)
    path = str(tmp_path / "model.gguf")
    write_random_gguf(path, cfg, seed=0)
    f = GGUFFile(path)
    md = dict(f.metadata)
    tensors = {n: f.tensor(n) for n in f.names()}
    # required metadata: every missing key is named
    bad = {k: v for k, v in md.items() if k not in ("llama.block_count", "llama.rope.dimension_count")}
    write_gguf(path, bad, tensors)
    with pytest.raises(ConfigError, match="llama.block_count, llama.rope.dimension_count"):
        llm_infer_amd.config_from_folder(path)
    write_gguf(path, {k: v for k, v in md.items() if k != "general.architecture"}, tensors)
    with pytest.raises(ConfigError, match="general.architecture"):
        llm_infer_amd.config_from_folder(path)
    write_gguf(path, dict(md, **{"general.architecture": "falcon"}), tensors)
    with pytest.raises(ConfigError, match="unknown GGUF architecture 'falcon'; known: llama"):
        llm_infer_amd.config_from_folder(path)
    # u64 where others write u32 (src/gguf.cpp:94-102), no vocabulary size: rows of the embedding
    import numpy as np
    big = {k: (np.uint64(v) if k.startswith("llama.") and isinstance(v, int) else
               np.float64(v) if k.startswith("llama.") and isinstance(v, float) else v)
           for k, v in md.items() if k != "llama.vocab_size"}
    write_gguf(path, big, tensors)
    got = llm_infer_amd.config_from_folder(path)
    assert got.vocab_size == cfg.vocab_size and got.num_hidden_layers == cfg.num_hidden_layers
    assert abs(got.rms_norm_eps - cfg.rms_norm_eps) < 1e-12
    # tensors: missing, unexpected and misshapen in one error, under the file's... model's names
    t2 = dict(tensors)
    del t2["blk.1.ffn_up.weight"]
    t2["blk.0.attn_q.weight"] = t2["blk.0.attn_q.weight"][:, :-8].contiguous()
    t2["extra.weight"] = torch.zeros(3)
    t2["rope_freqs.weight"] = torch.ones(8)                  # exported by other tools; never bound
    write_gguf(path, md, t2)
    from llm_infer_amd.engine.model import DecoderModel
    model = DecoderModel(cfg.model_spec(), dtype=torch.float32, device="cpu", allocate=False)
    from llm_infer_amd.weights.loader import load_into
    with pytest.raises(WeightError) as e:
        load_into(model, path, cfg)
    msg = str(e.value)
    assert "model.layers.1.mlp.up_proj.weight" in msg and "extra.weight" in msg and "rope_freqs" not in msg
    assert "model.layers.0.self_attn.q_proj.weight: expected [64, 64], got [64, 56]" in msg


def test_model_info_tells_what_a_folder_or_a_file_holds(tmp_path):
    """The tool of the reference's tools/gguf_info.cpp and tools/hf_info.cpp: configuration, tensors,
    tokenizer; exit status 1 and the loader's one error if the tensors do not fit."""
    import io

    from llm_infer_amd.info import describe, main
    from safetensors.torch import load_file, save_file
    cfg = llm_infer_amd.config_from_dict(dict(TINY_B, bos_token_id=1, eos_token_id=2))
    folder, path = str(tmp_path / "m"), str(tmp_path / "m.gguf")
    write_random_model(folder, cfg, 0)
    vocab = ["<unk>", "<s>", "</s>"] + [f"t{i}" for i in range(cfg.vocab_size - 4)] + ["<|eot_id|>"]
    write_random_gguf(path, cfg, 0, vocabulary=vocab)
    for where, fmt in ((folder, "config.json + safetensors"), (path, "GGUF")):
        out = io.StringIO()
        assert describe(where, 3, out) == 0
        text = out.getvalue()
        assert fmt in text and f"hidden_size: {cfg.hidden_size}" in text and "The tensors fit the model." in text
        assert f"Tensor count: {len(read_checkpoint(where, config=cfg).names())}" in text and "more" in text
    out = io.StringIO()
    describe(path, 0, out)
    assert f"Tokenizer vocab size: {cfg.vocab_size}" in out.getvalue() and "BOS token ID: 1" in out.getvalue()
    assert f"EOT token ID: {cfg.vocab_size - 1}" in out.getvalue()
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    del tensors["model.norm.weight"]
    save_file(tensors, os.path.join(folder, "model.safetensors"))
    out = io.StringIO()
    assert describe(folder, 0, out) == 1 and "missing tensors (1): model.norm.weight" in out.getvalue()
    assert main([]) == 1 and main(["-h"]) == 0 and main([str(tmp_path / "nothing")]) == 1
