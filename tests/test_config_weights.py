"""Configuration, registry, safetensors reader/writer, weight checks and random-weights mode (no GPU)."""
import json
import os
import struct

import pytest
import torch

import llm_infer_amd
import plain_llama as P
from llm_infer_amd.config import ConfigError, LlamaConfig
from llm_infer_amd.engine.model import DecoderModel
from llm_infer_amd.weights import (SafetensorsError, SafetensorsFile, WeightError, check_tensors, read_checkpoint,
                                   write_random_model, write_safetensors)
from llm_infer_amd.weights.loader import ParamSpec, kept_dtype
from tiny_configs import ALL, TINY_A, TINY_B, TINY_C


def test_defaults_follow_the_reference():
    c = llm_infer_amd.config_from_dict({
        "architectures": ["LlamaForCausalLM"], "num_hidden_layers": 2, "hidden_size": 64,
        "intermediate_size": 100, "num_attention_heads": 4, "vocab_size": 50, "max_position_embeddings": 32})
    assert c.num_key_value_heads == 4 and c.head_dim == 16            # config.cpp:81-82
    assert c.rope_theta == 10000.0 and c.rotary_dim == 16             # config.cpp:88-90
    assert c.rms_norm_eps == 1e-5 and not c.tie_word_embeddings       # config.cpp:93
    assert c.eos_token_ids == () and c.rope_pairing == "adjacent"
    # the one default that departs from the reference's HF constructor ("gelu", config.cpp:97): a Llama
    # folder without hidden_act runs silu, as the reference's GGUF constructor fixes it (config.cpp:163)
    assert c.hidden_act == "silu" and c.torch_dtype is None
    raw = {"hidden_size": 8, "num_attention_heads": 2, "num_hidden_layers": 1, "intermediate_size": 8, "vocab_size": 4}
    assert P.sizes(raw)["act"] == "silu" and P.sizes(dict(raw, hidden_act="gelu"))["act"] == "gelu"


def test_every_size_comes_from_the_config():
    for raw in ALL.values():
        c = llm_infer_amd.config_from_dict(raw)
        s = P.sizes(raw)
        assert (c.num_hidden_layers, c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim,
                c.intermediate_size, c.vocab_size, c.rope_theta, c.rotary_dim, c.rms_norm_eps,
                c.tie_word_embeddings) == (s["n_layers"], s["d"], s["n_heads"], s["n_kv"], s["hd"], s["ffn"],
                                           s["vocab"], s["theta"], s["rotary"], s["eps"], s["tied"])
        assert llm_infer_amd.config_from_dict(c.to_dict()) == c       # config.json round trip
    c = llm_infer_amd.config_from_dict(dict(TINY_A, eos_token_id=[3, 9], bos_token_id=1))
    assert c.eos_token_ids == (3, 9) and c.model_spec().stop_token_ids == (3, 9)
    assert llm_infer_amd.config_from_dict(dict(TINY_A, eos_token_id=7)).eos_token_ids == (7,)


@pytest.mark.parametrize("change,message", [
    ({"hidden_size": 66}, "divisible"), ({"num_key_value_heads": 3}, "multiple"),
    ({"hidden_act": "relu"}, "silu"), ({"partial_rotary_factor": 0.45}, "even"),
    ({"num_hidden_layers": 0}, "positive"), ({"torch_dtype": "int8"}, "Unsupported torch_dtype"),
    ({"rope_pairing": "odd"}, "rope_pairing"), ({"architectures": ["MambaForCausalLM"]}, "unknown architecture"),
    ({"architectures": []}, "names no architecture"),
])
def test_bad_configurations_are_refused(change, message):
    with pytest.raises(ConfigError, match=message):
        llm_infer_amd.config_from_dict(dict(TINY_A, **change))


def test_missing_keys_are_listed():
    raw = dict(TINY_A)
    del raw["vocab_size"], raw["intermediate_size"]
    with pytest.raises(ConfigError, match="intermediate_size, vocab_size"):
        llm_infer_amd.config_from_dict(raw)


def test_model_spec_is_data():
    spec = llm_infer_amd.config_from_dict(TINY_B).model_spec()
    assert len(spec.layers) == 3 and [e.layer for e in spec.schedule] == [0, 1, 2]
    l1 = spec.layers[1]
    mix, ffn = l1.sublayers                                   # the sub-layers in the order in which they run
    assert l1.block == "pre_norm" and (mix.role, ffn.role) == ("mixer", "feed_forward")
    assert mix.part.kind == "attention" and ffn.part.kind == "gated_mlp"
    assert mix.part.params["n_kv_heads"] == 1 and mix.part.params["scale"] == 32 ** -0.5
    assert mix.part.prefix == "model.layers.1.self_attn." and l1.position.params["theta"] == 500000.0
    assert mix.norm.prefix == "model.layers.1.input_layernorm." and mix.post_norm is None
    assert ffn.norm.prefix == "model.layers.1.post_attention_layernorm." and ffn.norm.kind == "rmsnorm"
    assert spec.head.params["tied"] and spec.final_norm.params["eps"] == 1e-6


def _model(raw):
    return DecoderModel(llm_infer_amd.config_from_dict(raw).model_spec(), torch.float32, "cpu", allocate=False)


def test_parameter_table_matches_the_plain_implementation():
    for raw in ALL.values():
        params = _model(raw).params()
        assert {k: tuple(v.shape) for k, v in params.items()} == P.tensor_shapes(raw)
        assert all(v.kind == "vector" for k, v in params.items() if "norm" in k)


def test_safetensors_round_trip_and_library_agreement(tmp_path):
    from safetensors.torch import load_file, save_file
    tensors = {"a": torch.randn(3, 5).to(torch.bfloat16), "b": torch.arange(7, dtype=torch.int32),
               "c": torch.randn(2, 2, 2), "d": torch.randn(4).to(torch.float16), "e": torch.empty(0, 3)}
    mine = str(tmp_path / "mine.safetensors")
    write_safetensors(mine, tensors, {"note": "x"})
    lib = load_file(mine)                                             # the library reads what we wrote
    f = SafetensorsFile(mine)
    assert f.metadata == {"note": "x"} and sorted(f.names()) == sorted(tensors)
    for k, t in tensors.items():
        assert torch.equal(lib[k], t) and torch.equal(f.tensor(k), t) and f.info(k) == (t.dtype, tuple(t.shape))
    theirs = str(tmp_path / "theirs.safetensors")
    save_file({k: v for k, v in tensors.items()}, theirs)            # and we read what the library wrote
    g = SafetensorsFile(theirs)
    for k, t in tensors.items():
        assert torch.equal(g.tensor(k), t)
    with pytest.raises(SafetensorsError, match="Tensor not found"):
        f.tensor("zz")


def _raw_file(path, header: dict, data: bytes, length=None):
    blob = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob) if length is None else length))
        f.write(blob)
        f.write(data)


def test_safetensors_errors(tmp_path):
    p = str(tmp_path / "x.safetensors")
    open(p, "wb").write(b"abc")
    with pytest.raises(SafetensorsError, match="Header too small"):
        SafetensorsFile(p)
    _raw_file(p, {}, b"", length=10 ** 9)
    with pytest.raises(SafetensorsError, match="Header too large"):
        SafetensorsFile(p)
    _raw_file(p, {}, b"", length=500)
    with pytest.raises(SafetensorsError, match="Invalid header length"):
        SafetensorsFile(p)
    with open(p, "wb") as f:
        f.write(struct.pack("<Q", 4) + b"{{{{")
    with pytest.raises(SafetensorsError, match="Invalid JSON"):
        SafetensorsFile(p)
    _raw_file(p, {"t": {"dtype": "Q4", "shape": [1], "data_offsets": [0, 4]}}, b"0000")
    with pytest.raises(SafetensorsError, match="Unknown dtype"):
        SafetensorsFile(p)
    _raw_file(p, {"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 4]}}, b"0000")
    with pytest.raises(SafetensorsError, match="size mismatch"):
        SafetensorsFile(p)
    _raw_file(p, {"t": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]},
                  "u": {"dtype": "F32", "shape": [1], "data_offsets": [2, 6]}}, b"000000")
    with pytest.raises(SafetensorsError, match="Invalid offset"):
        SafetensorsFile(p)
    _raw_file(p, {"t": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]}}, b"0000zz")
    with pytest.raises(SafetensorsError, match="incomplete buffer"):
        SafetensorsFile(p)


def test_one_error_lists_missing_unexpected_and_wrong(tmp_path):
    folder = str(tmp_path)
    w = P.random_weights(TINY_A, 0)
    del w["model.layers.1.mlp.up_proj.weight"], w["model.norm.weight"]
    w["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 32, dtype=torch.bfloat16)
    w["model.layers.0.self_attn.rotary.inv_freq"] = torch.zeros(8)
    w["model.layers.1.input_layernorm.weight"] = torch.zeros(64, dtype=torch.int32)
    P.write_model(folder, TINY_A, w)
    with pytest.raises(WeightError) as e:
        check_tensors(_model(TINY_A).params(), read_checkpoint(folder))
    msg = str(e.value)
    assert "missing tensors (2): model.norm.weight, model.layers.1.mlp.up_proj.weight" in msg \
        or "missing tensors (2): model.layers.1.mlp.up_proj.weight, model.norm.weight" in msg
    assert "unexpected tensors (1): model.layers.0.self_attn.rotary.inv_freq" in msg
    assert "model.layers.0.self_attn.q_proj.weight: expected [64, 64], got [64, 32]" in msg
    assert "model.layers.1.input_layernorm.weight: expected floating point" in msg
    with pytest.raises(WeightError, match="no model.safetensors"):
        read_checkpoint(str(tmp_path / "nowhere"))


def test_tied_head_may_be_in_the_file_but_untied_must_be(tmp_path):
    w = P.random_weights(TINY_B, 0)
    w["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    P.write_model(str(tmp_path / "b"), TINY_B, w)
    m = _model(TINY_B)
    check_tensors(m.params(), read_checkpoint(str(tmp_path / "b")), m.ignorable_names())
    w = P.random_weights(TINY_A, 0)
    del w["lm_head.weight"]
    P.write_model(str(tmp_path / "a"), TINY_A, w)
    with pytest.raises(WeightError, match="missing tensors \\(1\\): lm_head.weight"):
        check_tensors(_model(TINY_A).params(), read_checkpoint(str(tmp_path / "a")))


def test_kept_dtypes():
    bf, f16, f32 = torch.bfloat16, torch.float16, torch.float32
    assert kept_dtype(bf, "matrix", bf) == bf and kept_dtype(f16, "matrix", bf) == bf
    assert kept_dtype(f32, "matrix", bf) == f32                      # stored in 32-bit stays so
    assert kept_dtype(bf, "vector", bf) == f32 and kept_dtype(bf, "matrix", f32) == f32
    assert kept_dtype(torch.int64, "int", bf) == torch.int32


def test_the_model_files_choose_the_compute_dtype(tmp_path):
    from llm_infer_amd.weights import choose_dtype, stored_matrix_dtype
    bf, f16, f32 = torch.bfloat16, torch.float16, torch.float32
    said = []
    # nothing asked for: torch_dtype of config.json, else what is stored, else bfloat16; no word about it
    assert choose_dtype(None, "float16", f16, said.append) == f16
    assert choose_dtype(None, None, f16, said.append) == f16 and choose_dtype(None, None, f32, said.append) == f32
    assert choose_dtype(None, None, None, said.append) == bf and choose_dtype(None, "float32", None) == f32
    assert choose_dtype("float32", "float16", f16, said.append) == f32          # widening loses nothing
    assert said == []
    # one line when the stored values are narrowed or change their 16-bit type
    assert choose_dtype("bfloat16", "float16", f16, said.append) == bf and "three bits" in said[-1]
    assert choose_dtype("float16", None, bf, said.append) == f16 and "65504" in said[-1]
    assert choose_dtype("bf16", None, f32, said.append) == bf and "rounded" in said[-1]
    assert choose_dtype(None, "bfloat16", f16, said.append) == bf and "torch_dtype" in said[-1]
    assert len(said) == 4
    with pytest.raises(ValueError, match="one of bfloat16, float16, float32"):
        choose_dtype("int8", None, None)
    # a float16 folder opened with no option keeps float16 matrices (and float32 norms)
    cfg = llm_infer_amd.config_from_dict(TINY_A)
    for name, dt in (("float16", f16), ("float32", f32), ("bfloat16", bf)):
        folder = str(tmp_path / name)
        write_random_model(folder, cfg, seed=1, dtype=name)
        table = _model(TINY_A).params()
        ckpt = read_checkpoint(folder)
        stored = stored_matrix_dtype(table, ckpt)
        assert stored == dt and llm_infer_amd.config_from_folder(folder).torch_dtype == name
        compute = choose_dtype(None, llm_infer_amd.config_from_folder(folder).torch_dtype, stored, said.append)
        assert compute == dt and kept_dtype(stored, "matrix", compute) == dt and kept_dtype(f32, "vector", compute) == f32
    assert len(said) == 4


def test_random_weights_mode_writes_a_model_folder(tmp_path):
    cfg = llm_infer_amd.config_from_dict(TINY_C)
    a, b, c = (str(tmp_path / n) for n in "abc")
    write_random_model(a, cfg, seed=3)
    write_random_model(b, cfg, seed=3)
    write_random_model(c, cfg, seed=4)
    wa, wb, wc = P.load_weights(a), P.load_weights(b), P.load_weights(c)     # read by the library
    assert P.read_config(a)["num_attention_heads"] == 5 and P.read_config(a)["torch_dtype"] == "bfloat16"
    assert llm_infer_amd.config_from_folder(a) == llm_infer_amd.config_from_dict(dict(TINY_C, torch_dtype="bfloat16"))
    assert {k: tuple(v.shape) for k, v in wa.items()} == P.tensor_shapes(TINY_C)
    for k in wa:
        assert torch.equal(wa[k], wb[k]) and not torch.equal(wa[k], wc[k])
        if "norm" in k:
            assert wa[k].dtype == torch.float32 and abs(wa[k].mean().item() - 1) < 0.01
        else:
            assert wa[k].dtype == torch.bfloat16 and 0.015 < wa[k].float().std().item() < 0.025
    check_tensors(_model(TINY_C).params(), read_checkpoint(a))
    write_random_model(str(tmp_path / "h"), cfg, seed=3, dtype="float16")
    assert P.load_weights(str(tmp_path / "h"))["lm_head.weight"].dtype == torch.float16


def test_sharded_checkpoint(tmp_path):
    w = P.random_weights(TINY_A, 0)
    names = list(w)
    from safetensors.torch import save_file
    save_file({k: w[k] for k in names[:5]}, str(tmp_path / "s1.safetensors"))
    save_file({k: w[k] for k in names[5:]}, str(tmp_path / "s2.safetensors"))
    index = {"weight_map": {k: ("s1.safetensors" if i < 5 else "s2.safetensors") for i, k in enumerate(names)}}
    json.dump(index, open(tmp_path / "model.safetensors.index.json", "w"))
    ck = read_checkpoint(str(tmp_path))
    check_tensors(_model(TINY_A).params(), ck)
    assert torch.equal(ck.tensor(names[7]), w[names[7]])
