"""Typed configuration of the Llama decoder, read from its own config.json keys.

Keys and defaults are those of the reference's HF constructor
(src/model/config.cpp:74-137): ``num_key_value_heads`` defaults to the number of
heads (:81), ``head_dim`` to hidden/heads (:82), ``rope_theta`` to 10000 (:88),
``partial_rotary_factor`` to 1 (:89-90), ``rms_norm_eps`` to 1e-5 (:93).  One default
departs from that constructor on purpose: a config.json without ``hidden_act`` gets
"silu", the activation of the Llama decoder and what the reference's GGUF constructor,
the only one wired to its model, fixes (config.cpp:163); the HF constructor would take
"gelu" (config.cpp:97).  The
reference's model reads no ``tie_word_embeddings``, ``eos_token_id`` or
``architectures``; those are read here because a generation library needs them.
"""
from __future__ import annotations

import json
import os
import sys
from dataclasses import dataclass

from .spec import ConfigError, LayerSpec, ModelSpec, PartSpec, ScheduleEntry, SubLayerSpec

_REQUIRED = ("num_hidden_layers", "hidden_size", "intermediate_size", "num_attention_heads",
             "vocab_size", "max_position_embeddings")          # config.cpp:77-85 (.at() throws)
_DTYPES = ("float32", "float16", "bfloat16")


@dataclass(frozen=True)
class LlamaConfig:
    num_hidden_layers: int
    hidden_size: int
    intermediate_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    max_position_embeddings: int
    rope_theta: float
    rotary_dim: int
    rms_norm_eps: float
    hidden_act: str
    tie_word_embeddings: bool
    torch_dtype: str | None
    bos_token_id: int | None
    eos_token_ids: tuple
    rope_pairing: str
    architecture: str = "LlamaForCausalLM"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, c: dict) -> "LlamaConfig":
        missing = [k for k in _REQUIRED if k not in c]
        if missing:
            raise ConfigError("config.json lacks required keys: " + ", ".join(missing))
        n_heads = int(c["num_attention_heads"])
        hidden = int(c["hidden_size"])
        if n_heads <= 0:
            raise ConfigError("num_attention_heads must be positive")
        if "head_dim" not in c and hidden % n_heads != 0:
            # config.cpp:134-136
            raise ConfigError("hidden_size must be divisible by num_attention_heads")
        head_dim = int(c.get("head_dim") or hidden // n_heads)
        n_kv = int(c.get("num_key_value_heads") or n_heads)
        rotary_dim = int(head_dim * float(c.get("partial_rotary_factor", 1.0)))
        eos = c.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, list) else [eos]))
        act = c.get("hidden_act", "silu")          # not config.cpp:97's "gelu": see the module's docstring
        if c.get("rope_scaling") not in (None, {}):
            # the reference parses a rope scale and never uses it (include/llama.hpp:14)
            print("warning: rope_scaling is ignored, positions are rotated unscaled", file=sys.stderr)
        archs = c.get("architectures") or ["LlamaForCausalLM"]
        cfg = cls(
            num_hidden_layers=int(c["num_hidden_layers"]), hidden_size=hidden,
            intermediate_size=int(c["intermediate_size"]), num_attention_heads=n_heads,
            num_key_value_heads=n_kv, head_dim=head_dim, vocab_size=int(c["vocab_size"]),
            max_position_embeddings=int(c["max_position_embeddings"]),
            rope_theta=float(c.get("rope_theta", 10000.0)), rotary_dim=rotary_dim,
            rms_norm_eps=float(c.get("rms_norm_eps", 1e-5)), hidden_act=act,
            tie_word_embeddings=bool(c.get("tie_word_embeddings", False)),
            torch_dtype=c.get("torch_dtype"), bos_token_id=c.get("bos_token_id"),
            eos_token_ids=eos_ids, rope_pairing=c.get("rope_pairing", "adjacent"),
            architecture=archs[0])
        cfg.validate()
        return cfg

    # GGUF: the reference's own model files (src/gguf.cpp:86-168 reads these keys, u32 or u64)
    gguf_architecture = "llama"
    _GGUF_REQUIRED = ("context_length", "embedding_length", "block_count", "feed_forward_length",
                      "rope.dimension_count", "attention.head_count", "attention.layer_norm_rms_epsilon")

    @classmethod
    def from_gguf(cls, metadata: dict, tensor_shapes: dict) -> "LlamaConfig":
        """``metadata``: the file's key/value pairs; ``tensor_shapes``: GGUF tensor name -> shape."""
        md = {k[len("llama."):]: v for k, v in metadata.items() if k.startswith("llama.")}
        missing = ["llama." + k for k in cls._GGUF_REQUIRED if k not in md]
        if missing:
            raise ConfigError("the GGUF file lacks required metadata: " + ", ".join(missing))
        hidden, n_heads = int(md["embedding_length"]), int(md["attention.head_count"])
        if n_heads <= 0 or (hidden % n_heads != 0 and "attention.key_length" not in md):
            raise ConfigError("llama.embedding_length must be divisible by llama.attention.head_count")
        head_dim = int(md.get("attention.key_length") or hidden // n_heads)
        emb = tensor_shapes.get("token_embd.weight")
        # the reference falls back to a tokenizer key of another type (src/gguf.cpp:162-167); the
        # rows of the embedding table say it without doubt
        vocab = int(md.get("vocab_size") or (emb[0] if emb else 0) or len(metadata.get("tokenizer.ggml.tokens", ())))
        if "expert_count" in md and int(md["expert_count"]) > 0:
            raise ConfigError("this GGUF file holds a model with experts; only the dense decoder is built")
        eos = metadata.get("tokenizer.ggml.eos_token_id")
        bos = metadata.get("tokenizer.ggml.bos_token_id")
        cfg = cls(
            num_hidden_layers=int(md["block_count"]), hidden_size=hidden,
            intermediate_size=int(md["feed_forward_length"]), num_attention_heads=n_heads,
            num_key_value_heads=int(md.get("attention.head_count_kv") or n_heads), head_dim=head_dim,
            vocab_size=vocab, max_position_embeddings=int(md["context_length"]),
            rope_theta=float(md.get("rope.freq_base", 10000.0)), rotary_dim=int(md["rope.dimension_count"]),
            rms_norm_eps=float(md["attention.layer_norm_rms_epsilon"]), hidden_act="silu",
            tie_word_embeddings="output.weight" not in tensor_shapes, torch_dtype=None,
            bos_token_id=None if bos is None else int(bos),
            eos_token_ids=() if eos is None else (int(eos),), rope_pairing="adjacent")
        cfg.validate()
        return cfg

    def gguf_metadata(self) -> dict:
        """The metadata that reads back as this configuration."""
        md = {"general.architecture": "llama", "general.quantization_version": 2,
              "llama.context_length": self.max_position_embeddings, "llama.embedding_length": self.hidden_size,
              "llama.block_count": self.num_hidden_layers, "llama.feed_forward_length": self.intermediate_size,
              "llama.rope.dimension_count": self.rotary_dim, "llama.attention.head_count": self.num_attention_heads,
              "llama.attention.head_count_kv": self.num_key_value_heads,
              "llama.attention.layer_norm_rms_epsilon": float(self.rms_norm_eps),
              "llama.rope.freq_base": float(self.rope_theta), "llama.vocab_size": self.vocab_size}
        if self.head_dim * self.num_attention_heads != self.hidden_size:
            md["llama.attention.key_length"] = self.head_dim
        if self.bos_token_id is not None:
            md["tokenizer.ggml.bos_token_id"] = int(self.bos_token_id)
        if self.eos_token_ids:
            md["tokenizer.ggml.eos_token_id"] = int(self.eos_token_ids[0])
        return md

    @staticmethod
    def gguf_tensor_name(name: str) -> str:
        """This library's tensor name (the config.json world's) -> the GGUF name the reference binds
        (src/model/model.cpp:25-38, src/model/block.cpp:18-62)."""
        fixed = {"model.embed_tokens.weight": "token_embd.weight", "model.norm.weight": "output_norm.weight",
                 "lm_head.weight": "output.weight"}
        if name in fixed:
            return fixed[name]
        parts = {"input_layernorm": "attn_norm", "post_attention_layernorm": "ffn_norm",
                 "self_attn.q_proj": "attn_q", "self_attn.k_proj": "attn_k", "self_attn.v_proj": "attn_v",
                 "self_attn.o_proj": "attn_output", "mlp.gate_proj": "ffn_gate", "mlp.up_proj": "ffn_up",
                 "mlp.down_proj": "ffn_down"}
        head = "model.layers."
        if name.startswith(head) and name.endswith(".weight"):
            layer, _, rest = name[len(head):-len(".weight")].partition(".")
            if rest in parts and layer.isdigit():
                return f"blk.{layer}.{parts[rest]}.weight"
        return name

    # Tensors that a GGUF file of this architecture may hold without the model using them: the frequency
    # factors of a rotation scaling that other tools export beside the weights.  The reference binds
    # tensors by name and never looks at them (src/model/model.cpp:25-38), and applies no such scaling.
    gguf_ignorable = ("rope_freqs.weight",)

    @classmethod
    def from_folder(cls, folder: str) -> "LlamaConfig":
        with open(os.path.join(folder, "config.json")) as f:
            return cls.from_dict(json.load(f))

    def validate(self) -> None:
        for name in ("num_hidden_layers", "hidden_size", "intermediate_size", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "vocab_size", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(f"num_attention_heads ({self.num_attention_heads}) must be a multiple of "
                              f"num_key_value_heads ({self.num_key_value_heads})")
        if self.rotary_dim % 2 != 0 or not 0 < self.rotary_dim <= self.head_dim:
            raise ConfigError(f"the rotated part of a head must be even and within head_dim, got "
                              f"{self.rotary_dim} of {self.head_dim}")
        if self.hidden_act not in ("silu", "gelu"):
            # the reference warns and takes gelu (config.cpp:97-105); a wrong activation is refused here
            raise ConfigError(f"hidden_act {self.hidden_act!r}: the feed-forward's gate takes 'silu' or 'gelu' "
                              "(the tanh form, include/kernels_cpu.hpp:179-184)")
        if self.rope_pairing not in ("adjacent", "half"):
            raise ConfigError(f"rope_pairing must be 'adjacent' or 'half', got {self.rope_pairing!r}")
        if self.torch_dtype is not None and self.torch_dtype not in _DTYPES:
            raise ConfigError(f"Unsupported torch_dtype: {self.torch_dtype}")
        if not self.rope_theta > 0 or not self.rms_norm_eps >= 0:
            raise ConfigError("rope_theta must be positive and rms_norm_eps non-negative")

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        out = {
            "architectures": [self.architecture], "model_type": "llama",
            "num_hidden_layers": self.num_hidden_layers, "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size, "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads, "head_dim": self.head_dim,
            "vocab_size": self.vocab_size, "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta, "partial_rotary_factor": self.rotary_dim / self.head_dim,
            "rms_norm_eps": self.rms_norm_eps, "hidden_act": self.hidden_act,
            "tie_word_embeddings": self.tie_word_embeddings,
        }
        if self.torch_dtype is not None:
            out["torch_dtype"] = self.torch_dtype
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        if self.rope_pairing != "adjacent":
            out["rope_pairing"] = self.rope_pairing
        return out

    # ------------------------------------------------------------------ the model as data
    def model_spec(self) -> ModelSpec:
        """RMSNorm -> attention with rotation -> RMSNorm -> SwiGLU in every layer
        (src/model/block.cpp:106-224), final norm and output head (model.cpp:79-98)."""
        norm = PartSpec("rmsnorm", {"size": self.hidden_size, "eps": self.rms_norm_eps})
        position = PartSpec("rope", {"theta": self.rope_theta, "rotary_dim": self.rotary_dim,
                                     "head_dim": self.head_dim, "pairing": self.rope_pairing})
        mixer = PartSpec("attention", {
            "hidden_size": self.hidden_size, "n_heads": self.num_attention_heads,
            "n_kv_heads": self.num_key_value_heads, "head_dim": self.head_dim,
            "scale": self.head_dim ** -0.5, "window": None})
        ffn = PartSpec("gated_mlp", {"hidden_size": self.hidden_size,
                                     "intermediate_size": self.intermediate_size, "activation": self.hidden_act})
        layers = []
        for i in range(self.num_hidden_layers):
            p = f"model.layers.{i}."
            layers.append(LayerSpec(
                block="pre_norm",
                sublayers=(SubLayerSpec("mixer", mixer.with_prefix(p + "self_attn."),
                                        norm=norm.with_prefix(p + "input_layernorm.")),
                           SubLayerSpec("feed_forward", ffn.with_prefix(p + "mlp."),
                                        norm=norm.with_prefix(p + "post_attention_layernorm."))),
                position=position))
        spec = ModelSpec(
            hidden_size=self.hidden_size, vocab_size=self.vocab_size,
            max_positions=self.max_position_embeddings,
            embedding=PartSpec("embedding", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size},
                               "model.embed_tokens."),
            layers=tuple(layers),
            schedule=tuple(ScheduleEntry(i) for i in range(self.num_hidden_layers)),
            final_norm=norm.with_prefix("model.norm."),
            head=PartSpec("lm_head", {"vocab_size": self.vocab_size, "hidden_size": self.hidden_size,
                                      "tied": self.tie_word_embeddings}, "lm_head."),
            stop_token_ids=self.eos_token_ids)
        spec.validate()
        return spec
