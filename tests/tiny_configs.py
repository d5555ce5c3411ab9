"""Small configurations of the architecture that differ in every size and option."""

# 2 layers, GQA 4/2, head 16, ffn 172 (no multiple of 8), untied
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "intermediate_size": 172, "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-5,
    "max_position_embeddings": 128, "tie_word_embeddings": False, "hidden_act": "silu",
}

# 3 layers, MQA 3/1, head 32, tied head, other theta and eps
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
    "intermediate_size": 256, "vocab_size": 384, "rope_theta": 500000.0, "rms_norm_eps": 1e-6,
    "max_position_embeddings": 256, "tie_word_embeddings": True, "hidden_act": "silu",
}

# 1 layer, MHA 5/5, explicit head_dim 48 != hidden/heads, half of each head rotated,
# odd vocabulary, long context, the gate's other activation
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 1, "hidden_size": 80, "num_attention_heads": 5, "head_dim": 48,
    "intermediate_size": 136, "vocab_size": 331, "rope_theta": 1000.0, "rms_norm_eps": 1e-4,
    "partial_rotary_factor": 0.5,
    "max_position_embeddings": 1024, "tie_word_embeddings": False, "hidden_act": "gelu",
}

# head sizes that are no multiple of 16: 40 (GQA 6/2, 24 of the 40 dimensions rotated, tied head) and 100 (MHA)
TINY_D = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 72, "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 40,
    "intermediate_size": 100, "vocab_size": 210, "rope_theta": 20000.0, "rms_norm_eps": 1e-5,
    "partial_rotary_factor": 0.6,
    "max_position_embeddings": 192, "tie_word_embeddings": True, "hidden_act": "silu",
}
TINY_E = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 1, "hidden_size": 200, "num_attention_heads": 2, "num_key_value_heads": 2,
    "intermediate_size": 152, "vocab_size": 129, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
    "max_position_embeddings": 320, "tie_word_embeddings": False, "hidden_act": "silu",
}

# rotated pairs (j, j + 12) of a 32-wide head instead of adjacent ones (a checkpoint in the row order the
# reference's files are permuted from): GQA 6/3, explicit head size, three quarters of it rotated
TINY_F = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 88, "num_attention_heads": 6, "num_key_value_heads": 3, "head_dim": 32,
    "intermediate_size": 120, "vocab_size": 301, "rope_theta": 5000.0, "rms_norm_eps": 3e-6,
    "partial_rotary_factor": 0.75, "rope_pairing": "half",
    "max_position_embeddings": 160, "tie_word_embeddings": False, "hidden_act": "silu",
}

ALL = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D, "E": TINY_E, "F": TINY_F}
