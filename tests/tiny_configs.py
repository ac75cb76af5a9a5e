"""Small configurations of the architecture for tests.  They differ in every size and
option: heads and groups, head size, widths that are no power of two, layers, vocabulary,
eps, rotary base and scaling, bias, per-head norm, tied head, window."""

TINY_A = {   # Qwen2 style: bias, no qk norm, untied, head_dim = hidden / heads
    "architectures": ["Qwen2ForCausalLM"], "vocab_size": 256, "hidden_size": 64, "intermediate_size": 176,
    "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 2,
    "rms_norm_eps": 1e-6, "rope_theta": 10000.0, "max_position_embeddings": 128,
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "eos_token_id": 255,
}

TINY_B = {   # Qwen3 style: qk norm, MQA, explicit head_dim (q width 192 != hidden 96), tied
    "architectures": ["Qwen3ForCausalLM"], "vocab_size": 384, "hidden_size": 96, "intermediate_size": 288,
    "num_hidden_layers": 3, "num_attention_heads": 6, "num_key_value_heads": 1, "head_dim": 32,
    "rms_norm_eps": 1e-5, "rope_theta": 1000000.0, "max_position_embeddings": 256,
    "tie_word_embeddings": True, "torch_dtype": "bfloat16", "eos_token_id": [382, 383],
}

TINY_C = {   # Llama style: llama3 rotary scaling, head_dim 48, odd sizes, 5 heads in one group... 
    "architectures": ["LlamaForCausalLM"], "vocab_size": 331, "hidden_size": 80, "intermediate_size": 136,
    "num_hidden_layers": 2, "num_attention_heads": 5, "num_key_value_heads": 5, "head_dim": 48,
    "rms_norm_eps": 2e-5, "rope_theta": 500000.0, "max_position_embeddings": 512,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 64},
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "eos_token_id": 2,
}

TINY_W = {   # Qwen2 style with a sliding window in the upper layers
    "architectures": ["Qwen2ForCausalLM"], "vocab_size": 200, "hidden_size": 48, "intermediate_size": 80,
    "num_hidden_layers": 3, "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 16,
    "rms_norm_eps": 1e-6, "rope_theta": 10000.0, "max_position_embeddings": 4096,
    "use_sliding_window": True, "sliding_window": 70, "max_window_layers": 1,
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "eos_token_id": 199,
}

TINY_D = {   # Llama style with head size 64 and window: the matrix-core attention path
    "architectures": ["LlamaForCausalLM"], "vocab_size": 300, "hidden_size": 120, "intermediate_size": 200,
    "num_hidden_layers": 2, "num_attention_heads": 6, "num_key_value_heads": 2, "head_dim": 64,
    "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "max_position_embeddings": 4096,
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "eos_token_id": 1,
}

TINY_WD = {  # Qwen2 style with head size 64 and a sliding window in the upper layer: the matrix-core attention
             # over page tables with pages that were given back
    "architectures": ["Qwen2ForCausalLM"], "vocab_size": 211, "hidden_size": 128, "intermediate_size": 152,
    "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 64,
    "rms_norm_eps": 1e-6, "rope_theta": 10000.0, "max_position_embeddings": 4096,
    "use_sliding_window": True, "sliding_window": 70, "max_window_layers": 1,
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "eos_token_id": 210,
}

LAYER_8B = {   # two layers of the Llama-3.1-8B layer sizes with a small vocabulary: the kernels at real widths
    "architectures": ["LlamaForCausalLM"], "vocab_size": 1031, "hidden_size": 4096, "intermediate_size": 14336,
    "num_hidden_layers": 2, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
    "rms_norm_eps": 1e-5, "rope_theta": 500000.0, "max_position_embeddings": 131072,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "eos_token_id": 2,
}

LAYER_14B = {  # one layer of the Qwen3-14B layer sizes: widths that are no power of two, five query heads per kv head
    "architectures": ["Qwen3ForCausalLM"], "vocab_size": 1033, "hidden_size": 5120, "intermediate_size": 17408,
    "num_hidden_layers": 1, "num_attention_heads": 40, "num_key_value_heads": 8, "head_dim": 128,
    "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "max_position_embeddings": 40960,
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "eos_token_id": 2,
}

ALL = {"tiny_wd": TINY_WD, "tiny_a": TINY_A, "tiny_b": TINY_B, "tiny_c": TINY_C, "tiny_w": TINY_W, "tiny_d": TINY_D, "layer_8b": LAYER_8B, "layer_14b": LAYER_14B}
