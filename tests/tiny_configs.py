"""Small Llama configurations for the tests. A and B are two tiny shapes that
differ in every size and option; C has an explicit head_dim that is not
hidden/heads, a width, a feed-forward and a vocabulary that are no power of
two, and untied weights with scaling of the other type key ("type")."""
import copy

TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 8,
    "num_key_value_heads": 2, "intermediate_size": 176, "vocab_size": 256,
    "rope_theta": 10000.0, "rope_scaling": None, "rms_norm_eps": 1e-5,
    "tie_word_embeddings": True, "torch_dtype": "float32", "hidden_act": "silu",
    "max_position_embeddings": 2048,
}

TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 3, "hidden_size": 128, "num_attention_heads": 4,
    "num_key_value_heads": 1, "intermediate_size": 320, "vocab_size": 384,
    "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 64},
    "max_position_embeddings": 512, "rms_norm_eps": 1e-6,
    "tie_word_embeddings": False, "torch_dtype": "float32", "hidden_act": "silu",
}

TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 1, "hidden_size": 96, "num_attention_heads": 6,
    "num_key_value_heads": 3, "head_dim": 64, "intermediate_size": 200, "vocab_size": 300,
    "rope_theta": 1000.0,
    "rope_scaling": {"type": "llama3", "factor": 4.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 2.0, "original_max_position_embeddings": 32},
    "max_position_embeddings": 1024, "rms_norm_eps": 1e-3,
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "hidden_act": "silu",
}

# (name, config, weight std, norm-weight std, page size)
TINY = {
    "A": (TINY_A, 0.15, 0.0, 4),
    "B": (TINY_B, 0.10, 0.1, 16),
    "C": (TINY_C, 0.12, 0.1, 8),
}


def tiny(name):
    cfg, std, norm_std, page = TINY[name]
    return copy.deepcopy(cfg), std, norm_std, page
