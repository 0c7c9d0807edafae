"""Two tiny Llama configurations that differ in every size and option."""

TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "intermediate_size": 176, "vocab_size": 256, "rope_theta": 10000.0, "rope_scaling": None,
    "tie_word_embeddings": False, "rms_norm_eps": 1e-5, "max_position_embeddings": 256,
}

TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
    "intermediate_size": 256, "vocab_size": 512, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 64},
    "tie_word_embeddings": True, "rms_norm_eps": 1e-6, "max_position_embeddings": 128,
}

# head_dim not equal to hidden / heads, 48 wide (no power of two), five heads in groups of five.
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 1, "hidden_size": 80, "num_attention_heads": 5, "num_key_value_heads": 1, "head_dim": 48,
    "intermediate_size": 100, "vocab_size": 131, "rope_theta": 1000.0,
    "tie_word_embeddings": False, "rms_norm_eps": 1e-4, "max_position_embeddings": 300,
}
