"""Tiny configurations of the architecture for the tests.  A and B differ in
every size and option; C adds sizes that are awkward for tiled kernels; D and E
have the head sizes (64, 128) and widths (multiples of 64) that the matrix-core
kernels of the bfloat16 path take, so the schedules run through those too."""

TINY_A = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 16, "intermediate_size": 160, "vocab_size": 256, "rope_theta": 10000.0,
    "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "use_sliding_window": False,
    "max_position_embeddings": 128,
}
TINY_A_PAGE = 16

TINY_B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
    "head_dim": 32, "intermediate_size": 224, "vocab_size": 320, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "use_sliding_window": True,
    "sliding_window": 32, "max_window_layers": 1, "max_position_embeddings": 256,
    "eos_token_id": [7, 9],
}
TINY_B_PAGE = 8

# head size 48 (a step of 16 that is no power of two), 5 heads in one group, odd widths
TINY_C = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 120, "num_attention_heads": 5, "num_key_value_heads": 5,
    "head_dim": 48, "intermediate_size": 200, "vocab_size": 301, "rope_theta": 50000.0,
    "rms_norm_eps": 1e-4, "tie_word_embeddings": False, "use_sliding_window": True,
    "sliding_window": 20, "max_window_layers": 0, "max_position_embeddings": 512,
}
TINY_C_PAGE = 16

# head size 64, three query heads a kv head, a window on the second layer
TINY_D = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 128, "num_attention_heads": 6, "num_key_value_heads": 2,
    "head_dim": 64, "intermediate_size": 256, "vocab_size": 400, "rope_theta": 10000.0,
    "rms_norm_eps": 1e-6, "tie_word_embeddings": False, "use_sliding_window": True,
    "sliding_window": 48, "max_window_layers": 1, "max_position_embeddings": 256,
}
TINY_D_PAGE = 16

# head size 128, seven query heads on one kv head, an inner width long enough for a product cut along K
TINY_E = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 2, "hidden_size": 256, "num_attention_heads": 7, "num_key_value_heads": 1,
    "head_dim": 128, "intermediate_size": 1024, "vocab_size": 500, "rope_theta": 1000000.0,
    "rms_norm_eps": 1e-5, "tie_word_embeddings": True, "use_sliding_window": False,
    "max_position_embeddings": 256,
}
TINY_E_PAGE = 32
