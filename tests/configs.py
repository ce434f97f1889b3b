"""The tiny configurations the tests use.  They differ in every size and option: number of
layers, width, heads and groups, head size (with heads x head size equal to the width or not),
feed-forward width, vocabulary, rotary base, the norms' eps, tied or separate head, page
size, the spread of the random weights, and a sliding window on some layers (C only).  D has
the widths that the matrix-core kernels take."""

TINY_A = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4,
    "num_key_value_heads": 2, "head_dim": 16, "intermediate_size": 128, "vocab_size": 256,
    "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True,
    "max_position_embeddings": 1024, "initializer_range": 0.02, "hidden_act": "silu",
}
PAGE_A = 4

TINY_B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 8,
    "num_key_value_heads": 1, "head_dim": 32, "intermediate_size": 160, "vocab_size": 384,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-5, "tie_word_embeddings": False,
    "max_position_embeddings": 2048, "initializer_range": 0.05, "hidden_act": "silu",
}
PAGE_B = 8

# no size is a power of two; 3 query heads per kv head; layers 1 and 3 slide over 24 positions
TINY_C = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 4, "hidden_size": 72, "num_attention_heads": 6,
    "num_key_value_heads": 2, "head_dim": 48, "intermediate_size": 200, "vocab_size": 331,
    "rope_theta": 50000.0, "rms_norm_eps": 3e-6, "tie_word_embeddings": False,
    "max_position_embeddings": 4096, "initializer_range": 0.04, "hidden_act": "silu",
    "sliding_window": 24, "use_sliding_window": True,
    "layer_types": ["full_attention", "sliding_attention", "full_attention", "sliding_attention"],
}
PAGE_C = 16

# widths in multiples of 128 (none a power of two but the width), which the matrix-core
# products and the norms folded into them take: decode steps go through those kernels
TINY_D = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3",
    "num_hidden_layers": 3, "hidden_size": 128, "num_attention_heads": 6,
    "num_key_value_heads": 3, "head_dim": 64, "intermediate_size": 640, "vocab_size": 300,
    "rope_theta": 300000.0, "rms_norm_eps": 2e-6, "tie_word_embeddings": True,
    "max_position_embeddings": 2048, "initializer_range": 0.03, "hidden_act": "silu",
}
PAGE_D = 16

ALL = {"A": (TINY_A, PAGE_A, 0), "B": (TINY_B, PAGE_B, 1), "C": (TINY_C, PAGE_C, 2),
       "D": (TINY_D, PAGE_D, 3)}
