"""The two tiny GPT-2 configurations that the tests use. They differ in every size and option."""

TINY_A = {
    "model_type": "gpt2",
    "n_layer": 2,
    "n_embd": 64,
    "n_head": 4,
    "n_inner": None,
    "vocab_size": 512,
    "n_positions": 128,
    "layer_norm_epsilon": 1e-5,
    "activation_function": "gelu_new",
    "scale_attn_by_inverse_layer_idx": False,
    "reorder_and_upcast_attn": False,
    "initializer_range": 0.02,
    "tie_word_embeddings": True,
}

TINY_B = {
    "model_type": "gpt2",
    "n_layer": 3,
    "n_embd": 96,
    "n_head": 3,
    "n_inner": 320,
    "vocab_size": 1000,
    "n_positions": 256,
    "layer_norm_epsilon": 1e-6,
    "activation_function": "gelu",
    "scale_attn_by_inverse_layer_idx": True,
    "reorder_and_upcast_attn": True,
    "initializer_range": 0.02,
    "tie_word_embeddings": True,
}

TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1)}
