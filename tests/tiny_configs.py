"""The tiny GPT-2 configurations that the tests use. A and B differ in every size and option; C has sizes that are
no power of two anywhere (a head size of 112, two heads, an inner width of 100, a vocabulary of 257)."""

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

TINY_C = {
    "model_type": "gpt2",
    "n_layer": 2,
    "n_embd": 224,
    "n_head": 2,
    "n_inner": 100,
    "vocab_size": 257,
    "n_positions": 130,
    "layer_norm_epsilon": 1e-3,
    "activation_function": "silu",
    "scale_attn_by_inverse_layer_idx": True,
    "reorder_and_upcast_attn": False,
    "initializer_range": 0.02,
    "tie_word_embeddings": True,
}

TINY = {"A": (TINY_A, 0), "B": (TINY_B, 1), "C": (TINY_C, 2)}
