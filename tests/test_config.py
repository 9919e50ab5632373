import json
import os

import pytest

from levanter_amd.config import ConfigError, Gpt2Config, InferenceEngineConfig, LmConfig
from tiny_configs import TINY_A, TINY_B


def test_registry_maps_name_to_config_and_lists_known_on_error():
    assert LmConfig.get_choice_class("gpt2") is Gpt2Config
    assert "gpt2" in LmConfig.known_architectures()
    with pytest.raises(ConfigError, match="unknown model_type 'llama'.*gpt2"):
        LmConfig.from_dict({"model_type": "llama"})
    with pytest.raises(ConfigError, match="model_type"):
        LmConfig.from_dict({"n_embd": 8})


def test_gpt2_reads_its_config_json_keys_and_derives_sizes():
    a = LmConfig.from_dict(TINY_A)
    assert (a.n_layer, a.n_embd, a.n_head, a.head_dim, a.inner_dim, a.vocab_size, a.n_positions) == (2, 64, 4, 16, 256, 512, 128)
    assert a.activation_function == "gelu_new" and a.layer_norm_epsilon == 1e-5
    b = LmConfig.from_dict(TINY_B)
    assert (b.n_layer, b.n_embd, b.n_head, b.head_dim, b.inner_dim) == (3, 96, 3, 32, 320)
    assert b.scale_attn_by_inverse_layer_idx and b.reorder_and_upcast_attn and b.layer_norm_epsilon == 1e-6
    # keys of other tools in config.json are ignored; defaults are the reference's (gpt2.py:37-55)
    c = LmConfig.from_dict({"model_type": "gpt2", "vocab_size": 50257, "n_positions": 1024, "n_embd": 768, "n_layer": 12,
                            "n_head": 12, "torch_dtype": "float32", "task_specific_params": {}})
    assert c.activation_function == "gelu_new" and c.inner_dim == 3072 and not c.scale_attn_by_inverse_layer_idx


def test_round_trip_through_a_folder(tmp_path):
    b = LmConfig.from_dict(TINY_B)
    b.save(str(tmp_path))
    raw = json.load(open(os.path.join(tmp_path, "config.json")))
    assert raw["model_type"] == "gpt2" and raw["n_inner"] == 320
    assert LmConfig.load(str(tmp_path)) == b
    with pytest.raises(ConfigError, match="no config.json"):
        LmConfig.load(str(tmp_path / "nowhere"))


@pytest.mark.parametrize("patch,match", [
    ({"n_head": 5}, "not divisible"),
    ({"activation_function": "gelu_fast"}, "unknown activation_function"),
    ({"tie_word_embeddings": False}, "tie_word_embeddings"),
    ({"n_layer": 0}, "positive integer"),
    ({"layer_norm_epsilon": 0.0}, "layer_norm_epsilon"),
    ({"n_inner": -4}, "n_inner"),
    ({"scale_attn_weights": False}, "scale_attn_weights"),
])
def test_bad_configs_are_refused(patch, match):
    with pytest.raises(ConfigError, match=match):
        LmConfig.from_dict({**TINY_A, **patch})
    raw = dict(TINY_A)
    del raw["n_embd"]
    with pytest.raises(ConfigError, match="lacks the key 'n_embd'"):
        LmConfig.from_dict(raw)


def test_model_spec_holds_every_size_from_the_config():
    spec = LmConfig.from_dict(TINY_B).model_spec()
    assert len(spec.layers) == 3 and [e.layer for e in spec.plan] == [0, 1, 2]
    m = spec.layers[2].mixer
    assert m.kind == "causal_self_attention" and m.params["n_heads"] == 3 and m.params["head_dim"] == 32
    assert abs(m.params["scale"] - 1 / (32 ** 0.5) / 3.0) < 1e-12  # layer index 2: q / 3 (gpt2.py:192-193)
    assert spec.layers[0].feed_forward.params["inner_dim"] == 320 and spec.layers[0].feed_forward.params["activation"] == "gelu"
    t = spec.all_tensors()
    assert t["h.1.attn.c_attn.weight"].shape == (96, 288) and t["h.1.mlp.c_fc.weight"].shape == (96, 320)
    assert t["wte.weight"].shape == (1000, 96) and t["wpe.weight"].shape == (256, 96)
    assert "lm_head.weight" not in t and len(t) == 2 + 3 * 12 + 2
    a = LmConfig.from_dict(TINY_A).model_spec()
    assert abs(a.layers[1].mixer.params["scale"] - 0.25) < 1e-12  # no layer scale: 1 / sqrt(16)


def test_engine_config_defaults_and_checks():
    c = InferenceEngineConfig()
    assert c.max_seqs == 16 and c.max_pages_per_seq == 64 and c.imputed_max_pages == 16 * 64
    assert c.imputed_max_tokens_per_round == 16 and c.imputed_max_prefill_size == min(16 * 64, 2048)
    with pytest.raises(ConfigError, match="page_size"):
        InferenceEngineConfig(page_size=24)
    with pytest.raises(ConfigError, match="compute_dtype"):
        InferenceEngineConfig(compute_dtype="float16")
