import json
import os
import struct

import pytest
import torch

from helpers import read_weights, write_model
from levanter_amd.config import LmConfig
from levanter_amd.weights import SafetensorsError, WeightsError, load_tensors, random_tensors, save_file
from tiny_configs import TINY_A, TINY_B


def test_random_model_folder_round_trip_and_foreign_reader():
    d = write_model(TINY_B, 1, torch.bfloat16)
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    spec = LmConfig.load(d).model_spec()
    mine = load_tensors(d, spec)
    theirs = read_weights(d, torch.float32)  # the safetensors package reads what our writer wrote
    assert set(mine) == set(theirs) == set(spec.all_tensors())
    for k in mine:
        assert mine[k].dtype == torch.bfloat16  # stored bfloat16 stays bfloat16
        assert torch.equal(mine[k].float(), theirs[k])
    # seeded: same seed, same tensors; norm weights around one, the rest around zero with the configured std
    again = random_tensors(spec, 1, torch.bfloat16)
    assert all(torch.equal(again[k], mine[k]) for k in mine)
    other = random_tensors(spec, 2, torch.bfloat16)
    assert not torch.equal(other["wte.weight"], mine["wte.weight"])
    assert abs(float(mine["h.0.ln_1.weight"].float().mean()) - 1.0) < 0.02
    assert abs(float(mine["wte.weight"].float().std()) - 0.02) < 0.002


def test_float32_stays_float32_and_prefix_is_dropped(tmp_path):
    d = write_model(TINY_A, 0, torch.float32)
    spec = LmConfig.load(d).model_spec()
    t = load_tensors(d, spec)
    assert all(v.dtype == torch.float32 for v in t.values())
    # the optional "transformer." prefix (gpt2.py:80) and the ignorable buffers of GPT-2 checkpoints
    pre = {"transformer." + k: v for k, v in t.items()}
    pre["transformer.h.0.attn.bias"] = torch.ones(1, 1, 8, 8)
    pre["lm_head.weight"] = t["wte.weight"].clone()
    LmConfig.load(d).save(str(tmp_path))
    save_file(pre, str(tmp_path / "model.safetensors"))
    t2 = load_tensors(str(tmp_path), spec)
    assert all(torch.equal(t2[k], t[k]) for k in t)


def test_a_stored_head_must_be_the_token_table(tmp_path):
    """GPT-2's head is its token table (src/levanter/models/gpt2.py:361-362). A checkpoint may carry ``lm_head.weight``
    as a copy; one that differs (an untied fine-tune) would give other logits than its author's and is refused."""
    d = write_model(TINY_A, 0, torch.float32)
    spec = LmConfig.load(d).model_spec()
    t = load_tensors(d, spec)
    LmConfig.load(d).save(str(tmp_path))
    save_file({**t, "lm_head.weight": t["wte.weight"].clone()}, str(tmp_path / "model.safetensors"))
    t2 = load_tensors(str(tmp_path), spec)
    assert sorted(t2) == sorted(t) and torch.equal(t2["wte.weight"], t["wte.weight"])
    other = t["wte.weight"].clone()
    other[3, 5] += 1e-3
    save_file({**t, "lm_head.weight": other}, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightsError, match="lm_head.weight is not equal to wte.weight") as e:
        load_tensors(str(tmp_path), spec)
    assert e.value.differing_copies and not e.value.unexpected
    save_file({**t, "lm_head.weight": other[:-1]}, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightsError, match=r"lm_head.weight: file has \[511, 64\]"):
        load_tensors(str(tmp_path), spec)


def test_one_error_lists_missing_unexpected_and_misshapen(tmp_path):
    d = write_model(TINY_A, 0, torch.float32)
    spec = LmConfig.load(d).model_spec()
    t = load_tensors(d, spec)
    del t["h.1.mlp.c_fc.bias"]
    del t["ln_f.weight"]
    t["h.0.attn.rotary.inv_freq"] = torch.zeros(4)
    t["h.0.mlp.c_fc.weight"] = torch.zeros(64, 320)  # n_inner of the file is not the configuration's
    t["wpe.weight"] = torch.zeros(128, 64, dtype=torch.int32)
    LmConfig.load(d).save(str(tmp_path))
    save_file(t, str(tmp_path / "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        load_tensors(str(tmp_path), spec)
    msg = str(e.value)
    assert "missing tensors (2): h.1.mlp.c_fc.bias, ln_f.weight" in msg
    assert "unexpected tensors (1): h.0.attn.rotary.inv_freq" in msg
    assert "h.0.mlp.c_fc.weight: file has [64, 320], the configuration needs [64, 256]" in msg
    assert "wpe.weight" in msg and "wrong dtypes" in msg
    assert e.value.missing == ["h.1.mlp.c_fc.bias", "ln_f.weight"]


def test_missing_and_truncated_files(tmp_path):
    spec = LmConfig.from_dict(TINY_A).model_spec()
    with pytest.raises(FileNotFoundError, match="model.safetensors"):
        load_tensors(str(tmp_path), spec)
    d = write_model(TINY_A, 0, torch.float32)
    blob = open(os.path.join(d, "model.safetensors"), "rb").read()
    (tmp_path / "model.safetensors").write_bytes(blob[: len(blob) // 2])
    with pytest.raises(SafetensorsError, match="truncated"):
        load_tensors(str(tmp_path), spec)
    (tmp_path / "model.safetensors").write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="truncated"):
        load_tensors(str(tmp_path), spec)
    (tmp_path / "model.safetensors").write_bytes(struct.pack("<Q", 4) + b"nope")
    with pytest.raises(SafetensorsError, match="not JSON"):
        load_tensors(str(tmp_path), spec)


def test_sharded_checkpoint_with_index(tmp_path):
    d = write_model(TINY_A, 0, torch.float32)
    spec = LmConfig.load(d).model_spec()
    t = load_tensors(d, spec)
    names = sorted(t)
    half = len(names) // 2
    shards = {"model-00001-of-00002.safetensors": names[:half], "model-00002-of-00002.safetensors": names[half:]}
    weight_map = {}
    for fn, ks in shards.items():
        save_file({k: t[k] for k in ks}, str(tmp_path / fn))
        weight_map.update({k: fn for k in ks})
    json.dump({"metadata": {}, "weight_map": weight_map}, open(tmp_path / "model.safetensors.index.json", "w"))
    t2 = load_tensors(str(tmp_path), spec)
    assert all(torch.equal(t2[k], t[k]) for k in t)
    os.remove(tmp_path / "model-00002-of-00002.safetensors")
    with pytest.raises(FileNotFoundError, match="shards"):
        load_tensors(str(tmp_path), spec)
