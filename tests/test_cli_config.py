import pytest

from levanter_amd.config import ConfigError
from levanter_amd.config.cli import parse_config, parse_overrides
from levanter_amd.main.sample_lm import SampleLmConfig, _compute_dtype, main


def test_overrides_and_yaml(tmp_path):
    (tmp_path / "s.yaml").write_text(
        "hf_checkpoint: /models/x\ntrainer:\n  mp: p=bfloat16,c=bfloat16\nmax_new_tokens: 32\n"
        "engine:\n  max_pages: 256\n  max_seqs: 8\n  page_size: 16\n  max_rounds: 16\nprompts:\n  - a\n  - b\n")
    c = parse_config(SampleLmConfig, ["--config_path", str(tmp_path / "s.yaml"), "--engine.max_seqs", "4", "--temperature=0",
                                      "--prompt_ids", "[[1, 2], [3]]", "--profile"])
    assert c.hf_checkpoint == "/models/x" and c.max_new_tokens == 32 and c.temperature == 0 and c.profile is True
    assert c.engine.max_pages == 256 and c.engine.max_seqs == 4 and c.engine.page_size == 16 and c.engine.max_rounds == 16
    assert c.prompts == ["a", "b"] and c.prompt_ids == [[1, 2], [3]]
    assert _compute_dtype(c) == "bfloat16"
    # the reference's defaults (src/levanter/main/sample_lm.py:52-58)
    d = SampleLmConfig()
    assert (d.max_new_tokens, d.temperature, d.seed, d.n_generations, d.n_rounds, d.stop_sequence) == (192, 0.7, 2, 1, 4, ".")
    assert parse_overrides(["--a.b", "1", "--a.c", "x", "y"]) == {"a": {"b": 1, "c": ["x", "y"]}}


def test_unknown_options_and_bad_values():
    with pytest.raises(ConfigError, match="unknown option.*engine.pages"):
        parse_config(SampleLmConfig, ["--engine.pages", "3"])
    with pytest.raises(ConfigError, match="page_size"):
        parse_config(SampleLmConfig, ["--engine.page_size", "24"])
    with pytest.raises(ConfigError, match="exactly one"):
        main(SampleLmConfig())
    with pytest.raises(ConfigError, match="checkpoint_path"):
        main(SampleLmConfig(checkpoint_path="x"))


def test_help_lists_every_option_with_its_default(capsys):
    with pytest.raises(SystemExit) as e:
        parse_config(SampleLmConfig, ["--help"])
    assert e.value.code == 0
    out = capsys.readouterr().out
    for line in ("--hf_checkpoint (Optional[str]; default None)", "--engine.max_seqs (int; default 16)", "--engine.page_size (int; default 16)",
                 "--trainer.mp (Optional[str]; default None)", "--max_new_tokens (int; default 192)", "--temperature (float; default 0.7)",
                 "--n_rounds (int; default 4)", "--profile (bool; default False)"):
        assert line in out, line
