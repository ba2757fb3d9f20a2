"""The command line: writing a random-weights model folder and generating from it."""

import json

import pytest

from helpers import TINY
from qwen3_from_scratch_amd.engine import cli


def test_write_random_then_generate(cpu_ops, tmp_path, capsys):
    cfg = tmp_path / "cfg.json"
    cfg.write_text(json.dumps(TINY["A"]["config"]))
    model = tmp_path / "model"
    assert cli.main(["--write_random", str(model), "--from_config", str(cfg), "--seed", "4"]) == 0
    assert (model / "config.json").exists() and (model / "model.safetensors").exists()
    capsys.readouterr()
    args = ["--path", str(model), "--device", "cpu", "--dtype", "float32", "--num_blocks", "16",
            "--max_new_tokens", "5", "--temperature", "0", "--ignore_eos"]
    assert cli.main(args + ["--prompt_ids", "5,17,3"]) == 0
    one = capsys.readouterr().out.split()
    assert len(one) == 5 and all(t.isdigit() for t in one)
    assert cli.main(args + ["--prompt_ids", "5,17,3", "--prompt_ids", "9,9"]) == 0
    lines = capsys.readouterr().out.strip().split("\n")
    assert len(lines) == 2 and lines[0].split() == one


def test_yaml_entry(cpu_ops, tmp_path, model_folders, capsys):
    text = "generation:\n  temperature: 0\n  max_new_tokens: 3\nmodels:\n  - name: tiny\n    path: %s\n    dtype: float32\n    device: cpu\nscheduler:\n  num_blocks: 8\n" % model_folders["A"]
    (tmp_path / "e.yaml").write_text(text)
    assert cli.main(["--config_path", str(tmp_path / "e.yaml"), "--model", "tiny", "--prompt_ids", "1,2,3",
                     "--ignore_eos"]) == 0
    assert len(capsys.readouterr().out.split()) == 3
    with pytest.raises(SystemExit):
        cli.main(["--prompt_ids", "1"])
