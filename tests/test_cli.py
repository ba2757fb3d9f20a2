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
    # a token named with --eos_id ends the request that produces it (the folder names none)
    args.remove("--ignore_eos")
    assert cli.main(args + ["--prompt_ids", "5,17,3", "--eos_id", "100000", "--eos_id", one[2]]) == 0
    assert capsys.readouterr().out.split() == one[:one.index(one[2]) + 1]
    with pytest.raises(Exception) as caught:
        cli.main(args + ["--prompt_ids", "5,17,3", "--component", "mlp=nothing_of_that_name"])
    assert "nothing_of_that_name" in str(caught.value)
    with pytest.raises(Exception) as caught:
        cli.main(args + ["--prompt_ids", "5,17,3", "--kv_cache_dtype", "bfloat16"])
    assert "kv_cache_dtype" in str(caught.value)


def test_yaml_entry(cpu_ops, tmp_path, model_folders, capsys):
    text = "generation:\n  temperature: 0\n  max_new_tokens: 3\nmodels:\n  - name: tiny\n    path: %s\n    dtype: float32\n    device: cpu\nscheduler:\n  num_blocks: 8\n" % model_folders["A"]
    (tmp_path / "e.yaml").write_text(text)
    assert cli.main(["--config_path", str(tmp_path / "e.yaml"), "--model", "tiny", "--prompt_ids", "1,2,3",
                     "--ignore_eos"]) == 0
    assert len(capsys.readouterr().out.split()) == 3
    with pytest.raises(SystemExit):
        cli.main(["--prompt_ids", "1"])


class _WordTokenizer:
    """A stand-in for a model folder's tokenizer (no network, no files): words are numbers."""

    eos_token_id = 7

    def __init__(self):
        self.templates = []

    def apply_chat_template(self, messages, tokenize=False, add_generation_prompt=True):
        assert tokenize is False and add_generation_prompt is True
        self.templates.append(messages)
        text = " ".join("%d %s" % (1 if m["role"] == "user" else 2, m["content"]) for m in messages)
        return text + " 2"                                # the opening of the assistant's turn

    def __call__(self, text):
        class Encoded:
            input_ids = [int(t) for t in text.split()]
        return Encoded()

    def decode(self, ids, skip_special_tokens=True):
        return "".join("<%d>" % i for i in ids)


def test_chat_messages_go_through_the_template(cpu_ops, model_folders, monkeypatch, capsys):
    """Messages (a list of role/content dicts) are turned into text by the tokenizer's chat
    template, with the assistant's turn opened, as the reference's engine does
    (src/qwen3_from_scratch/inference/sync_engine.py:238-251); a string is encoded as it is; the
    command line's --chat sends its prompts as a user's messages."""
    from qwen3_from_scratch_amd.engine import SyncEngine, sync_engine

    tokenizer = _WordTokenizer()
    monkeypatch.setattr(sync_engine, "_load_tokenizer", lambda path: tokenizer)
    engine = SyncEngine(path=model_folders["A"], dtype="float32", device="cpu", num_blocks=16, max_num_seqs=2)
    assert 7 in engine.eos_ids
    request = engine.add_request([{"role": "user", "content": "5 17 3"}])
    assert request.prompt == [1, 5, 17, 3, 2] and tokenizer.templates == [[{"role": "user", "content": "5 17 3"}]]
    engine.abort(request)
    assert engine.add_request("5 17 3").prompt == [5, 17, 3]
    while engine.scheduler.has_work():
        engine.step()
    text = engine.generate([{"role": "user", "content": "9 9"}], 4, temperature=0.0, ignore_eos=True)
    assert text.count("<") == 4
    same = engine.generate("1 9 9 2", 4, temperature=0.0, ignore_eos=True)
    assert same == text
    capsys.readouterr()
    args = ["--path", model_folders["A"], "--device", "cpu", "--dtype", "float32", "--num_blocks", "16",
            "--max_new_tokens", "4", "--temperature", "0", "--ignore_eos", "--prompt", "9 9"]
    assert cli.main(args + ["--chat"]) == 0
    assert capsys.readouterr().out.strip() == text
    assert cli.main(args) == 0
    assert capsys.readouterr().out.strip() != text
