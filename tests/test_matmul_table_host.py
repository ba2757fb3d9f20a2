"""The table of kernel choices and the program that makes it, without a GPU: what the tuner
finds is stubbed; the entry format, the merge with an existing table and the shipped file's
well-formedness are checked."""

import json

from qwen3_from_scratch_amd import ops
from qwen3_from_scratch_amd.ops import tune


def test_an_entry_names_the_library_candidate_or_the_tile_shape():
    own = tune._entry("plain", 64, 4096, 12288, "bfloat16", dict(own=5, splits=8, library=0, us=29.04))
    assert own == {"kind": "plain", "rows": 64, "N": 4096, "K": 12288, "out": "bfloat16", "own": 5, "splits": 8,
                   "us": 29.0}
    lib = tune._entry("scaled", 24, 6144, 4096, "bfloat16", dict(own=-1, splits=1, library=3))
    assert lib == {"kind": "scaled", "rows": 24, "N": 6144, "K": 4096, "out": "bfloat16", "library": 3, "us": 0.0}


def test_merge_keeps_old_sizes_and_replaces_the_ones_tuned_again(tmp_path, monkeypatch, capsys):
    old = {"note": "x", "entries": [
        {"kind": "plain", "rows": 64, "N": 4096, "K": 4096, "out": "bfloat16", "library": 2, "us": 15.0},
        {"kind": "plain", "rows": 2048, "N": 4096, "K": 4096, "out": "bfloat16", "library": 1, "us": 61.0},
        {"kind": "plain", "rows": 64, "N": 4096, "K": 4096, "library": 7, "out": "float32", "us": 16.0}]}
    path = tmp_path / "table.json"
    path.write_text(json.dumps(old))
    asked = {}

    def found(hidden, heads, kv_heads, head_dim, intermediate, rows, vocab=0, only_head=False):
        asked.update(hidden=hidden, rows=rows, vocab=vocab, only_head=only_head)
        return [tune._entry("plain", 64, 4096, 4096, "bfloat16", dict(own=3, splits=4, library=0, us=13.0)),
                tune._entry("residual", 24, 4096, 12288, "bfloat16", dict(own=0, splits=8, library=0))]

    monkeypatch.setattr(tune, "tune_layer", found)
    tune.main(["--hidden", "4096", "--heads", "32", "--kv-heads", "8", "--head-dim", "128", "--intermediate", "12288",
               "--rows", "24,64", "--merge", str(path)])
    table = json.loads(capsys.readouterr().out)
    assert asked == dict(hidden=4096, rows=[24, 64], vocab=0, only_head=False)
    by_key = {(e["kind"], e["rows"], e["N"], e["K"], e["out"]): e for e in table["entries"]}
    assert len(by_key) == len(table["entries"]) == 4
    assert by_key[("plain", 64, 4096, 4096, "bfloat16")]["own"] == 3                    # tuned again: replaced
    assert "library" not in by_key[("plain", 64, 4096, 4096, "bfloat16")]
    assert by_key[("plain", 2048, 4096, 4096, "bfloat16")]["library"] == 1              # kept
    assert by_key[("plain", 64, 4096, 4096, "float32")]["library"] == 7                 # another output type: kept
    assert by_key[("residual", 24, 4096, 12288, "bfloat16")]["splits"] == 8             # new


def test_the_shipped_table_is_well_formed():
    with open(ops.TABLE_FILE, encoding="utf-8") as fh:
        table = json.load(fh)
    seen = set()
    for e in table["entries"]:
        key = (e["kind"], e["rows"], e["N"], e["K"], e.get("out", "bfloat16"))
        assert key not in seen, key
        seen.add(key)
        assert e["kind"] in ops._KINDS and e.get("out", "bfloat16") in ("bfloat16", "float32")
        assert ("own" in e) != ("library" in e), key
        assert 1 <= e.get("splits", 1) <= 64 and e["N"] > 0 and e["K"] > 0
        # rows are filed as the launcher rounds them: in steps of 8 up to 64 rows and for the
        # products that carry a norm, in steps of 32 beyond
        step = 8 if (e["kind"] != "plain" or e["rows"] <= 64) else 32
        assert e["rows"] > 16 and e["rows"] % step == 0, key
        if e["kind"] != "plain":
            assert e["rows"] <= ops.FUSED_ROWS_MOST
