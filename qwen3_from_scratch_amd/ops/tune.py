"""Make the table of kernel choices for the many-row products of a model's sizes.

    python -m qwen3_from_scratch_amd.ops.tune --hidden 4096 --heads 32 --kv-heads 8 --head-dim 128 \
        --intermediate 12288 --vocab 151936 \
        --rows 24,32,48,64,96,128,256,512,576,1024,2048 > table.json

For each row count and each of the layer's products (q/k/v, output, gate/up, down) the
tuner times the vendor library's candidates and the hand-written kernel's tile shapes on
random operands, with cold caches, and the fastest is written down as a table entry; row
counts from 17 to 128 also get entries for the products that carry a norm. The output is
the file `matmul_table.json` beside this module reads (`--merge FILE` adds to an existing
table, newer entries replacing older ones for the same size). Nothing in the engine runs
this: the table is data, made beforehand, so that every process chooses the same kernels.
"""

import argparse
import json
import sys

import torch

from .. import ops


def _entry(kind, rows, N, K, out, plan):
    e = {"kind": kind, "rows": rows, "N": N, "K": K, "out": out}
    if plan["own"] >= 0:
        e.update(own=plan["own"], splits=plan["splits"])
    else:
        e.update(library=plan["library"])
    e["us"] = round(plan.get("us", 0.0), 1)
    return e


def tune_layer(hidden, heads, kv_heads, head_dim, intermediate, rows_list, seed=0, vocab=0, only_head=False):
    device = torch.device("cuda")
    g = torch.Generator(device=device).manual_seed(seed)

    def rand(shape, scale=1.0):
        return (torch.randn(shape, generator=g, device=device) * scale).to(torch.bfloat16)

    qkv_n = (heads + 2 * kv_heads) * head_dim
    weights = {
        "qkv": rand((qkv_n, hidden), 0.02), "o": rand((hidden, heads * head_dim), 0.02),
        "gate_up": rand((2 * intermediate, hidden), 0.02), "down": rand((hidden, intermediate), 0.02),
    }
    if only_head:
        weights = {}
    if vocab:
        weights["head"] = rand((vocab, hidden), 0.02)
    norm_weight = torch.ones(hidden, dtype=torch.bfloat16, device=device)
    entries = {}
    ops.matmul_init()
    ops.matmul_tuner(True)
    try:
        for M in rows_list:
            for name, w in weights.items():
                N, K = w.shape
                x = rand((M, K))
                out_dtype = torch.float32 if name == "head" else torch.bfloat16     # logits are float32
                out_name = "float32" if name == "head" else "bfloat16"
                ops.linear(x, w, out_dtype=out_dtype)
                p = ops.matmul_plan(M, N, K, out_dtype)
                if p is not None:
                    rows = ops.matmul_rows_key("plain", M)
                    entries[("plain", rows, N, K, out_name)] = _entry(
                        "plain", rows, N, K, out_name, dict(own=p[4], splits=p[5], library=p[6], us=p[3]))
                if name != "head" and 16 < M <= ops.FUSED_ROWS_MOST and ops.fused_rows_take(w, M):
                    residual = torch.zeros((M, N), dtype=torch.float32, device=device)
                    if name in ("o", "down") and N == hidden:
                        ops.linear_residual_norm(x, w, None, residual, norm_weight)
                        kinds = ["residual"]
                    else:
                        sums = torch.ones((-(-K // 1024), ops.sums_stride(M)), dtype=torch.float32, device=device)
                        if name == "gate_up":
                            ops.linear_swiglu(x, w, unscaled=(sums, 1e-6, K))
                            kinds = ["scaled_swiglu"]
                        else:
                            ops.linear(x, w, unscaled=(sums, 1e-6, K))
                            kinds = ["scaled"]
                    for kind in kinds:
                        f = ops.matmul_fused_plan(kind, M, N, K)
                        if f is not None:
                            rows = ops.matmul_rows_key(kind, M)
                            entries[(kind, rows, N, K, "bfloat16")] = _entry(
                                kind, rows, N, K, "bfloat16", dict(own=f[0], splits=f[1], library=0))
                        # where the library serves a product that carries a norm, it is the plain product with
                        # float32 output (the division follows in a kernel of its own): that size's choice too
                        p32 = ops.matmul_plan(M, N, K, torch.float32)
                        if f is not None and f[0] < 0 and kind != "residual" and p32 is not None:
                            rows = ops.matmul_rows_key("plain", M)
                            entries[("plain", rows, N, K, "float32")] = _entry(
                                "plain", rows, N, K, "float32", dict(own=p32[4], splits=p32[5], library=p32[6], us=p32[3]))
            print("rows %d done" % M, file=sys.stderr, flush=True)
    finally:
        ops.matmul_tuner(False)
    return list(entries.values())


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--hidden", type=int, required=True)
    ap.add_argument("--heads", type=int, required=True)
    ap.add_argument("--kv-heads", type=int, required=True)
    ap.add_argument("--head-dim", type=int, required=True)
    ap.add_argument("--intermediate", type=int, required=True)
    ap.add_argument("--vocab", type=int, default=0, help="also the vocabulary product of this many columns")
    ap.add_argument("--rows", default="24,32,48,64,96,128,256,512,1024,2048")
    ap.add_argument("--only-head", action="store_true", help="the vocabulary product alone")
    ap.add_argument("--merge", default=None, help="an existing table to add to")
    args = ap.parse_args(argv)
    rows = [int(r) for r in args.rows.split(",") if r]
    entries = {}
    if args.merge:
        with open(args.merge, encoding="utf-8") as fh:
            for e in json.load(fh)["entries"]:
                entries[(e["kind"], e["rows"], e["N"], e["K"], e.get("out", "bfloat16"))] = e
    for e in tune_layer(args.hidden, args.heads, args.kv_heads, args.head_dim, args.intermediate, rows, vocab=args.vocab, only_head=args.only_head):
        entries[(e["kind"], e["rows"], e["N"], e["K"], e["out"])] = e
    ordered = [entries[k] for k in sorted(entries)]
    text = ",\n".join("  " + json.dumps(e, sort_keys=True) for e in ordered)
    print('{"note": "kernel choices for many-row products, made by python -m qwen3_from_scratch_amd.ops.tune on an '
          'MI355X; us = microseconds of the chosen kernel with cold caches", "entries": [\n%s\n]}' % text)


if __name__ == "__main__":
    main()
