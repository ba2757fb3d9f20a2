"""The in-process engine, in the manner of the reference's examples/sync_engine_example.py:
one streamed request with its metrics, one whole answer, one batch under continuous batching.

    python examples/sync_engine_example.py --config_path engine.yaml --model qwen3-0.6b
    python examples/sync_engine_example.py --path /tmp/m   # a folder without a tokenizer: token ids in and out
"""

import argparse
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

from qwen3_from_scratch_amd.engine import SyncEngine  # noqa: E402


def main(args):
    options = {k: v for k, v in (("dtype", args.dtype),) if v is not None}
    engine = (SyncEngine(args.config_path, args.model, **options) if args.config_path
              else SyncEngine(path=args.path, **options))
    sampling = {} if args.temperature is None else {"temperature": args.temperature}
    engine.warmup()
    has_text = engine.tokenizer is not None
    one = [{"role": "user", "content": "介绍一下自己"}] if has_text else [5, 17, 3, 9]
    print("=== one request, streamed ===")
    chunk = None
    for chunk in engine.generate_stream(one, max_new_tokens=args.max_new_tokens, **sampling):
        print(chunk.delta if has_text else chunk.token_id, end="" if has_text else " ", flush=True)
    m = chunk.metrics
    print("\nTTFT: %.4fs | tokens: %d | TPS: %.2f | total: %.4fs" % (m.ttft, m.token_count, m.tps, m.total_elapsed))
    print("=== one request, whole ===")
    print(engine.generate("你好" if has_text else [2, 4, 6], max_new_tokens=args.max_new_tokens, **sampling))
    print("=== a batch ===")
    prompts = ([[{"role": "user", "content": t}] for t in ("介绍一下自己", "1+1等于几", "什么是深度学习")]
               if has_text else [[5, 17, 3], [2, 4, 6, 8], [9]])
    texts, batch = engine.batch_generate(prompts, max_new_tokens=args.max_new_tokens, **sampling)
    for t in texts:
        print("- %s" % t)
    print("requests: %d | tokens: %d | total: %.4fs | throughput: %.2f tokens/s"
          % (batch.num_requests, batch.total_tokens, batch.total_elapsed, batch.aggregate_tps))
    for i, r in enumerate(batch.per_request):
        print("  req%d: TTFT %.4fs, TPS %.2f, tokens %d" % (i, r.ttft, r.tps, r.token_count))


if __name__ == "__main__":
    p = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    p.add_argument("--config_path")
    p.add_argument("--model")
    p.add_argument("--path")
    p.add_argument("--max_new_tokens", type=int, default=16)
    p.add_argument("--dtype", default=None, help="bfloat16 or float32; default: the configuration's")
    p.add_argument("--temperature", type=float, default=None, help="0 = greedy; default: the configuration's")
    a = p.parse_args()
    if not (a.path or (a.config_path and a.model)):
        p.error("give --config_path and --model, or --path")
    main(a)
