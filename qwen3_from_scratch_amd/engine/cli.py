"""Command line: generate from a model folder, or make one with random weights.

    python -m qwen3_from_scratch_amd --config_path engine.yaml --model qwen3-0.6b --prompt "..." [--chat]
    python -m qwen3_from_scratch_amd --path DIR --prompt_ids 5,17,3 --max_new_tokens 16 --temperature 0
    python -m qwen3_from_scratch_amd --write_random DIR --from_config config.json --seed 1

`--config_path` and `--model` are the reference's flags (examples/server.py:59-70);
the other options carry the names of its YAML keys
(src/qwen3_from_scratch/factory/batch_config.py:83-149).
"""

import argparse
import json
import sys


def main(argv=None):
    p = argparse.ArgumentParser(prog="qwen3_from_scratch_amd", description=__doc__.split("\n\n")[0])
    p.add_argument("--config_path", help="engine YAML in the reference's layout")
    p.add_argument("--model", help="name of the model entry in the YAML")
    p.add_argument("--path", help="model folder (config.json + model.safetensors), instead of a YAML")
    p.add_argument("--dtype", default=None, help="bfloat16 (default) or float32")
    p.add_argument("--device", default=None)
    p.add_argument("--max_len", type=int, default=None)
    p.add_argument("--prompt", action="append", default=[], help="text prompt (needs a tokenizer); repeatable")
    p.add_argument("--prompt_ids", action="append", default=[], help="comma-separated token ids; repeatable")
    p.add_argument("--chat", action="store_true",
                   help="each --prompt is a user's message: the tokenizer's chat template is applied, with the "
                        "opening of the assistant's turn (as the reference's examples send their prompts)")
    p.add_argument("--max_new_tokens", type=int, default=None)
    p.add_argument("--temperature", type=float, default=None)
    p.add_argument("--top_k", type=int, default=None)
    p.add_argument("--seed", type=int, default=0, help="sampling seed, and the seed of --write_random")
    p.add_argument("--ignore_eos", action="store_true")
    p.add_argument("--eos_id", type=int, action="append", default=[], metavar="TOKEN",
                   help="a token that ends a request, beside those the model folder names; repeatable")
    p.add_argument("--component", action="append", default=[], metavar="SLOT=NAME",
                   help="another registered implementation for a kind of part (the YAML's `components`), e.g. "
                        "mlp=my_feed_forward; repeatable")
    p.add_argument("--kv_cache_dtype", default=None, help="must equal --dtype: the cache is kept in the compute dtype")
    p.add_argument("--max_num_seqs", type=int, default=None)
    p.add_argument("--max_num_tokens", type=int, default=None)
    p.add_argument("--block_size", type=int, default=None)
    p.add_argument("--num_blocks", type=int, default=None)
    p.add_argument("--gpu_utilization", type=float, default=None)
    p.add_argument("--chunked_prefill_size", type=int, default=None)
    p.add_argument("--enable_prefix_cache", type=lambda v: str(v).lower() in ("1", "true", "yes", "on"), default=None,
                   metavar="BOOL", help="requests take over cached blocks of a prefix they share (default true)")
    p.add_argument("--tiled_weights", type=lambda v: str(v).lower() in ("1", "true", "yes", "on"), default=None,
                   metavar="BOOL", help="keep the second, tile-ordered copy of the matrices (default true: faster "
                                        "decoding, twice the memory)")
    p.add_argument("--log_interval", type=int, default=0)
    p.add_argument("--write_random", metavar="DIR", help="write a random-weights model folder and exit")
    p.add_argument("--from_config", metavar="JSON", help="config.json for --write_random")
    p.add_argument("--std", type=float, default=0.02)
    p.add_argument("--norm_jitter", type=float, default=0.1)
    args = p.parse_args(argv)

    if args.write_random:
        if not args.from_config:
            p.error("--write_random needs --from_config")
        from ..config.registry import lookup_architecture
        from ..weights import write_random_model

        with open(args.from_config) as fh:
            data = json.load(fh)
        config_class, _ = lookup_architecture(data["architectures"][0])
        write_random_model(args.write_random, config_class.from_dict(data), seed=args.seed, std=args.std,
                           norm_jitter=args.norm_jitter)
        print("wrote %s" % args.write_random)
        return 0

    from .sync_engine import SyncEngine

    overrides = {k: getattr(args, k) for k in (
        "dtype", "device", "max_len", "max_num_seqs", "max_num_tokens", "block_size", "num_blocks",
        "gpu_utilization", "chunked_prefill_size", "enable_prefix_cache", "tiled_weights")
        if getattr(args, k) is not None}
    overrides["seed"] = args.seed
    if args.eos_id:
        overrides["eos_ids"] = tuple(args.eos_id)
    if args.kv_cache_dtype is not None:
        overrides["kv_cache_dtype"] = args.kv_cache_dtype
    if args.component:
        overrides["components"] = {}
        for item in args.component:
            slot, _, name = item.partition("=")
            if not slot or not name:
                p.error("--component takes SLOT=NAME, found %r" % item)
            overrides["components"][slot] = name
    if args.config_path:
        if not args.model:
            p.error("--config_path needs --model")
        engine = SyncEngine(args.config_path, args.model, log_interval=args.log_interval, **overrides)
    elif args.path:
        engine = SyncEngine(path=args.path, log_interval=args.log_interval, **overrides)
    else:
        p.error("give --config_path and --model, or --path")
    texts = [[{"role": "user", "content": t}] for t in args.prompt] if args.chat else list(args.prompt)
    prompts = texts + [[int(t) for t in s.split(",") if t.strip()] for s in args.prompt_ids]
    if not prompts:
        p.error("give --prompt or --prompt_ids")
    sampling = {}
    if args.temperature is not None:
        sampling["temperature"] = args.temperature
    if args.top_k is not None:
        sampling["top_k"] = args.top_k
    sampling["ignore_eos"] = args.ignore_eos
    if len(prompts) == 1:
        chunk = None
        ids = []
        for chunk in engine.generate_stream(prompts[0], args.max_new_tokens, **sampling):
            ids.append(chunk.token_id)
            if engine.tokenizer is not None:
                print(chunk.delta, end="", flush=True)
        if engine.tokenizer is None:
            print(" ".join(map(str, ids)))
        else:
            print()
        if chunk is not None:
            m = chunk.metrics
            print("TTFT: %.4fs | tokens: %d | TPS: %.2f | total: %.4fs"
                  % (m.ttft, m.token_count, m.tps, m.total_elapsed), file=sys.stderr)
    else:
        texts, batch = engine.batch_generate(prompts, args.max_new_tokens, **sampling)
        for t in texts:
            print(t)
        print("requests: %d | tokens: %d | total: %.4fs | throughput: %.2f tokens/s"
              % (batch.num_requests, batch.total_tokens, batch.total_elapsed, batch.aggregate_tps),
              file=sys.stderr)
    return 0
