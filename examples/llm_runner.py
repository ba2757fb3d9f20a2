"""The asynchronous engine, in the manner of the reference's examples/llm_runner.py:

    python examples/llm_runner.py --config_path engine.yaml --model qwen3-0.6b
    python examples/llm_runner.py --path /tmp/m            # a folder without a tokenizer: token ids in and out

Two callers stream at the same time; the engine batches them.
"""

import argparse
import asyncio
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))

from qwen3_from_scratch_amd.engine import LLMEngine  # noqa: E402


async def main(args):
    options = {k: v for k, v in (("dtype", args.dtype),) if v is not None}
    if args.config_path:
        engine = LLMEngine(args.config_path, args.model, **options)
    else:
        engine = LLMEngine(path=args.path, **options)
    sampling = {} if args.temperature is None else {"temperature": args.temperature}
    try:
        await engine.warmup()
        has_text = engine.engine.tokenizer is not None
        prompts = ([[{"role": "user", "content": "介绍一下自己"}], [{"role": "user", "content": "1+1等于几"}]]
                   if has_text else [[5, 17, 3, 9], [2, 4, 6]])

        async def ask(tag, prompt):
            chunk = None
            async for chunk in engine.generate_stream(prompt, max_new_tokens=args.max_new_tokens, ignore_eos=True,
                                                      **sampling):
                print("[%s] %s" % (tag, chunk.delta if has_text else chunk.token_id), flush=True)
            return tag, chunk

        for tag, chunk in await asyncio.gather(*(ask("req%d" % i, p) for i, p in enumerate(prompts))):
            m = chunk.metrics
            print("%s: TTFT %.4fs | tokens %d | TPS %.2f | total %.4fs"
                  % (tag, m.ttft, m.token_count, m.tps, m.total_elapsed))
    finally:
        engine.close()


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
    asyncio.run(main(a))
