"""Decode and prefill throughput of the Qwen3-8B-shaped model on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L]
                    [--shape 8b|14b|32b|0.6b] [--prompt P] [--context C]
                    [--workload decode|continuous|served|prefix|products]

Random bfloat16 weights, uniform-random prompts of 2,048 tokens, greedy decoding
through the engine's own step loop (scheduler, step function, sampling). A
"step" is one decode step of the whole batch. One JSON line is printed:
`value` is decoded tokens per second at the default batch; `prefill` is one
2,048-token prompt in one step (the median of three); `roofline` prices the decode step against HBM
bandwidth, the published peak and the rate a plain read kernel reaches on this GPU (`measured_peak`);
`points` holds decoding at batch 1 and 64 and a prompt of 8,192 tokens in one step (tokens a second), `points_roofline` their fractions of the published peaks. The default run is the
8B shape with prompts of 2,048 in a context of 8,192; `--shape`, `--prompt` and
`--context` move the decode measurement to the larger shapes and to longer
contexts (the prefill measurement stays at 2,048 tokens).
"""

import argparse
import json
import sys
import time

PEAK_HBM = 8.0e12            # bytes/s, MI355X HBM3E
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}   # dense MFMA peaks

QWEN3_8B = dict(architectures=["Qwen3ForCausalLM"], vocab_size=151936, hidden_size=4096, hidden_act="silu",
                num_hidden_layers=36, max_position_embeddings=40960, num_attention_heads=32,
                num_key_value_heads=8, head_dim=128, intermediate_size=12288, rms_norm_eps=1e-6,
                rope_theta=1000000.0, tie_word_embeddings=False)
QWEN3_14B = dict(QWEN3_8B, hidden_size=5120, num_hidden_layers=40, num_attention_heads=40, intermediate_size=17408)
QWEN3_32B = dict(QWEN3_8B, hidden_size=5120, num_hidden_layers=64, num_attention_heads=64, intermediate_size=25600)
# the model the reference's own measurements are of, by the sizes its configuration defaults to
# (src/qwen3_from_scratch/factory/config.py:19-42)
QWEN3_06B = dict(QWEN3_8B, hidden_size=1024, num_hidden_layers=28, num_attention_heads=16, intermediate_size=4096,
                 rms_norm_eps=1e-5, rope_theta=100000.0)
SHAPES = {"8b": ("Qwen3-8B", QWEN3_8B), "14b": ("Qwen3-14B", QWEN3_14B), "32b": ("Qwen3-32B", QWEN3_32B),
          "0.6b": ("Qwen3-0.6B", QWEN3_06B)}
PREFILL = 2048
LONG_PREFILL = 8192          # a second prompt length, reported under `points`
BLOCK = 16


def layer_params(c):
    qkv = (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim * c.hidden_size
    o = c.hidden_size * c.num_attention_heads * c.head_dim
    mlp = 3 * c.hidden_size * c.intermediate_size
    return qkv + o + mlp


def decode_bytes(c, contexts, itemsize):
    """Bytes one decode step has to read: every weight it uses once, and the
    keys and values of the live requests."""
    weights = (c.num_hidden_layers * layer_params(c) + c.vocab_size * c.hidden_size) * itemsize
    kv_per_token = 2 * c.num_hidden_layers * c.num_key_value_heads * c.head_dim * itemsize
    return weights + kv_per_token * sum(contexts)


def prefill_flops(c, tokens):
    gemm = 2.0 * tokens * c.num_hidden_layers * layer_params(c) + 2.0 * c.vocab_size * c.hidden_size
    attn = 4.0 * (tokens * (tokens + 1) / 2) * c.head_dim * c.num_attention_heads * c.num_hidden_layers
    return gemm + attn


def _model_tensors(model):
    """Every tensor a loaded model keeps on the device, each once."""
    import torch

    seen, found, stack = set(), [], [model]
    while stack:
        obj = stack.pop()
        if id(obj) in seen:
            continue
        seen.add(id(obj))
        if isinstance(obj, torch.Tensor):
            if obj.is_cuda and obj.untyped_storage().data_ptr() not in seen:
                seen.add(obj.untyped_storage().data_ptr())
                found.append(obj)
        elif isinstance(obj, (list, tuple)):
            stack.extend(obj)
        elif isinstance(obj, dict):
            stack.extend(obj.values())
        elif hasattr(obj, "__dict__") and type(obj).__module__.startswith("qwen3_from_scratch_amd"):
            stack.extend(vars(obj).values())
    return found


def continuous(args, config, model, shape_name, gen, sync):
    """64 requests admitted at once and served by continuous batching: prompt lengths uniform in
    [128, 4096], generated tokens uniform in [64, 512], prompts cut into portions of 512 beside
    the decoding requests, a budget of 576 tokens a step. Run twice; the second run (graphs
    captured, library kernels chosen) is the one reported."""
    import random

    import torch

    from qwen3_from_scratch_amd.engine import SyncEngine

    requests, portion, context = 64, 512, 8192
    rng = random.Random(0)
    sizes = [(rng.randint(128, 4096), rng.randint(64, 512)) for _ in range(requests)]
    engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=context, block_size=BLOCK,
                        num_blocks=requests * context // BLOCK // 2, max_num_seqs=requests,
                        max_num_tokens=portion + requests, chunked_prefill_size=portion,
                        enable_prefix_cache=False)         # the second pass computes every prompt again
    for _ in range(2):
        for prompt, generated in sizes:
            engine.add_request(torch.randint(0, config.vocab_size, (prompt,), generator=gen).tolist(),
                               engine.default_params(generated, temperature=0.0, ignore_eos=True))
        sync()
        t0 = time.perf_counter()
        steps = 0
        while engine.scheduler.has_work():
            engine.step()
            steps += 1
        sync()
        seconds = time.perf_counter() - t0
    tokens_in, tokens_out = sum(p for p, _ in sizes), sum(g for _, g in sizes)
    print(json.dumps({
        "metric": "continuous batching, tokens/s in and out, %s %s"
                  % (shape_name, "bf16" if args.dtype == "bfloat16" else "fp32"),
        "value": round((tokens_in + tokens_out) / seconds, 1), "unit": "tokens/s", "n_gpus": 1,
        "higher_is_better": True, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "seconds": round(seconds, 3), "steps": steps, "generated_tokens_per_s": round(tokens_out / seconds, 1),
        "config": {"model": "%s-shaped, random weights N(0, 0.02)" % shape_name, "requests": requests,
                   "prompt_tokens": tokens_in, "generated_tokens": tokens_out, "prefill_portion": portion,
                   "step_token_budget": portion + requests, "context_len": context, "kv_block_size": BLOCK,
                   "layers": config.num_hidden_layers, "sampling": "greedy"},
    }))
    return 0


def served(args, config, model, shape_name, gen, sync):
    """The load of the reference's own benchmark (docs/benchmark.md:40-68, exps/run_eval_scope_bench.sh):
    200 requests, 20 in flight at any time, 512 prompt tokens and 512 generated tokens each (end-of-sequence
    ignored), a new request admitted when one ends; without its HTTP server: requests enter and tokens leave
    through the engine's own loop. Sampling as the engine defaults to (temperature 1.0, as the reference).
    Run twice; the second run is the one reported."""
    import torch

    from qwen3_from_scratch_amd.engine import SyncEngine
    from qwen3_from_scratch_amd.engine.scheduler import RequestStatus

    number, parallel, prompt_tokens, new_tokens = 200, 20, 512, 512
    context = prompt_tokens + new_tokens
    engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=context, block_size=BLOCK,
                        num_blocks=(parallel + 1) * (context // BLOCK + 1), max_num_seqs=parallel,
                        max_num_tokens=512 + parallel, chunked_prefill_size=512, enable_prefix_cache=False)
    for _ in range(2):
        prompts = [torch.randint(0, config.vocab_size, (prompt_tokens,), generator=gen).tolist() for _ in range(number)]
        admitted, first, ended, live, queued = {}, {}, {}, {}, 0
        sync()
        t0 = time.perf_counter()
        steps = 0
        while queued < number or live:
            while queued < number and len(live) < parallel:
                request = engine.add_request(prompts[queued], engine.default_params(new_tokens, ignore_eos=True))
                admitted[request.request_id] = time.perf_counter()
                live[request.request_id] = request
                queued += 1
            engine.step()
            steps += 1
            now = time.perf_counter()
            for rid, request in list(live.items()):
                if request.generated and rid not in first:
                    first[rid] = now
                if request.status == RequestStatus.FINISHED:
                    ended[rid] = now
                    del live[rid]
        sync()
        seconds = time.perf_counter() - t0
    latency = [ended[r] - admitted[r] for r in ended]
    ttft = [first[r] - admitted[r] for r in ended]
    tpot = [(ended[r] - first[r]) / (new_tokens - 1) for r in ended]
    mean = lambda xs: sum(xs) / len(xs)
    print(json.dumps({
        "metric": "output tokens/s, %d requests, %d in flight, %d in + %d out, %s %s"
                  % (number, parallel, prompt_tokens, new_tokens, shape_name,
                     "bf16" if args.dtype == "bfloat16" else "fp32"),
        "value": round(number * new_tokens / seconds, 1), "unit": "tokens/s", "n_gpus": 1, "higher_is_better": True,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic", "seconds": round(seconds, 3),
        "steps": steps, "requests_per_s": round(number / seconds, 2), "latency_avg_s": round(mean(latency), 3),
        "ttft_avg_ms": round(1e3 * mean(ttft), 1), "tpot_avg_ms": round(1e3 * mean(tpot), 2),
        "config": {"model": "%s-shaped, random weights N(0, 0.02)" % shape_name, "requests": number,
                   "in_flight": parallel, "prompt_tokens": prompt_tokens, "generated_tokens": new_tokens,
                   "prefill_portion": 512, "kv_block_size": BLOCK, "layers": config.num_hidden_layers,
                   "sampling": "temperature 1.0", "server": "none: the engine's own loop"},
    }))
    return 0


def products(args, config, shape_name, sync):
    """The four products of a layer at 2,048, 576 and 64 rows: the kernel that the contest
    chose (library candidates and the hand-written tiled kernel, timed with cold caches) beside
    every tile shape of the hand-written kernel, microseconds with the weight coming from
    memory (as many weights in turn as exceed the last-level cache; the calls are captured in a
    graph, so the time is the GPU's)."""
    import torch

    from qwen3_from_scratch_amd import ops

    c = config
    shapes = [("qkv", (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim, c.hidden_size),
              ("o", c.hidden_size, c.num_attention_heads * c.head_dim),
              ("gate_up", 2 * c.intermediate_size, c.hidden_size), ("down", c.hidden_size, c.intermediate_size)]

    def timed(f, calls, replays=5):
        """Microseconds of one call on the GPU: `calls` of them captured in a graph (no host
        time between them), the graph replayed."""
        for _ in range(2):
            f()                                  # sizes are met, and timed, outside the capture
        sync()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for _ in range(calls):
                    f()
        torch.cuda.current_stream().wait_stream(side)
        graph.replay()
        sync()
        t0 = time.perf_counter()
        for _ in range(replays):
            graph.replay()
        sync()
        return (time.perf_counter() - t0) / (replays * calls) * 1e6

    rows = {}
    for M in [int(m) for m in __import__("os").environ.get("Q3_ROWS", "2048,576,64").split(",")]:
        for name, N, K in shapes:
            x = torch.randn(M, K, device="cuda:0").to(torch.bfloat16)
            copies = max(3, -(-600_000_000 // (N * K * 2)))    # more than the 256 MB cache holds, in turn
            ws = [(torch.randn(N, K, device="cuda:0") * 0.02).to(torch.bfloat16) for _ in range(copies)]
            out = torch.empty(M, N, device="cuda:0", dtype=torch.bfloat16)
            turn = [0]

            def chosen():
                turn[0] = (turn[0] + 1) % copies
                ops.linear(x, ws[turn[0]], out=out)

            entry = {"chosen_us": round(min(timed(chosen, copies), timed(chosen, copies)), 1), "plan": ops.matmul_plan(M, N, K),
                     "us_at_1_pflops": round(2.0 * M * N * K / 1e9, 1)}
            for shape in range(ops.gemm_tiles_configs()):
                def own():
                    turn[0] = (turn[0] + 1) % copies
                    ops.gemm_tiles(x, ws[turn[0]], shape, out=out)
                entry["tiles_%d_us" % shape] = round(min(timed(own, copies), timed(own, copies)), 1)
                splits = ops.gemm_tiles_splits(shape, M, N, K)
                if splits > 1:
                    def shared():
                        turn[0] = (turn[0] + 1) % copies
                        ops.gemm_tiles(x, ws[turn[0]], shape, out=out, splits=splits)
                    entry["tiles_%d_in_%d_us" % (shape, splits)] = round(min(timed(shared, copies), timed(shared, copies)), 1)
            rows["%s_%d" % (name, M)] = entry
            del ws
    print(json.dumps({"metric": "products of a layer, microseconds, %s bf16" % shape_name, "unit": "us", "n_gpus": 1,
                      "higher_is_better": False, "dtype": "bf16", "data": "synthetic", "products": rows}))
    return 0


def shared_prefix(args, config, model, shape_name, gen, sync):
    """64 requests that begin with the same 2,048 tokens (a system prompt, say) and go on with 32
    to 256 tokens of their own, 64 generated tokens each, with the prefix index on and off. Each
    engine serves such a load twice, with new tokens behind the shared ones each time; the second
    pass is the one reported (with the index on it finds the shared blocks of the first pass, as
    a server that has seen the system prompt before would)."""
    import random

    import torch

    from qwen3_from_scratch_amd.engine import SyncEngine

    requests, stem_len, context = 64, 2048, 4096
    rng = random.Random(0)
    stem = torch.randint(0, config.vocab_size, (stem_len,), generator=gen).tolist()
    tails = [rng.randint(32, 256) for _ in range(requests)]
    seconds, hits = {}, {}
    for on in (False, True):
        engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=context, block_size=BLOCK,
                            num_blocks=requests * context // BLOCK // 2, max_num_seqs=requests,
                            max_num_tokens=512 + requests, chunked_prefill_size=512, enable_prefix_cache=on)
        for _ in range(2):
            before = engine.runner.manager.prefix_hits
            # every pass has new tokens behind the shared ones: only those can be found again
            prompts = [stem + torch.randint(0, config.vocab_size, (n,), generator=gen).tolist() for n in tails]
            for p in prompts:
                engine.add_request(p, engine.default_params(64, temperature=0.0, ignore_eos=True))
            sync()
            t0 = time.perf_counter()
            while engine.scheduler.has_work():
                engine.step()
            sync()
            seconds[on] = time.perf_counter() - t0
            hits[on] = engine.runner.manager.prefix_hits - before
        del engine
    tokens_in = sum(len(p) for p in prompts)
    print(json.dumps({
        "metric": "shared-prefix load, seconds, %s %s" % (shape_name, "bf16" if args.dtype == "bfloat16" else "fp32"),
        "value": round(seconds[True], 3), "unit": "s", "n_gpus": 1, "higher_is_better": False,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "seconds_without_prefix_index": round(seconds[False], 3), "prompt_tokens": tokens_in,
        "prompt_tokens_taken_over": hits[True], "generated_tokens": 64 * requests,
        "config": {"model": "%s-shaped, random weights N(0, 0.02)" % shape_name, "requests": requests,
                   "shared_tokens": stem_len, "prefill_portion": 512, "context_len": context, "kv_block_size": BLOCK,
                   "layers": config.num_hidden_layers, "sampling": "greedy"},
    }))
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration (0 = all)")
    ap.add_argument("--dtype", default="bfloat16")
    ap.add_argument("--shape", default="8b", choices=sorted(SHAPES))
    ap.add_argument("--prompt", type=int, default=2048, help="tokens every request holds when decoding starts")
    ap.add_argument("--context", type=int, default=8192, help="tokens of cache per request")
    ap.add_argument("--workload", default="decode", choices=["decode", "continuous", "served", "prefix", "products"],
                    help="continuous: 64 requests at once, prompts of 128 to 4,096 tokens, 64 to 512 generated "
                         "tokens each, prompts in portions of 512 (its own JSON line; --steps and --warmup unused); "
                         "prefix: 64 requests that share their first 2,048 tokens, with the prefix index on and off; "
                         "products: a layer's four products by the chosen kernel and by each tile shape of the "
                         "hand-written one")
    ap.add_argument("--single-copy", action="store_true",
                    help="hold the matrices once (no tile-ordered copy for steps of few rows): half the weights' memory, slower decoding")
    ap.add_argument("--no-points", action="store_true", help="skip the batch-1 and batch-64 points")
    ap.add_argument("--no-probes", action="store_true",
                    help="skip the measurement of this GPU's read and matrix rates (for profiles of the engine alone)")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL,
                    help="length of the prompt whose one step is the prefill measurement (2,048 in the default line)")
    ap.add_argument("--skip-prefill", action="store_true",
                    help="skip the prefill measurement (for profiles of decoding alone; the line then has no value for it)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus %d is not supported" % args.gpus)
        return 2

    import torch

    from qwen3_from_scratch_amd.config import ModelConfig
    from qwen3_from_scratch_amd.engine import SyncEngine, random_model

    shape_name, raw = SHAPES[args.shape]
    raw = dict(raw)
    prompt_len, context = args.prompt, args.context
    if not 0 < prompt_len + args.warmup + args.steps < context <= raw["max_position_embeddings"]:
        print("bench.py: --prompt, --warmup and --steps must fit in --context, and that in the model's positions")
        return 2
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    config = ModelConfig.from_dict(raw)
    itemsize = 2 if args.dtype == "bfloat16" else 4
    torch.cuda.set_device(0)
    if args.workload == "products":
        return products(args, config, shape_name, torch.cuda.synchronize)
    model = random_model(config, dtype=args.dtype, device="cuda:0", seed=0, std=0.02, tiled_weights=not args.single_copy)
    gen = torch.Generator().manual_seed(1)

    def prompts(n, length):
        return [torch.randint(0, config.vocab_size, (length,), generator=gen).tolist() for _ in range(n)]

    def engine_for(batch):
        pages = batch * (context // BLOCK)
        return SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=context,
                          block_size=BLOCK, num_blocks=pages, max_num_seqs=batch,
                          max_num_tokens=max(PREFILL, batch), chunked_prefill_size=PREFILL,
                          enable_prefix_cache=False)       # every token of every prompt is computed

    def sync():
        torch.cuda.synchronize()

    if args.workload == "continuous":
        return continuous(args, config, model, shape_name, gen, sync)
    if args.workload == "served":
        return served(args, config, model, shape_name, gen, sync)
    if args.workload == "prefix":
        return shared_prefix(args, config, model, shape_name, gen, sync)

    # ---- prefill: one prompt of 2,048 tokens in one step (and of 8,192 for `points`) ----
    def prefill_of(tokens, timed=3):
        """Seconds of one step that is one whole prompt of `tokens` tokens: a warm-up, then the
        median of `timed` runs, each a new prompt."""
        room = tokens + 64
        engine = SyncEngine(model=model, path="", dtype=args.dtype, device="cuda:0", max_len=room,
                            block_size=BLOCK, num_blocks=-(-room // BLOCK), max_num_seqs=1,
                            max_num_tokens=tokens, chunked_prefill_size=tokens, enable_prefix_cache=False)
        timings = []
        for _ in range(1 + timed):
            engine.add_request(prompts(1, tokens)[0], engine.default_params(1, temperature=0.0, ignore_eos=True))
            sync()
            t0 = time.perf_counter()
            plan = engine.step()
            sync()
            timings.append(time.perf_counter() - t0)
            assert len(plan) == 1 and plan[0].num_tokens == tokens
            while engine.scheduler.has_work():
                engine.step()
        return sorted(timings[1:])[timed // 2]

    prefill = None
    prefill_s = None if args.skip_prefill else prefill_of(args.prefill_tokens)
    if prefill_s is not None:
        prefill = {"value": round(args.prefill_tokens / prefill_s, 1), "tokens": args.prefill_tokens,
                   "ms": round(prefill_s * 1e3, 3),
                   "frac": round(prefill_flops(config, args.prefill_tokens) / prefill_s / PEAK_FLOPS[args.dtype], 4)}

    # ---- decode ----
    def decode(batch, steps, warmup):
        engine = engine_for(batch)
        params = engine.default_params(context - prompt_len - 1, temperature=0.0, ignore_eos=True)
        requests = [engine.add_request(p, params) for p in prompts(batch, prompt_len)]
        while any(r.is_prefill for r in requests) or len(engine.scheduler.waiting):
            engine.step()
        for _ in range(warmup):
            engine.step()
        contexts = [r.num_tokens for r in requests]
        sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            plan = engine.step()
        sync()
        dt = time.perf_counter() - t0
        assert len(plan) == batch and all(s.num_tokens == 1 for s in plan)
        mean_contexts = [n + steps / 2 for n in contexts]
        return batch * steps / dt, dt / steps, mean_contexts

    tps, step_s, contexts = decode(args.batch, args.steps, args.warmup)
    need = decode_bytes(config, contexts, itemsize)
    roofline = {"bound": "hbm", "achieved": round(need / step_s / 1e9, 1), "peak": PEAK_HBM / 1e9,
                "unit": "GB/s", "frac": round(need / step_s / PEAK_HBM, 4)}
    points, points_roofline = {}, {}
    if not args.no_points and not args.skip_prefill and config.max_position_embeddings > LONG_PREFILL + 64:
        long_s = prefill_of(LONG_PREFILL, timed=1)          # one more step of a tenth of a second
        points["prefill_%d" % LONG_PREFILL] = round(LONG_PREFILL / long_s, 1)
        points_roofline["prefill_%d" % LONG_PREFILL] = round(
            prefill_flops(config, LONG_PREFILL) / long_s / PEAK_FLOPS[args.dtype], 4)
    if not args.no_points:
        for b in (1, 64):
            if b == args.batch:
                points["decode_b%d" % b] = round(tps, 1)
                points_roofline["decode_b%d" % b] = roofline["frac"]
                continue
            p_tps, p_step_s, p_contexts = decode(b, max(16, args.steps // 4), max(4, args.warmup // 2))
            points["decode_b%d" % b] = round(p_tps, 1)
            points_roofline["decode_b%d" % b] = round(decode_bytes(config, p_contexts, itemsize) / p_step_s / PEAK_HBM, 4)
    resident = sum(t.untyped_storage().nbytes() for t in _model_tensors(model))
    # what this GPU delivers, measured here: a plain read of 4 GB, the matrix instruction from registers
    from qwen3_from_scratch_amd import ops
    read_rate = matrix_rate = None
    if not args.no_probes:
        read_rate, matrix_rate = ops.measured_read_rate(), ops.measured_matrix_rate()
        roofline["measured_peak"] = round(read_rate / 1e9, 1)
        roofline["frac_of_measured"] = round(need / step_s / read_rate, 4)
    if prefill is not None and args.dtype == "bfloat16" and matrix_rate:
        prefill["measured_peak_tflops"] = round(matrix_rate / 1e12, 1)
        prefill["frac_of_measured"] = round(prefill_flops(config, args.prefill_tokens) / prefill_s / matrix_rate, 4)

    line = {
        "metric": "decode tok/s at batch 1/8/64 + prefill tok/s at 2048 tokens, %s %s"
                  % (shape_name, "bf16" if args.dtype == "bfloat16" else "fp32"),
        "value": round(tps, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic",
        "config": {
            "model": "%s-shaped, random weights N(0, 0.02)" % shape_name, "global_batch": args.batch,
            "seq_len": prompt_len, "parallelism": "single-gpu", "context_len": context,
            "layers": config.num_hidden_layers, "layers_full": full_layers, "hidden_size": config.hidden_size,
            "num_attention_heads": config.num_attention_heads, "num_key_value_heads": config.num_key_value_heads,
            "head_dim": config.head_dim, "intermediate_size": config.intermediate_size,
            "vocab_size": config.vocab_size, "rope_theta": config.rope_theta, "rms_norm_eps": config.rms_norm_eps,
            "tie_word_embeddings": config.tie_word_embeddings, "kv_block_size": BLOCK, "sampling": "greedy",
        },
        "prefill": prefill, "roofline": roofline, "points": points,
        # the same fraction of the HBM peak for the other batch sizes; what the weights hold on the GPU (bfloat16
        # matrices are kept twice, row-major and in the few-row kernel's order); how many-row products get their kernels
        "points_roofline": points_roofline, "resident_weight_gb": round(resident / 1e9, 2),
        "matmul_choice": "table and rule, no timing",
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
