"""The in-process engine: continuous batching over the step function.

Interface and metric fields are those of the reference's SyncEngine
(src/qwen3_from_scratch/inference/sync_engine.py:28-182): `warmup`,
`generate_stream`, `generate`, `batch_generate`; `StreamChunk` and `PerfMetrics`
(inference/llm_engine.py:48-68), `BatchPerfMetrics` (sync_engine.py:17-25).
Besides the YAML file of the reference, an `EngineConfig` can be passed, and
prompts may be lists of token ids, which is all a model of random weights
understands.
"""

import itertools
import json
import os
import time
from dataclasses import dataclass

import torch

from ..config.engine_config import EngineConfig
from ..sampling import Sampler, SamplingParams
from .batch import StepEntry
from .loading import load_model
from .runner import ModelRunner
from .scheduler import Request, RequestStatus, Scheduled, Scheduler


@dataclass
class PerfMetrics:
    ttft: float
    token_count: int
    tps: float
    total_elapsed: float


@dataclass
class StreamChunk:
    delta: str
    metrics: PerfMetrics
    req_id: str = ""
    prompt_tokens: int = 0
    token_id: int = -1


@dataclass
class BatchPerfMetrics:
    per_request: list
    num_requests: int
    total_tokens: int
    total_elapsed: float
    aggregate_tps: float


def _load_tokenizer(path):
    if not any(os.path.isfile(os.path.join(path, f)) for f in ("tokenizer.json", "tokenizer_config.json")):
        return None
    from transformers import AutoTokenizer

    return AutoTokenizer.from_pretrained(path)


@dataclass
class _InFlight:
    """A step that is on the GPU: its plan, and its tokens on their way."""

    plan: list
    sampled: object


class SyncEngine:
    def __init__(self, config_path=None, model_name=None, log_interval=0, *, config=None, model=None,
                 **overrides):
        """`SyncEngine(config_path, model_name)` reads the reference's YAML;
        `SyncEngine(config=EngineConfig(path=...))` or keyword options
        (`path=..., dtype=..., max_num_seqs=...`) do without a file. `model`
        hands in an already loaded model."""
        if config is None:
            if config_path is not None:
                config = EngineConfig.from_yaml(str(config_path), model_name, **overrides)
            else:
                config = EngineConfig(**overrides)
        self.config = config
        self.model_name = model_name or config.name
        self.log_interval = log_interval
        self.model = model if model is not None else load_model(config.path, config.dtype, config.device,
                                                                 tiled_weights=config.tiled_weights,
                                                                 components=config.components)
        self.tokenizer = _load_tokenizer(config.path) if config.path else None
        mc = self.model.config
        self.max_len = min(config.max_len, mc.max_position_embeddings)
        num_blocks = config.num_blocks or self._blocks_from_memory()
        self.runner = ModelRunner(self.model, config.block_size, num_blocks, max_requests=config.max_num_seqs,
                                  use_graphs=config.use_graphs, prefix_cache=config.enable_prefix_cache)
        self.sampler = Sampler(self.model.device)
        self.scheduler = Scheduler(
            self.runner.manager, config.max_num_seqs, config.max_num_tokens, config.chunked_prefill_size,
            max_len=self.max_len, release=self.runner.finish, portion_multiple=self.model.portion_multiple())
        self.eos_ids = self._eos_ids()
        self._ids = itertools.count()
        self.steps = 0
        # one step ahead of the tokens only where a step is a graph replay: otherwise the host
        # is busy launching kernels anyway
        self.lookahead = bool(config.lookahead) and self.runner.use_graphs
        self._ahead = None

    # ---- set-up ----
    def _blocks_from_memory(self):
        """Pages that fit in `gpu_utilization` of the free memory beside the
        requests' fixed-size states, as the reference
        sizes its cache (src/qwen3_from_scratch/inference/kv_cache/paged_cache.py:36-49).
        A page stands for its tokens in every layer of every group."""
        per_token = per_request = 0
        for need in self.model.plane_needs:
            if need is None:
                continue
            per_token += need.bytes_per_token(self.model.precision.act)
            per_request += need.bytes_of_state()    # a slot per request (and a spare one) in every plane with a state
        per_page = max(1, per_token * self.config.block_size)
        if self.model.device.type == "cuda":
            free = torch.cuda.mem_get_info(self.model.device)[0]
        else:
            free = 1 << 30
        budget = int(free * self.config.gpu_utilization) - per_request * (self.config.max_num_seqs + 1)
        wanted = max(0, budget) // per_page
        enough = self.config.max_num_seqs * (-(-self.max_len // self.config.block_size))
        return max(1, min(wanted, enough))

    def _eos_ids(self):
        ids = set(self.model.config.eos_token_ids) | set(self.config.eos_ids)
        gen = os.path.join(self.config.path, "generation_config.json") if self.config.path else ""
        if gen and os.path.isfile(gen):
            with open(gen) as fh:
                eos = json.load(fh).get("eos_token_id")
            if isinstance(eos, int):
                ids.add(eos)
            elif isinstance(eos, list):
                ids.update(eos)
        if self.tokenizer is not None and self.tokenizer.eos_token_id is not None:
            ids.add(int(self.tokenizer.eos_token_id))
        return tuple(sorted(ids))

    # ---- requests ----
    def _encode(self, prompt):
        if isinstance(prompt, (list, tuple)) and (not prompt or isinstance(prompt[0], int)):
            return list(prompt)
        if self.tokenizer is None:
            raise ValueError("the model folder has no tokenizer: pass prompts as lists of token ids")
        if not isinstance(prompt, str):
            prompt = self.tokenizer.apply_chat_template(prompt, tokenize=False, add_generation_prompt=True)
        return list(self.tokenizer(prompt).input_ids)

    def _decode(self, ids):
        if self.tokenizer is None:
            return ""
        return self.tokenizer.decode(ids, skip_special_tokens=True)

    def default_params(self, max_new_tokens=None, **kw):
        gen = self.config.generation
        return SamplingParams(
            temperature=kw.get("temperature", gen.temperature),
            top_k=kw.get("top_k", gen.top_k),
            seed=kw.get("seed", self.config.seed),
            max_new_tokens=max_new_tokens if max_new_tokens else gen.max_new_tokens,
            ignore_eos=kw.get("ignore_eos", False),
        )

    def add_request(self, prompt, params=None, request_id=None):
        """Queue a prompt (text, chat messages or token ids); returns the Request."""
        request = Request(
            request_id=request_id if request_id is not None else "req-%d" % next(self._ids),
            prompt=self._encode(prompt), params=params or self.default_params(), eos_ids=self.eos_ids)
        self.scheduler.add(request)
        return request

    def abort(self, request):
        """Stop a request before it has finished; its pages and slot are given back."""
        self.scheduler.abort(request)

    # ---- the loop body ----
    def step(self):
        """Schedule, run the step function, sample, book-keep. Returns the plan
        (a list of Scheduled); requests that got a token have it in
        `last_token_id`, finished ones have status FINISHED.

        While the same requests decode on, the next step is put on the GPU
        before this one's tokens are read back (`_launch_ahead`), so that the
        GPU does not wait for the host between steps; the plan returned is
        always that of the step whose tokens have arrived."""
        current, self._ahead = self._ahead, None
        if current is not None and not any(s.request.status == RequestStatus.RUNNING for s in current.plan):
            current = None               # its requests ended or were taken out meanwhile: nothing to report
        if current is None:
            plan = self.scheduler.schedule()
            if not plan:
                return plan
            current = self._launch(plan)
        if self.lookahead:
            self._ahead = self._launch_ahead(current)
        tokens = self.sampler.collect(current.sampled) if current.sampled is not None else []
        it = iter(tokens)
        plan, sampled = [], []
        for s in current.plan:
            token = next(it) if s.samples else None
            if s.request.status != RequestStatus.RUNNING:
                continue                 # ended (or was taken out) while this step was on its way
            plan.append(s)
            if s.samples:
                sampled.append(token)
        self.scheduler.after_step(plan, sampled)
        self.steps += 1
        return plan

    def _launch(self, plan):
        """Put a scheduled plan on the GPU: the step function, then sampling."""
        entries = []
        for s in plan:
            req = s.request
            tokens = req.tokens[req.computed: req.computed + s.num_tokens]
            entries.append(StepEntry(req.request_id, tokens, [s.num_tokens - 1] if s.samples else []))
        logits = self.runner.step(entries)
        sampling = [s.request for s in plan if s.samples]
        sampled = None
        if sampling:
            sampled = self.sampler.launch(logits, [r.params for r in sampling], [len(r.generated) for r in sampling])
        return _InFlight(plan, sampled)

    def _launch_ahead(self, current):
        """The step after `current`, if it is certain enough what it will be:
        every running request decodes in `current`, none of them ends with
        `current`'s token by its count, nobody waits, and pages are there.
        Its input tokens are `current`'s sampled ones, read on the device. A
        request that ends with `current`'s token after all (an end-of-sequence
        token) has then made one step too many, whose token is dropped and
        whose pages went back with the others'."""
        sched = self.scheduler
        plan = current.plan
        if sched.waiting or len(plan) != len(sched.running) or current.sampled is None:
            return None
        spare = [0] * len(self.runner.manager.groups)
        for s in plan:
            req = s.request
            if (s.num_tokens != 1 or not s.samples or req.status != RequestStatus.RUNNING or req.is_prefill
                    or len(req.generated) + 2 > req.params.max_new_tokens
                    or not self.runner.manager.can_grow(req.request_id, 1, spare)):
                return None
        entries = [StepEntry(s.request.request_id, [0], [0]) for s in plan]
        logits = self.runner.step(entries, device_tokens=current.sampled.tokens)
        sampled = self.sampler.launch(logits, [s.request.params for s in plan],
                                      [len(s.request.generated) + 1 for s in plan])
        return _InFlight([Scheduled(s.request, 1, True) for s in plan], sampled)

    # ---- the reference's interface ----
    def warmup(self, prompt=None, num_tokens=3):
        """A short request, so that what is built or tuned at first use does
        not count against the first real request."""
        if prompt is None:
            prompt = [1, 2, 3] if self.tokenizer is None else "你好"
        for _ in self.generate_stream(prompt, num_tokens):
            pass

    def generate_stream(self, prompt, max_new_tokens=None, **sampling):
        request = self.add_request(prompt, self.default_params(max_new_tokens, **sampling))
        start = time.perf_counter()
        first = None
        count = 0
        while True:
            plan = self.step()
            now = time.perf_counter()
            for s in plan:
                if s.request is not request or not s.samples:
                    continue
                count += 1
                if first is None:
                    first = now
                    metrics = PerfMetrics(now - start, 1, 0.0, now - start)
                else:
                    span = now - first
                    metrics = PerfMetrics(first - start, count, (count - 1) / span if span > 0 else 0.0,
                                          now - start)
                yield StreamChunk(self._decode([request.last_token_id]), metrics, str(request.request_id),
                                  len(request.prompt), request.last_token_id)
                if request.status == RequestStatus.FINISHED:
                    return

    def generate(self, prompt, max_new_tokens=None, **sampling):
        """The whole answer as text (token ids joined by spaces without a tokenizer)."""
        chunks = list(self.generate_stream(prompt, max_new_tokens, **sampling))
        if self.tokenizer is None:
            return " ".join(str(c.token_id) for c in chunks)
        return "".join(c.delta for c in chunks)

    def generate_ids(self, prompts, max_new_tokens=None, **sampling):
        """Token-level batch generation: list of generated id lists, in order."""
        requests = [self.add_request(p, self.default_params(max_new_tokens, **sampling)) for p in prompts]
        while any(r.status != RequestStatus.FINISHED for r in requests):
            self.step()
        return [list(r.generated) for r in requests]

    def batch_generate(self, prompts, max_new_tokens=None, **sampling):
        """All prompts queued at once and batched continuously until all have
        ended; returns (texts in order, BatchPerfMetrics)."""
        start = time.perf_counter()
        requests = [self.add_request(p, self.default_params(max_new_tokens, **sampling)) for p in prompts]
        first, last, counts = {}, {}, {}
        while any(r.status != RequestStatus.FINISHED for r in requests):
            plan = self.step()
            now = time.perf_counter()
            for s in plan:
                if s.samples:
                    rid = s.request.request_id
                    first.setdefault(rid, now)
                    last[rid] = now
                    counts[rid] = counts.get(rid, 0) + 1
            if self.log_interval > 0 and self.steps % self.log_interval == 0:
                done = sum(r.status == RequestStatus.FINISHED for r in requests)
                total = sum(len(r.generated) for r in requests)
                print("[batch] step=%d pending=%d completed=%d total_tokens=%d aggregate_tps=%.2f"
                      % (self.steps, len(requests) - done, done, total, total / max(now - start, 1e-9)))
        elapsed = time.perf_counter() - start
        per_request = []
        for r in requests:
            rid = r.request_id
            n = counts.get(rid, 0)
            span = last.get(rid, start) - first.get(rid, start)
            per_request.append(PerfMetrics(first.get(rid, start) - start, n,
                                           (n - 1) / span if span > 0 else 0.0, last.get(rid, start) - start))
        total = sum(len(r.generated) for r in requests)
        texts = [self._decode(r.generated) if self.tokenizer is not None
                 else " ".join(map(str, r.generated)) for r in requests]
        return texts, BatchPerfMetrics(per_request, len(requests), total, elapsed,
                                       total / elapsed if elapsed > 0 else 0.0)
