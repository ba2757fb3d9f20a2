"""The asynchronous engine: any number of coroutines stream from one model at once.

Interface of the reference's LLMEngine
(src/qwen3_from_scratch/inference/llm_engine.py:71-340; used as in
examples/llm_runner.py:11-24): `LLMEngine(config_path, model_name)`,
`wait_ready()`, `await warmup()`, `async for chunk in generate_stream(prompt,
max_new_tokens, tools, tool_choice, enable_thinking, ignore_eos)`, `close()`;
`StreamChunk` and `PerfMetrics` carry the same fields.

The reference keeps the tokenizer and the scheduler in a thread of the caller's
process and the model in a worker process that it feeds through queues
(:86-103, :144-199). Here one background thread owns a `SyncEngine` (model,
cache, scheduler, sampler): it takes new requests from a queue, makes a step,
and hands every request's new token to the event loop that asked for it. The
kernels release the interpreter lock while they run, so the callers' loops go
on meanwhile. Requests that arrive while others are being served join the next
step: continuous batching across callers.
"""

import asyncio
import itertools
import queue
import threading
import time

from .scheduler import RequestStatus
from .sync_engine import PerfMetrics, StreamChunk, SyncEngine


class _Stream:
    """What the engine thread knows of one caller."""

    def __init__(self, loop, results):
        self.loop = loop
        self.results = results          # an asyncio.Queue that lives in `loop`
        self.request = None

    def send(self, item):
        self.loop.call_soon_threadsafe(self.results.put_nowait, item)


class LLMEngine:
    def __init__(self, config_path=None, model_name=None, *, config=None, model=None, **overrides):
        """Same arguments as `SyncEngine`. The model is loaded by the engine's
        own thread; `wait_ready()` returns when it is there."""
        self._arguments = (config_path, model_name, config, model, overrides)
        self._incoming = queue.Queue()
        self._ready = threading.Event()
        self._failure = None
        self._finished = False
        self._streams = {}
        self._ids = itertools.count()
        self.engine = None
        self.thread = threading.Thread(target=self._run, name="llm-engine", daemon=True)
        self.thread.start()

    # ---- the engine's thread ----
    def _run(self):
        config_path, model_name, config, model, overrides = self._arguments
        try:
            self.engine = SyncEngine(config_path, model_name, config=config, model=model, **overrides)
        except Exception as exc:                # the callers learn of it in wait_ready()
            self._failure = exc
            self._ready.set()
            return
        self._ready.set()
        engine = self.engine
        while not self._finished:
            self._take_incoming(wait=not engine.scheduler.has_work())
            if self._finished or not engine.scheduler.has_work():
                continue
            try:
                plan = engine.step()
            except Exception as exc:            # nothing can go on: every caller is told
                for stream in self._streams.values():
                    stream.send(exc)
                self._streams.clear()
                self._failure = exc
                return
            for s in plan:
                stream = self._streams.get(s.request.request_id)
                if stream is None or not s.samples:
                    continue
                stream.send((s.request.last_token_id, engine._decode([s.request.last_token_id])))
                if s.request.status == RequestStatus.FINISHED:
                    stream.send(None)
                    del self._streams[s.request.request_id]
        for stream in self._streams.values():   # closed while requests were live
            stream.send(RuntimeError("the engine was closed"))
        self._streams.clear()

    def _take_incoming(self, wait):
        try:
            item = self._incoming.get(timeout=0.05) if wait else self._incoming.get_nowait()
        except queue.Empty:
            return
        while True:
            if item is not None:
                self._handle(item)
            try:
                item = self._incoming.get_nowait()
            except queue.Empty:
                return

    def _handle(self, item):
        kind, request_id = item[0], item[1]
        engine = self.engine
        if kind == "abort":
            stream = self._streams.pop(request_id, None)
            if stream is not None and stream.request is not None \
                    and stream.request.status != RequestStatus.FINISHED:
                engine.abort(stream.request)
            return
        _, _, prompt, template, max_new_tokens, sampling, stream = item
        try:
            if template is not None:
                if engine.tokenizer is None:
                    raise ValueError("the model folder has no tokenizer: pass prompts as lists of token ids")
                prompt = engine.tokenizer.apply_chat_template(prompt, tokenize=False, **template)
            stream.request = engine.add_request(prompt, engine.default_params(max_new_tokens, **sampling),
                                                request_id=request_id)
        except Exception as exc:                # a prompt that cannot be served: its caller alone is told
            stream.send(exc)
            return
        self._streams[request_id] = stream
        stream.send(len(stream.request.prompt))

    # ---- the callers' side ----
    def wait_ready(self):
        """Block until the model is loaded (llm_engine.py:303-310)."""
        self._ready.wait()
        if self._failure is not None:
            raise RuntimeError("the engine could not start") from self._failure

    async def warmup(self, prompt=None, num_tokens=3):
        """Wait for the model and run one short request, so that what is built
        or tuned at first use does not count against the first real request
        (llm_engine.py:312-327)."""
        await asyncio.get_running_loop().run_in_executor(None, self._ready.wait)
        self.wait_ready()
        if prompt is None:
            prompt = [1, 2, 3] if self.engine.tokenizer is None else "你好"
        async for _ in self.generate_stream(prompt, num_tokens, ignore_eos=True):
            pass

    async def generate_stream(self, prompt, max_new_tokens=None, tools=None, tool_choice=None,
                              enable_thinking=None, ignore_eos=False, **sampling):
        """Yields a StreamChunk per generated token. `prompt`: text, a list of
        chat messages (rendered by the tokenizer's chat template with the
        generation prompt added; `tools`, `tool_choice` and `enable_thinking`
        are passed to it, llm_engine.py:221-236), or a list of token ids.
        `sampling`: temperature, top_k, seed. Leaving the loop early takes the
        request out of the engine."""
        template = None
        if isinstance(prompt, (list, tuple)) and prompt and isinstance(prompt[0], dict):
            template = {"add_generation_prompt": True}
            for key, value in (("tools", tools), ("tool_choice", tool_choice), ("enable_thinking", enable_thinking)):
                if value is not None:
                    template[key] = value
        if self._finished:
            raise RuntimeError("the engine is closed")
        if self._failure is not None:
            raise RuntimeError("the engine has stopped") from self._failure
        request_id = "req-%d" % next(self._ids)
        stream = _Stream(asyncio.get_running_loop(), asyncio.Queue())
        sampling = dict(sampling, ignore_eos=ignore_eos)
        start = time.perf_counter()
        self._incoming.put(("add", request_id, prompt, template, max_new_tokens, sampling, stream))
        first = None
        count = prompt_tokens = 0
        ended = False
        try:
            while True:
                item = await stream.results.get()
                if item is None:
                    ended = True
                    return
                if isinstance(item, BaseException):
                    ended = True
                    raise item
                if isinstance(item, int):       # the prompt's length, once the request is queued
                    prompt_tokens = item
                    continue
                token_id, text = item
                now = time.perf_counter()
                count += 1
                if first is None:
                    first = now
                    metrics = PerfMetrics(now - start, 1, 0.0, now - start)
                else:
                    span = now - first
                    metrics = PerfMetrics(first - start, count, (count - 1) / span if span > 0 else 0.0, now - start)
                yield StreamChunk(text, metrics, request_id, prompt_tokens, token_id)
        finally:
            if not ended:
                self._incoming.put(("abort", request_id))

    def close(self):
        """Stop the engine's thread; requests still live are told so."""
        self._finished = True
        self._incoming.put(None)
        self.thread.join()
