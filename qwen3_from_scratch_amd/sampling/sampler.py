"""Sampling: logits (R, V) to one token per row."""

from dataclasses import dataclass

import numpy as np
import torch

from .. import ops


@dataclass
class SamplingParams:
    """Per-request sampling options. The reference has one sampler per engine,
    chosen as: temperature <= 0 greedy; temperature > 0 and top_k > 0 top-k;
    else temperature (src/qwen3_from_scratch/inference/model_worker.py:32-41).
    The same rule holds here per request, and a seed makes a request's tokens
    reproducible whatever it is batched with."""

    temperature: float = 0.0
    top_k: int = 0
    seed: int = 0
    max_new_tokens: int = 100
    ignore_eos: bool = False


class Sampled:
    """A step's tokens on their way: `tokens` on the device (the next step may
    read them there), a pinned copy on the host, and the event after which the
    copy has arrived."""

    def __init__(self, tokens, host, event):
        self.tokens = tokens
        self.host = host
        self.event = event


class Sampler:
    """Greedy: arg-max (inference/sampler.py:17-21). Temperature:
    a draw from softmax(logits / temperature) (:24-33). Top-k: the same among
    the k largest logits (:36-56). All three go through the same kernels over
    the float32 logits; draws use Gumbel noise keyed by (seed, index of the token
    being generated).

    `launch` queues a step's sampling behind its kernels and returns at once;
    `collect` waits for the tokens. Up to `RING` launches may be uncollected at
    a time: each has staging buffers of its own."""

    RING = 4

    def __init__(self, device):
        self.device = torch.device(device)
        self._rings = {}

    def _staging(self, R):
        """Pinned host memory and its device twin for a step's parameters (five
        int32 words per row: seed in two, temperature, top_k, counter) and
        tokens (one int32 per row); RING sets per batch size, used in turn."""
        ring = self._rings.get(R)
        if ring is None:
            if len(self._rings) > 64:
                self._rings.clear()
            ring = self._rings[R] = {"next": 0, "sets": []}
        if len(ring["sets"]) < self.RING:
            host = torch.empty(6 * R, dtype=torch.int32)
            if self.device.type == "cuda":
                host = host.pin_memory()
            entry = {"host": host, "dev": torch.empty(6 * R, dtype=torch.int32, device=self.device), "event": None}
            ring["sets"].append(entry)
            return entry
        entry = ring["sets"][ring["next"]]
        ring["next"] = (ring["next"] + 1) % self.RING
        if entry["event"] is not None:
            entry["event"].synchronize()           # its last user's copies are done
        return entry

    def launch(self, logits, params, counters):
        """`params[r]` and `counters[r]` (number of tokens the request has
        generated before this one) belong to row r. Returns a `Sampled`."""
        R = logits.shape[0]
        entry = self._staging(R)
        host, dev = entry["host"], entry["dev"]
        words = host.numpy()
        words[0:2 * R].view(np.int64)[:] = [p.seed for p in params]
        words[2 * R:3 * R].view(np.float32)[:] = [p.temperature for p in params]
        words[3 * R:4 * R] = [p.top_k for p in params]
        words[4 * R:5 * R] = counters
        # queued behind the step's kernels without waiting for them
        dev[:5 * R].copy_(host[:5 * R], non_blocking=True)
        any_top_k = any(p.top_k > 0 and p.temperature > 0 for p in params)
        tokens = dev[5 * R:6 * R]
        ops.sample(logits, dev[2 * R:3 * R].view(torch.float32), dev[3 * R:4 * R], dev[0:2 * R].view(torch.int64),
                   dev[4 * R:5 * R], out=tokens, any_top_k=any_top_k)
        host[5 * R:6 * R].copy_(tokens, non_blocking=True)
        event = None
        if self.device.type == "cuda":
            event = torch.cuda.Event()
            event.record()
        entry["event"] = event
        return Sampled(tokens, host[5 * R:6 * R], event)

    def collect(self, sampled):
        """The tokens of a `launch`, as a list."""
        if sampled.event is not None:
            sampled.event.synchronize()
        return sampled.host.tolist()

    def sample(self, logits, params, counters):
        """`launch` and `collect` in one call."""
        if logits.shape[0] == 0:
            return []
        return self.collect(self.launch(logits, params, counters))
