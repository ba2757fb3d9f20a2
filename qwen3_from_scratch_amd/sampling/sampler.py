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


class Sampler:
    """Greedy: arg-max (inference/sampler.py:17-21). Temperature:
    a draw from softmax(logits / temperature) (:24-33). Top-k: the same among
    the k largest logits (:36-56). All three are one kernel launch over the
    float32 logits; draws use Gumbel noise keyed by (seed, index of the token
    being generated)."""

    def __init__(self, device):
        self.device = torch.device(device)
        self._buffers = {}

    def _buffer(self, R):
        """Five int32 words per row, pinned on the host and on the device: seed (two words),
        temperature, top_k, counter; one copy brings a step's parameters."""
        pair = self._buffers.get(R)
        if pair is None:
            host = torch.empty(5 * R, dtype=torch.int32)
            if self.device.type == "cuda":
                host = host.pin_memory()
            pair = (host, torch.empty(5 * R, dtype=torch.int32, device=self.device))
            if len(self._buffers) > 64:
                self._buffers.clear()
            self._buffers[R] = pair
        return pair

    def sample(self, logits, params, counters):
        """`params[r]` and `counters[r]` (number of tokens the request has
        generated so far) belong to row r. Returns a list of token ids."""
        R = logits.shape[0]
        if R == 0:
            return []
        host, dev = self._buffer(R)
        words = host.numpy()
        words[0:2 * R].view(np.int64)[:] = [p.seed for p in params]
        words[2 * R:3 * R].view(np.float32)[:] = [p.temperature for p in params]
        words[3 * R:4 * R] = [p.top_k for p in params]
        words[4 * R:5 * R] = counters
        # queued behind the step's kernels without waiting for them; the list below is the only wait
        dev.copy_(host, non_blocking=True)
        any_top_k = any(p.top_k > 0 and p.temperature > 0 for p in params)
        out = ops.sample(logits, dev[2 * R:3 * R].view(torch.float32), dev[3 * R:4 * R], dev[0:2 * R].view(torch.int64),
                         dev[4 * R:5 * R], any_top_k=any_top_k)
        return out.tolist()
