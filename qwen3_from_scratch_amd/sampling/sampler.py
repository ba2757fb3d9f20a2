"""Sampling: logits (R, V) to one token per row."""

from dataclasses import dataclass

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

    def sample(self, logits, params, counters):
        """`params[r]` and `counters[r]` (number of tokens the request has
        generated so far) belong to row r. Returns a list of token ids."""
        R = logits.shape[0]
        if R == 0:
            return []
        host = torch.empty((R, 4), dtype=torch.int64)
        temps = torch.empty(R, dtype=torch.float32)
        for r, (p, c) in enumerate(zip(params, counters)):
            temps[r] = p.temperature
            host[r, 0] = p.top_k
            host[r, 1] = p.seed
            host[r, 2] = c
        dev = host.to(self.device)
        out = ops.sample(logits, temps.to(self.device), dev[:, 0].to(torch.int32).contiguous(),
                         dev[:, 1].contiguous(), dev[:, 2].to(torch.int32).contiguous())
        return out.tolist()
