"""The step function: run a batch of (request, its next tokens) from the cache."""

import torch

from ..cache import CacheManager, CacheStorage
from .batch import StepEntry, pack_step


class ModelRunner:
    """Owns the model, the cache manager and the cache's device memory.

    `step(entries)` runs only the tokens it is given, as one batch, on top of
    what earlier steps left in the cache, and returns float32 logits at the
    wanted places. The reference's counterpart returns sampled ids for the
    last row of every sequence (src/qwen3_from_scratch/inference/model_worker.py:212-227);
    sampling is a separate call here.
    """

    def __init__(self, model, page_size, num_pages, max_requests):
        self.model = model
        self.device = model.device
        self.manager = CacheManager(model.plane_needs, page_size, num_pages, max_requests)
        self.storage = CacheStorage(self.manager, model.precision.act, self.device)
        self.vocab_size = model.spec.vocab_size
        self.max_positions = getattr(model.position, "max_positions", None)

    def step(self, entries):
        """entries: list of StepEntry. Returns logits (R, V) float32 on the
        device, rows in the order of the entries and of their `want`."""
        if not entries:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        seen = set()
        for e in entries:
            if e.request_id in seen:
                raise ValueError("request %r appears twice in one step" % (e.request_id,))
            seen.add(e.request_id)
            if not e.tokens:
                raise ValueError("request %r brings no tokens" % (e.request_id,))
            if min(e.tokens) < 0 or max(e.tokens) >= self.vocab_size:
                raise ValueError("request %r has a token outside 0..%d" % (e.request_id, self.vocab_size - 1))
        m = self.manager
        if self.max_positions is not None:
            for e in entries:
                if self.length(e.request_id) + len(e.tokens) > self.max_positions:
                    raise ValueError("request %r would pass position %d, the model's last"
                                     % (e.request_id, self.max_positions - 1))
        admitted, reserved = [], []
        try:
            for e in entries:
                if not m.has(e.request_id):
                    m.admit(e.request_id)
                    admitted.append(e.request_id)
                m.reserve(e.request_id, len(e.tokens))
                reserved.append(e.request_id)
        except Exception:
            for rid in admitted:
                m.release(rid)
            raise
        lengths = [m.length(e.request_id) for e in entries]
        slots = [m.slot(e.request_id) for e in entries]
        tables = [[m.block_table(e.request_id, g) for e in entries] for g in range(len(m.groups))]
        batch, block_tables = pack_step(entries, lengths, slots, tables, self.device)
        self.storage.clear_fresh_slots()
        self.storage.bind(block_tables)
        logits = self.model.forward(batch, self.storage)
        for e in entries:
            m.commit(e.request_id, len(e.tokens))
        return logits

    def length(self, request_id):
        return self.manager.length(request_id) if self.manager.has(request_id) else 0

    def finish(self, request_id):
        """The request has ended; what it holds is given back."""
        if self.manager.has(request_id):
            self.manager.release(request_id)
