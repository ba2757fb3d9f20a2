"""The step function: run a batch of (request, its next tokens) from the cache."""

import contextlib
import gc

import torch

from ..cache import CacheManager, CacheStorage
from .batch import StepEntry, pack_step, packed_layout, packed_size


def padded_batch(n):
    """The batch size a graph is captured for when `n` requests decode: the
    next of 1, 2, 3, 4, 6, 8, 12, 16, 24, ... so that batches whose size moves up
    and down as requests come and go share a few graphs. The rows that fill a
    batch up stand for nobody: token 0 at position 0, written to the cache's
    spare page and slot, their logits dropped."""
    size = 1
    while size < n:
        if size < 4:
            size += 1
        else:                       # a power of two is followed by its one-and-a-half, that by the next power
            size = size * 3 // 2 if size & (size - 1) == 0 else size * 4 // 3
    return size


@contextlib.contextmanager
def collector_paused():
    """No object is finalized by the cyclic collector inside this block: what
    is already dead is collected on entry, and the automatic collector is off
    until the block ends.

    A stream capture must not be interrupted by a finalizer that talks to the
    device. The collector runs whenever enough containers have been allocated,
    in the middle of any Python code, and finalizes whatever dead cycles it
    finds: an engine that a caller dropped while something still pointed back
    at it (a closure over one of its own methods is enough), and with it its
    captured graphs. Destroying a captured graph synchronizes the device, which
    is an error while a capture is open, and an error in a destructor ends the
    process (SIGABRT). The same engine dropped without a cycle is freed at once
    by its reference count, outside any capture."""
    gc.collect()
    was_enabled = gc.isenabled()
    gc.disable()
    try:
        yield
    finally:
        if was_enabled:
            gc.enable()


class DecodeDescription:
    """The packed description of a step of `B` rows of one token each, kept in
    one host buffer between steps (host memory only: a graph's device twin is
    the caller's). The first rows are the step's requests, the rest fill the
    batch up (see `padded_batch`): token 0 at position 0 on the spare page and
    slot. While the same requests decode on, each one token further, the buffer
    is patched in place: tokens, positions and lengths by one, block tables in
    their new entries; anything else packs it afresh."""

    def __init__(self, B, widths, host, spare_pages, spare_slot, windowed):
        self.B = B
        self.widths = list(widths)
        self.layout = packed_layout(B, B, B, self.widths)
        self.host = host                     # int32 tensor of at least layout.total words
        self.spare_pages = list(spare_pages)
        self.spare_slot = spare_slot
        self.windowed = list(windowed)       # per group: entries may turn -1 anywhere in a table
        self.last_ids = self.last_lengths = self.last_slots = self.last_table_lens = None

    def fill(self, entries, ids, lengths, slots, tables, device=None, dev=None):
        """Bring the buffer to this step. `ids[i]` tells requests (and admissions of one request) apart.
        Returns the StepBatch and block tables if the buffer was packed afresh, else None."""
        fresh = None
        if (self.last_ids is not None and ids == self.last_ids and slots == self.last_slots
                and all(n == m + 1 for n, m in zip(lengths, self.last_lengths))):
            self._advance(entries, tables)
        else:
            fill = self.B - len(entries)
            fresh = pack_step(
                list(entries) + [StepEntry(None, [0])] * fill, list(lengths) + [0] * fill,
                list(slots) + [self.spare_slot] * fill,
                [list(group) + [[self.spare_pages[g]]] * fill for g, group in enumerate(tables)],
                device, fixed_widths=self.widths, buffers=(self.host, dev), all_rows=True)
        self.last_ids, self.last_lengths, self.last_slots = list(ids), list(lengths), list(slots)
        self.last_table_lens = [[len(t) for t in group] for group in tables]
        return fresh

    def _advance(self, entries, tables):
        lay, n, host = self.layout, len(entries), self.host.numpy()
        first = lay.tokens.start
        host[first:first + n] = [e.tokens[0] for e in entries]
        first = lay.positions.start
        host[first:first + n] += 1              # the rows that fill up stay where they are
        first = lay.kv_lens.start
        host[first:first + n] += 1              # keys visible after the step
        for g, (group_tables, (sl, w)) in enumerate(zip(tables, lay.tables)):
            for i, t in enumerate(group_tables):
                had = 0 if self.windowed[g] else self.last_table_lens[g][i]
                if len(t) > w:
                    raise ValueError("a block table is wider than the fixed width %d" % w)
                if len(t) > had:
                    host[sl.start + i * w + had: sl.start + i * w + len(t)] = t[had:]


class _DecodeGraph:
    """A captured HIP graph of the model's forward pass for `B` rows of one
    token each, none longer than `max_kv_len`; the first rows are the step's
    requests, the rest fill up (see `padded_batch`). The batch description lives
    in fixed device memory that is refilled before every replay; what the
    kernels' launches depend on (the longest sequence, hence how keys are
    split over workgroups) is fixed at `max_kv_len`, a power of two, so a
    batch gets a new graph each time its longest request doubles."""

    def __init__(self, runner, B, max_kv_len):
        m = runner.manager
        self.B = B
        self.max_kv_len = max_kv_len
        widths = [m.table_width(g, runner.max_request_tokens) for g in range(len(m.groups))]
        n = packed_size(B, B, B, widths)
        self.host = torch.empty(n, dtype=torch.int32).pin_memory()
        self.dev = torch.zeros(n, dtype=torch.int32, device=runner.device)
        storage = runner.storage
        self.description = DecodeDescription(
            B, widths, self.host, [storage.spare_page(g) for g in range(len(m.groups))], storage.spare_slot,
            [grp.window > 0 for grp in m.groups])
        self.graph = None
        self.logits = None
        self.copied = torch.cuda.Event()

    def run(self, runner, entries, lengths, slots, tables, device_tokens=None):
        self.copied.synchronize()          # the last step's copy has left the host buffer
        ids = [(e.request_id, runner.manager.admission(e.request_id)) for e in entries]
        if self.graph is None:
            self.description.last_ids = None
        fresh = self.description.fill(entries, ids, lengths, slots, tables, runner.device, self.dev)
        if fresh is None:
            self.dev.copy_(self.host, non_blocking=True)
        elif self.graph is None:
            batch, block_tables = fresh
            batch.max_kv_len = self.max_kv_len
            self._capture(runner, batch, block_tables)
        self.copied.record()
        if device_tokens is not None:      # the tokens are still on the device: they replace the placeholders
            self.dev[0:len(entries)].copy_(device_tokens)
        self.graph.replay()
        return self.logits

    def retire(self, device):
        """Before the graph and its buffers are let go: its last replay has ended, and so has
        whatever was queued behind it to read its logits (the sampler of a step that is still
        on its way)."""
        torch.cuda.synchronize(device)

    def _capture(self, runner, batch, block_tables):
        runner.storage.bind(block_tables)
        # once eagerly on a side stream (libraries build and tune at first use), then capture
        side = torch.cuda.Stream(device=runner.device)
        side.wait_stream(torch.cuda.current_stream(runner.device))
        with torch.cuda.stream(side):
            runner.model.forward(batch, runner.storage)
        torch.cuda.current_stream(runner.device).wait_stream(side)
        torch.cuda.synchronize(runner.device)
        graph = torch.cuda.CUDAGraph()
        with collector_paused():
            with torch.cuda.graph(graph):
                self.logits = runner.model.forward(batch, runner.storage)
        self.graph = graph


class ModelRunner:
    """Owns the model, the cache manager and the cache's device memory.

    `step(entries)` runs only the tokens it is given, as one batch, on top of
    what earlier steps left in the cache, and returns float32 logits at the
    wanted places. The reference's counterpart returns sampled ids for the
    last row of every sequence (src/qwen3_from_scratch/inference/model_worker.py:212-227);
    sampling is a separate call here.

    Steps in which every request brings a single token replay a captured HIP
    graph (one per batch size), which takes the launch overhead of some
    hundreds of kernels off the critical path; the graph runs the same model
    code, kernels and cache as any other step.
    """

    def __init__(self, model, page_size, num_pages, max_requests, use_graphs=True, prefix_cache=False):
        self.model = model
        self.device = model.device
        self.manager = CacheManager(model.plane_needs, page_size, num_pages, max_requests, prefix_cache=prefix_cache)
        self.storage = CacheStorage(self.manager, model.precision.act, self.device)
        self.vocab_size = model.spec.vocab_size
        # the shortest table of positions among the model's position part and the layers' own
        tables = [getattr(part, "max_positions", None)
                  for part in [model.position] + list(getattr(model, "layer_positions", {}).values())]
        self.max_positions = min((n for n in tables if n is not None), default=None)
        self.max_request_tokens = self.manager.capacity_tokens()
        if self.max_positions is not None:
            self.max_request_tokens = min(self.max_request_tokens, self.max_positions)
        self.use_graphs = bool(use_graphs) and self.device.type == "cuda" and model.graph_safe()
        self._graphs = {}
        self.max_graphs = 32

    def step(self, entries, device_tokens=None):
        """entries: list of StepEntry. Returns logits (R, V) float32 on the
        device, rows in the order of the entries and of their `want`. The
        tensor may be overwritten by the next call of step().
        `device_tokens`: an int32 device tensor with one token per entry, for a
        step of single tokens that are not on the host yet (the last step's
        sampled ones); the entries' own tokens are then placeholders."""
        if not entries:
            return torch.empty((0, self.vocab_size), dtype=torch.float32, device=self.device)
        single = all(len(e.tokens) == 1 for e in entries)
        if device_tokens is not None and not (single and device_tokens.shape == (len(entries),)
                                              and device_tokens.dtype == torch.int32):
            raise ValueError("device tokens come one per entry (int32), for entries of one token each")
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
        admitted = []
        try:
            for e in entries:
                if not m.has(e.request_id):
                    m.admit(e.request_id)
                    admitted.append(e.request_id)
                m.reserve(e.request_id, len(e.tokens))
        except Exception:
            for rid in admitted:
                m.release(rid)
            raise
        lengths = [m.length(e.request_id) for e in entries]
        slots = [m.slot(e.request_id) for e in entries]
        tables = [[m.block_table(e.request_id, g) for e in entries] for g in range(len(m.groups))]
        self.storage.clear_fresh_slots()
        if self.use_graphs and single:
            logits = self._step_graph(entries, lengths, slots, tables, device_tokens)
        else:
            batch, block_tables = pack_step(entries, lengths, slots, tables, self.device)
            if device_tokens is not None:
                batch.token_ids.copy_(device_tokens)
            self.storage.bind(block_tables)
            logits = self.model.forward(batch, self.storage)
        for e in entries:
            m.commit(e.request_id, len(e.tokens))
        return logits

    def _step_graph(self, entries, lengths, slots, tables, device_tokens=None):
        B = len(entries)
        rows = padded_batch(B)
        longest = max(lengths) + 1
        bucket = 256
        while bucket < longest:
            bucket *= 2
        bucket = min(bucket, self.max_request_tokens)
        graph = self._graphs.pop((rows, bucket), None)
        if graph is None:
            if len(self._graphs) >= self.max_graphs:       # drop the one used longest ago, once it is idle
                self._graphs.pop(next(iter(self._graphs))).retire(self.device)
            graph = _DecodeGraph(self, rows, bucket)
        self._graphs[(rows, bucket)] = graph                # most recently used last
        logits = graph.run(self, entries, lengths, slots, tables, device_tokens)
        wanted = [i for i, e in enumerate(entries) for _ in e.want]
        if wanted == list(range(B)):
            return logits if rows == B else logits.narrow(0, 0, B)
        index = torch.tensor(wanted, dtype=torch.long, device=self.device)
        return logits.index_select(0, index)

    def length(self, request_id):
        return self.manager.length(request_id) if self.manager.has(request_id) else 0

    def finish(self, request_id):
        """The request has ended; what it holds is given back."""
        if self.manager.has(request_id):
            self.manager.release(request_id)
