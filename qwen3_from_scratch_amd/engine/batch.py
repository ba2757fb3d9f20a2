"""One step's batch: the tokens it brings and where they sit."""

from dataclasses import dataclass, field

import numpy as np
import torch


@dataclass
class StepEntry:
    """A request's next tokens in this step and the places among them (0-based
    indices into `tokens`) whose logits are wanted."""

    request_id: object
    tokens: list
    want: list = field(default_factory=list)


@dataclass
class StepBatch:
    """Device tensors (int32) and host numbers that describe the packed batch.

    Rows of all entries are packed on one token axis without padding, in the
    order of the entries (src/qwen3_from_scratch/inference/model_worker.py:177-210
    builds the same quantities as separate uploads and a global context).
    """

    num_tokens: int
    num_seqs: int
    token_ids: torch.Tensor        # (T,)
    positions: torch.Tensor        # (T,) absolute position of each token in its request
    seq_index: torch.Tensor        # (T,) which entry a token belongs to
    cu_seqlens_q: torch.Tensor     # (B+1,) prefix sums of tokens per entry
    kv_lens: torch.Tensor          # (B,) keys visible after this step's write
    state_slots: torch.Tensor      # (B,) per-request slot of fixed-size state
    logits_rows: torch.Tensor      # (R,) packed rows whose logits are wanted
    max_q_len: int
    min_q_len: int
    max_kv_len: int
    max_kv_len_portions: int       # the same among the entries that bring more than one token
    q_lens: list                   # host copies
    kv_lens_host: list


@dataclass
class PackedLayout:
    """Where each part of a step's description lies in its one int32 buffer, in
    words: `pack_step` writes by it and whoever patches a packed buffer in place
    (a graph's fixed buffer between replays) finds the parts by it."""

    tokens: slice
    positions: slice
    seq_index: slice
    cu_seqlens_q: slice
    kv_lens: slice
    state_slots: slice
    logits_rows: slice
    tables: list              # per group (slice, width)
    total: int


def packed_layout(B, T, R, widths):
    """The layout of a step of B entries, T tokens and R wanted rows whose
    block tables are `widths[g]` entries wide in group g."""
    at = 0
    parts = []
    for n in (T, T, T, B + 1, B, B, R):
        parts.append(slice(at, at + n))
        at += n
    tables = []
    for w in widths:
        tables.append((slice(at, at + B * w), w))
        at += B * w
    return PackedLayout(*parts, tables=tables, total=at)


def packed_size(B, T, R, widths):
    return packed_layout(B, T, R, widths).total


def pack_step(entries, lengths, slots, tables_per_group, device, min_table_width=1, fixed_widths=None,
              buffers=None, all_rows=False):
    """Build the batch on the host and move it to the device in one copy.

    `lengths[i]`: tokens entry i's request already has in the cache.
    `tables_per_group[g][i]`: the request's page list in group g (-1 = given back).
    `fixed_widths`: block-table widths to use instead of the longest list's.
    `buffers`: (pinned host int32 tensor, device int32 tensor) to pack into, so
    that the batch lives at the same addresses every step (for graph replay);
    with None for the device tensor the batch stays in the host tensor.
    `all_rows`: ask for logits at every packed row, whatever `want` says.
    Returns (StepBatch, [block table per group]).
    """
    B = len(entries)
    q_lens = [len(e.tokens) for e in entries]
    T = sum(q_lens)
    kv = [lengths[i] + q_lens[i] for i in range(B)]
    rows = []
    offset = 0
    for i, e in enumerate(entries):
        for w in e.want:
            if not (0 <= w < q_lens[i]):
                raise ValueError("request %r wants place %d of %d tokens" % (e.request_id, w, q_lens[i]))
            rows.append(offset + w)
        offset += q_lens[i]
    if all_rows:
        rows = list(range(T))
    R = len(rows)
    if fixed_widths is not None:
        widths = list(fixed_widths)
        for tables, w in zip(tables_per_group, widths):
            if any(len(t) > w for t in tables):
                raise ValueError("a block table is wider than the fixed width %d" % w)
    else:
        widths = [max([min_table_width] + [len(t) for t in tables]) for tables in tables_per_group]
    lay = packed_layout(B, T, R, widths)
    total = lay.total
    if buffers is not None:
        host_t, dev_t = buffers
        if host_t.numel() < total:
            raise ValueError("the packing buffer is too small")
        host = host_t.numpy()
    else:
        host = np.empty(total, dtype=np.int32)
    host[lay.tokens] = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries]) if T else 0
    host[lay.positions] = np.concatenate([np.arange(lengths[i], kv[i]) for i in range(B)]) if T else 0
    host[lay.seq_index] = np.repeat(np.arange(B), q_lens) if T else 0
    host[lay.cu_seqlens_q] = np.concatenate([[0], np.cumsum(q_lens)])
    host[lay.kv_lens] = kv
    host[lay.state_slots] = slots
    host[lay.logits_rows] = rows
    for tables, (sl, w) in zip(tables_per_group, lay.tables):
        flat = host[sl].reshape(B, w)
        flat[:] = -1
        for i, t in enumerate(tables):
            flat[i, :len(t)] = t
    if buffers is not None:
        if dev_t is not None:
            dev_t[:total].copy_(host_t[:total], non_blocking=True)
        dev = dev_t if dev_t is not None else host_t
    else:
        dev = torch.from_numpy(host)
        if torch.device(device).type == "cuda":
            dev = dev.pin_memory().to(device, non_blocking=True)
    s_tok, s_pos, s_seq, s_cu, s_kv, s_slot, s_rows, s_tables = (
        lay.tokens, lay.positions, lay.seq_index, lay.cu_seqlens_q, lay.kv_lens, lay.state_slots, lay.logits_rows,
        lay.tables)
    batch = StepBatch(
        num_tokens=T, num_seqs=B,
        token_ids=dev[s_tok], positions=dev[s_pos], seq_index=dev[s_seq],
        cu_seqlens_q=dev[s_cu], kv_lens=dev[s_kv], state_slots=dev[s_slot], logits_rows=dev[s_rows],
        max_q_len=max(q_lens) if q_lens else 0, min_q_len=min(q_lens) if q_lens else 0,
        max_kv_len=max(kv) if kv else 0,
        max_kv_len_portions=max([n for n, q in zip(kv, q_lens) if q > 1] or [0]),
        q_lens=q_lens, kv_lens_host=kv,
    )
    block_tables = [dev[sl].view(B, w) for sl, w in s_tables]
    return batch, block_tables
