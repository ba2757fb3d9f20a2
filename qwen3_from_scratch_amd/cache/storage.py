"""The device memory behind the cache manager's page numbers and slots."""

from dataclasses import dataclass

import torch


@dataclass
class LayerCacheView:
    """What one mixer sees of the cache in one step."""

    keys: torch.Tensor = None          # (pages, kv_heads, page_size, head_dim)
    values: torch.Tensor = None        # (pages, kv_heads, head_dim, page_size)
    block_table: torch.Tensor = None   # int32 (B, W), this step's requests in batch order
    writes: bool = True
    state: torch.Tensor = None         # (slots, *state_shape); index with batch.state_slots


class CacheStorage:
    """Per paged group two tensors in the activation dtype: keys
    (planes, pages, kv_heads, page_size, head_dim) and values
    (planes, pages, kv_heads, head_dim, page_size). Within a page one head's
    keys are contiguous, so a workgroup that serves one key head streams
    page_size * head_dim elements at a time; values are kept transposed within
    the page, so that the keys a matrix-core lane multiplies together lie side
    by side in memory and need no transposition on the way to the registers.
    Per state group one tensor (planes, slots, *shape), zeroed per slot at
    admission. Every group has one page, and every state group one slot, more
    than the manager hands out (`spare_page`, `spare_slot`): rows that only
    fill a batch up to a size a captured graph exists for write there."""

    def __init__(self, manager, act_dtype, device):
        self.manager = manager
        self.device = torch.device(device)
        self.keys, self.values = [], []
        for grp in manager.groups:
            shape = (len(grp.planes), grp.pool.num_pages + 1, grp.kv_heads, manager.page_size, grp.head_dim)
            self.keys.append(torch.zeros(shape, dtype=act_dtype, device=self.device))
            self.values.append(torch.zeros(shape[:3] + (grp.head_dim, manager.page_size),
                                           dtype=act_dtype, device=self.device))
        self.states = []
        for grp in manager.state_groups:
            self.states.append(torch.zeros(
                (len(grp.planes), manager.max_requests + 1) + tuple(grp.shape),
                dtype=grp.dtype, device=self.device))
        self._block_tables = None

    def spare_page(self, group):
        return self.manager.groups[group].pool.num_pages

    @property
    def spare_slot(self):
        return self.manager.max_requests

    def bytes(self):
        return sum(t.numel() * t.element_size() for t in self.keys + self.values + self.states)

    def clear_fresh_slots(self):
        fresh, self.manager.fresh_slots = self.manager.fresh_slots, []
        if fresh and self.states:
            index = torch.tensor(fresh, dtype=torch.long, device=self.device)
            for t in self.states:
                t[:, index] = 0

    def bind(self, block_tables):
        """`block_tables`: per paged group the step's int32 (B, W) device tensor."""
        self._block_tables = block_tables

    def view(self, plane, writes=True):
        m = self.manager
        view = LayerCacheView(writes=writes)
        g = m.group_of_plane[plane]
        if g >= 0:
            local = m.groups[g].planes.index(plane)
            view.keys = self.keys[g][local]
            view.values = self.values[g][local]
            view.block_table = self._block_tables[g]
        s = m.state_group_of_plane[plane]
        if s >= 0:
            local = m.state_groups[s].planes.index(plane)
            view.state = self.states[s][local]
        return view
