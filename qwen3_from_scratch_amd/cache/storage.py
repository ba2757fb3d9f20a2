"""The device memory behind the cache manager's page numbers and slots."""

from dataclasses import dataclass, field

import torch


@dataclass
class LayerCacheView:
    """What one mixer sees of the cache in one step."""

    paged: dict = field(default_factory=dict)   # name of a PagedTensor -> (pages, *page shape)
    block_table: torch.Tensor = None            # int32 (B, W), this step's requests in batch order
    writes: bool = True
    state: torch.Tensor = None                  # (slots, *state_shape); index with batch.state_slots


class CacheStorage:
    """Per paged group, one tensor for each `PagedTensor` its mixers declared: (planes, pages,
    *page shape) in the declared dtype or the activation dtype; the in-page layout is the
    mixer's own (see `PagedTensor`), this class only allocates what is declared. Per state
    group one tensor (planes, slots, *shape), zeroed per slot at admission. Every group has one
    page, and every state group one slot, more than the manager hands out (`spare_page`,
    `spare_slot`): rows that only fill a batch up to a size a captured graph exists for write
    there."""

    def __init__(self, manager, act_dtype, device):
        self.manager = manager
        self.device = torch.device(device)
        self.paged = []                                # per group {name: tensor}
        for grp in manager.groups:
            tensors = {}
            for t in grp.tensors:
                shape = (len(grp.planes), grp.pool.num_pages + 1) + t.page_shape(manager.page_size)
                tensors[t.name] = torch.zeros(shape, dtype=t.dtype or act_dtype, device=self.device)
            self.paged.append(tensors)
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
        tensors = [t for group in self.paged for t in group.values()] + self.states
        return sum(t.numel() * t.element_size() for t in tensors)

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
            view.paged = {name: tensor[local] for name, tensor in self.paged[g].items()}
            view.block_table = self._block_tables[g]
        s = m.state_group_of_plane[plane]
        if s >= 0:
            local = m.state_groups[s].planes.index(plane)
            view.state = self.states[s][local]
        return view
