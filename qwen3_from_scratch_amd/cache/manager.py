"""The cache manager: which pages and which state slot every live request holds.

Layers are put in groups by what their mixers keep (`CacheNeed`): layers that
keep the same paged tensors for all tokens share a group, layers that keep a
window of them form another, and so on. A group has a page pool of
its own and, per request, one block table that serves all its layers: page p of
a group exists once in each of the group's layers' planes. A request's pages
go back to the pool when it ends, and, in a windowed group, as soon as every
position a page covers lies behind the window. Mixers that keep a state of
fixed size get one slot per live request, the same slot number in all such
groups; it is handed out at admission and taken back when the request ends.

The reference has one homogeneous pool with reference counts for a prefix
index (src/qwen3_from_scratch/inference/block_manager.py:26-138); the
arithmetic of `pages_missing` is its `can_allocate` (:90-95).

The prefix index (off unless asked for). Full blocks of a request's tokens are
registered as nodes of a tree: a node is (its parent node, the block's tokens)
and owns one page in every group. A new request walks the tree from the root
with its own tokens and takes a reference to every node it meets, instead of
computing those blocks again; it always keeps at least one token to compute.
Where the reference hashes each block by its own tokens alone and compares
token lists (block_manager.py:45-64), the key here is the exact pair (parent,
tokens), so two different prefixes never meet in one node. The reference
forgets a block when its last holder ends (:129-138); here a node without
holders stays, and its pages count as free: when a pool runs dry the node
left longest ago is forgotten and its pages are handed out. Only models whose
groups all keep every key, and that keep no per-request state, can share
prefixes (a window gives pages back while the request lives, and a state
cannot be rebuilt from pages); for others the index stays off.
"""

from collections import OrderedDict
from dataclasses import dataclass, field

from .pages import OutOfPages, PagePool


@dataclass
class _Group:
    tensors: tuple                       # the PagedTensors that every layer of the group keeps
    window: int
    planes: list
    pool: PagePool


@dataclass
class _StateGroup:
    shape: tuple
    dtype: object
    planes: list


@dataclass
class _Held:
    length: int = 0                      # tokens whose keys are in the cache
    reserved: int = 0                    # tokens beyond `length` that pages are held for
    tables: list = field(default_factory=list)   # per group: page of each block, -1 once given back
    slot: int = -1
    admission: int = 0                   # which admission of the manager's this is
    # the prefix index's view of the first blocks: the node whose page the block is, or -1 for a
    # page of the request's own (a block that another request had registered first)
    nodes: list = field(default_factory=list)
    chain: int = 0                               # the node that stands for the content of those blocks (0: none)


@dataclass
class _Node:
    parent: int
    tokens: tuple
    pages: list                          # one page per group
    holders: int = 0


class CacheManager:
    def __init__(self, needs, page_size, num_pages, max_requests, prefix_cache=False):
        """`needs`: one CacheNeed (or None) per cache plane of the model.
        `num_pages`: pages in every group's pool. `max_requests`: state slots.
        `prefix_cache`: keep the prefix index, if the model's groups allow it."""
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        self.page_size = page_size
        self.max_requests = max_requests
        self.groups = []
        self.state_groups = []
        self.group_of_plane = []
        self.state_group_of_plane = []
        for plane, need in enumerate(needs):
            g = s = -1
            if need is not None and need.paged:
                key = (tuple(need.paged), need.window)
                for i, grp in enumerate(self.groups):
                    if (grp.tensors, grp.window) == key:
                        g = i
                if g < 0:
                    self.groups.append(_Group(*key, planes=[], pool=PagePool(num_pages)))
                    g = len(self.groups) - 1
                self.groups[g].planes.append(plane)
            if need is not None and need.has_state:
                key = (tuple(need.state_shape), need.state_dtype)
                for i, grp in enumerate(self.state_groups):
                    if (grp.shape, grp.dtype) == key:
                        s = i
                if s < 0:
                    self.state_groups.append(_StateGroup(*key, planes=[]))
                    s = len(self.state_groups) - 1
                self.state_groups[s].planes.append(plane)
            self.group_of_plane.append(g)
            self.state_group_of_plane.append(s)
        self._slots = list(range(max_requests - 1, -1, -1))
        self._requests = {}
        self._admissions = 0
        self.fresh_slots = []     # slots handed out since the storage last cleared them
        self.prefix_cache = bool(prefix_cache) and bool(self.groups) and not self.state_groups \
            and all(g.window <= 0 for g in self.groups)
        self._nodes = {}                  # node id -> _Node
        self._index = {}                  # (parent id, tokens of the block) -> node id
        self._idle = OrderedDict()        # nodes without holders, the one left longest ago first
        self._next_node = 1               # 0 is the root
        self.prefix_hits = 0              # tokens that requests did not have to compute

    # ---- requests ----
    def has(self, request_id):
        return request_id in self._requests

    def live(self):
        return list(self._requests)

    def length(self, request_id):
        return self._requests[request_id].length

    def slot(self, request_id):
        return self._requests[request_id].slot

    def admission(self, request_id):
        """A number that differs between two admissions of the same request id:
        who remembers a request's pages checks it before trusting them."""
        return self._requests[request_id].admission

    def admit(self, request_id):
        if request_id in self._requests:
            raise KeyError("request %r is already live" % (request_id,))
        if not self._slots:
            raise OutOfPages("all %d request slots are taken" % self.max_requests)
        self._admissions += 1
        held = _Held(tables=[[] for _ in self.groups], slot=self._slots.pop(), admission=self._admissions)
        self._requests[request_id] = held
        self.fresh_slots.append(held.slot)
        return held.slot

    # ---- growth ----
    def _blocks_for(self, tokens):
        return -(-tokens // self.page_size)

    def pages_missing(self, request_id, new_tokens):
        """Per group, the pages still to be taken before `new_tokens` more can be written."""
        held = self._requests.get(request_id)
        length = held.length if held else 0
        target = self._blocks_for(length + new_tokens)
        return [target - (len(held.tables[g]) if held else 0) for g in range(len(self.groups))]

    def can_grow(self, request_id, new_tokens, spare=None):
        """True if every group's pool can cover `new_tokens` more for the request.
        `spare`, if given, is a per-group count of pages already promised to
        others in this step; it is updated when the answer is True."""
        if request_id not in self._requests and not self._slots:
            return False
        missing = self.pages_missing(request_id, new_tokens)
        taken = spare if spare is not None else [0] * len(self.groups)
        for g, grp in enumerate(self.groups):
            if max(0, missing[g]) + taken[g] > grp.pool.num_free + len(self._idle):
                return False
        if spare is not None:
            for g in range(len(self.groups)):
                spare[g] += max(0, missing[g])
        return True

    def reserve(self, request_id, new_tokens):
        """Take the pages that positions length .. length + new_tokens - 1 need.
        Either all groups get theirs or nothing changes."""
        held = self._requests[request_id]
        missing = self.pages_missing(request_id, new_tokens)
        for g, grp in enumerate(self.groups):
            if missing[g] > grp.pool.num_free + len(self._idle):
                raise OutOfPages(
                    "request %r needs %d more pages of group %d, %d are free"
                    % (request_id, missing[g], g, grp.pool.num_free + len(self._idle)))
        for g, grp in enumerate(self.groups):
            for _ in range(max(0, missing[g])):
                while grp.pool.num_free == 0:
                    self._forget_oldest()
                held.tables[g].append(grp.pool.take())
        held.reserved = max(held.reserved, new_tokens)

    def commit(self, request_id, new_tokens):
        """The step wrote `new_tokens` more positions. Pages of windowed groups
        that no later query can see are given back."""
        held = self._requests[request_id]
        if new_tokens > held.reserved:
            raise RuntimeError("commit of %d tokens, only %d reserved" % (new_tokens, held.reserved))
        held.length += new_tokens
        held.reserved = 0
        for g, grp in enumerate(self.groups):
            if grp.window <= 0:
                continue
            # the next query sits at position >= length and sees keys > its position - window
            first_needed = held.length - grp.window + 1
            dead_blocks = max(0, first_needed) // self.page_size
            table = held.tables[g]
            for b in range(min(dead_blocks, len(table))):
                if table[b] >= 0:
                    grp.pool.give(table[b])
                    table[b] = -1

    def release(self, request_id):
        """The request has ended: everything it holds goes back. Blocks that are
        nodes of the prefix index lose a holder; their pages stay with the node."""
        held = self._requests.pop(request_id)
        for g, grp in enumerate(self.groups):
            for b, page in enumerate(held.tables[g]):
                if page >= 0 and not (b < len(held.nodes) and held.nodes[b] >= 0):
                    grp.pool.give(page)
        for node_id in reversed(held.nodes):          # the deepest is forgotten first
            if node_id < 0:
                continue
            node = self._nodes[node_id]
            node.holders -= 1
            if node.holders == 0:
                self._idle[node_id] = None
        self._slots.append(held.slot)

    # ---- the prefix index ----
    def share_prefix(self, request_id, tokens):
        """For a request that holds nothing yet: take a reference to every
        leading full block of `tokens` that the index knows, up to the last
        block that still leaves a token to compute. Returns the number of
        tokens the request now holds."""
        held = self._requests[request_id]
        if not self.prefix_cache or held.length or held.reserved or any(held.tables):
            return held.length
        ps, parent = self.page_size, 0
        for b in range((len(tokens) - 1) // ps):
            node_id = self._index.get((parent, tuple(tokens[b * ps:(b + 1) * ps])))
            if node_id is None:
                break
            node = self._nodes[node_id]
            if node.holders == 0:
                del self._idle[node_id]
            node.holders += 1
            held.nodes.append(node_id)
            for g in range(len(self.groups)):
                held.tables[g].append(node.pages[g])
            parent = node_id
        held.chain = parent
        held.length = len(held.nodes) * ps
        self.prefix_hits += held.length
        return held.length

    def register_prefix(self, request_id, tokens):
        """`tokens`: the request's tokens from its first on, at least as many as
        it holds. Its full blocks that the index has not seen become nodes. A
        block that another request has registered meanwhile stays this
        request's own page; the blocks after it hang below that other node."""
        if not self.prefix_cache:
            return
        held = self._requests[request_id]
        ps = self.page_size
        full = min(held.length, len(tokens)) // ps
        for b in range(len(held.nodes), full):
            key = (held.chain, tuple(tokens[b * ps:(b + 1) * ps]))
            known = self._index.get(key)
            if known is not None:
                held.nodes.append(-1)
                held.chain = known
                continue
            node_id = self._next_node
            self._next_node += 1
            self._nodes[node_id] = _Node(key[0], key[1], [held.tables[g][b] for g in range(len(self.groups))], 1)
            self._index[key] = node_id
            held.nodes.append(node_id)
            held.chain = node_id

    def _forget_oldest(self):
        if not self._idle:
            raise OutOfPages("the page pool is empty")
        node_id, _ = self._idle.popitem(last=False)
        node = self._nodes.pop(node_id)
        del self._index[(node.parent, node.tokens)]
        for g, grp in enumerate(self.groups):
            grp.pool.give(node.pages[g])

    def forget_prefixes(self):
        """Drop every node that has no holder (their pages go back to the pools)."""
        while self._idle:
            self._forget_oldest()

    # ---- views ----
    def block_table(self, request_id, group):
        return self._requests[request_id].tables[group]

    def num_free(self, group=0):
        """Pages that can be handed out: the pool's, and those of index nodes nobody holds."""
        return self.groups[group].pool.num_free + len(self._idle)

    def num_pages(self, group=0):
        return self.groups[group].pool.num_pages

    def table_width(self, group, tokens):
        """Entries a block table of `group` needs for a request of `tokens` tokens. A windowed
        group's table is as long as any other's: a block keeps its place in the table when its
        page goes back (the entry turns -1), so kernels find a key's page by its position alone."""
        if not 0 <= group < len(self.groups):
            raise IndexError("no group %d" % group)
        return -(-tokens // self.page_size)

    def capacity_tokens(self):
        """Tokens one request can hold at most (bounded by the smallest pool)."""
        if not self.groups:
            return 1 << 62
        return min(g.pool.num_pages for g in self.groups) * self.page_size

    def audit(self):
        """Every page is free, held by exactly one request, or owned by exactly
        one index node whose holders are the requests that list it; slots likewise."""
        holders = {}
        for rid, held in self._requests.items():
            for b, node_id in enumerate(held.nodes):
                if node_id < 0:
                    continue
                holders[node_id] = holders.get(node_id, 0) + 1
                node = self._nodes.get(node_id)
                if node is None:
                    raise AssertionError("request %r lists node %d, which is forgotten" % (rid, node_id))
                for g in range(len(self.groups)):
                    if held.tables[g][b] != node.pages[g]:
                        raise AssertionError("request %r block %d is not its node's page" % (rid, b))
        for node_id, node in self._nodes.items():
            if node.holders != holders.get(node_id, 0):
                raise AssertionError("node %d counts %d holders, %d requests list it"
                                     % (node_id, node.holders, holders.get(node_id, 0)))
            if (node.holders == 0) != (node_id in self._idle):
                raise AssertionError("node %d is idle and held at once, or neither" % node_id)
            if self._index.get((node.parent, node.tokens)) != node_id:
                raise AssertionError("node %d is not where the index looks for it" % node_id)
        if len(self._index) != len(self._nodes):
            raise AssertionError("the index and the nodes disagree")
        for g, grp in enumerate(self.groups):
            seen = set()
            owners = [("node %d" % i, [n.pages[g]]) for i, n in self._nodes.items()]
            owners += [("request %r" % (rid,), [page for b, page in enumerate(held.tables[g])
                                               if not (b < len(held.nodes) and held.nodes[b] >= 0)])
                       for rid, held in self._requests.items()]
            for who, pages in owners:
                for page in pages:
                    if page < 0:
                        continue
                    if page in seen:
                        raise AssertionError("page %d of group %d is held twice" % (page, g))
                    if not grp.pool.is_held(page):
                        raise AssertionError("page %d of group %d is held by %s but marked free" % (page, g, who))
                    seen.add(page)
            if len(seen) + grp.pool.num_free != grp.pool.num_pages:
                raise AssertionError(
                    "group %d: %d held + %d free != %d pages"
                    % (g, len(seen), grp.pool.num_free, grp.pool.num_pages))
        slots = [h.slot for h in self._requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._slots):
            raise AssertionError("a request slot is held twice")
        if len(slots) + len(self._slots) != self.max_requests:
            raise AssertionError("a request slot is lost")
