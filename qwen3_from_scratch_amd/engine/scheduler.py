"""The scheduler: which requests run in the next step, and with how many tokens.

It follows the reference's policy (src/qwen3_from_scratch/inference/scheduler.py):
decoding requests first, one token each, then portions of prompts under what is
left of the step's budgets of sequences and tokens (:48-57, :95-148); when pages
run out while decoding, the newest decoding request is preempted (:69-82).
Three things differ on purpose. A preempted request keeps the tokens it has
generated and, when it runs again, goes through prompt and generated tokens in
portions before it decodes on, so no token is produced twice (the reference
drops them, :155-162). Waiting requests are admitted in arrival order without
overtaking, and a preempted request returns to the front of the queue. And if
no request at all can advance because prompts in progress hold every page, the
newest of them is preempted, so that a step can always be made.

With the cache manager's prefix index on, a request that is admitted first takes
over the leading full blocks that the index already holds for its tokens
(the reference's `share_prefix`, scheduler.py:121-135) and starts its prompt
behind them; after every step the blocks a request has filled are registered. A
preempted request finds its own blocks again if nobody needed their pages meanwhile.
"""

from collections import deque
from dataclasses import dataclass, field
from enum import Enum

from ..cache import OutOfPages
from ..sampling import SamplingParams


class RequestStatus(Enum):
    WAITING = 0
    RUNNING = 1
    FINISHED = 2


@dataclass
class Request:
    request_id: object
    prompt: list
    params: SamplingParams = field(default_factory=SamplingParams)
    eos_ids: tuple = ()
    generated: list = field(default_factory=list)
    computed: int = 0              # tokens of prompt + generated whose keys are in the cache
    prefill_target: int = 0        # tokens to go through in portions before decoding (on)
    status: RequestStatus = RequestStatus.WAITING
    last_token_id: int = -1
    preemptions: int = 0
    blocks_offered: int = 0        # full blocks that the prefix index has been offered

    def __post_init__(self):
        self.prompt = list(self.prompt)
        self.prefill_target = len(self.prompt)

    @property
    def tokens(self):
        return self.prompt + self.generated

    @property
    def num_tokens(self):
        return len(self.prompt) + len(self.generated)

    @property
    def is_prefill(self):
        return self.computed < self.prefill_target


@dataclass
class Scheduled:
    request: Request
    num_tokens: int        # tokens of this step: request.tokens[computed : computed + num_tokens]
    samples: bool          # whether the step's last token yields the request's next token


class Scheduler:
    def __init__(self, manager, max_num_seqs, max_num_tokens, chunked_prefill_size,
                 max_len=None, release=None, portion_multiple=1):
        """`manager`: the cache manager (asked what fits; pages are taken by the
        step itself). `release(request_id)`: gives back what a request holds.
        `portion_multiple`: every portion of a prompt except its last is cut to a
        multiple of this many tokens (what the model's parts ask for); the
        reference has no counterpart."""
        if portion_multiple < 1 or portion_multiple > min(chunked_prefill_size, max_num_tokens):
            raise ValueError("portions must be multiples of %d tokens, which chunked_prefill_size (%d) and "
                             "max_num_tokens (%d) must allow" % (portion_multiple, chunked_prefill_size, max_num_tokens))
        self.portion_multiple = portion_multiple
        if max_num_seqs > manager.max_requests:
            raise ValueError("max_num_seqs (%d) exceeds the cache's request slots (%d)"
                             % (max_num_seqs, manager.max_requests))
        self.manager = manager
        self.max_num_seqs = max_num_seqs
        self.max_num_tokens = max_num_tokens
        self.chunked_prefill_size = chunked_prefill_size
        self.max_len = max_len
        self.release = release or (lambda rid: manager.release(rid) if manager.has(rid) else None)
        self.waiting = deque()
        self.running = deque()

    # ---- admission ----
    def add(self, request):
        """Queue a request. One that can never fit is refused here, rather than
        left to wait for ever (the reference returns False, scheduler.py:39-46)."""
        total = len(request.prompt) + request.params.max_new_tokens
        if not request.prompt:
            raise ValueError("request %r has an empty prompt" % (request.request_id,))
        if total > self.manager.capacity_tokens():
            raise ValueError("request %r needs %d tokens, the cache holds %d"
                             % (request.request_id, total, self.manager.capacity_tokens()))
        if self.max_len is not None and total > self.max_len:
            raise ValueError("request %r needs %d positions, the limit is %d"
                             % (request.request_id, total, self.max_len))
        request.status = RequestStatus.WAITING
        self.waiting.append(request)

    def has_work(self):
        return bool(self.waiting or self.running)

    def abort(self, request):
        """Take a request out, wherever it is; what it holds is given back."""
        if request in self.waiting:
            self.waiting.remove(request)
        if request in self.running:
            self.running.remove(request)
        self.release(request.request_id)
        request.status = RequestStatus.FINISHED

    # ---- one step's plan ----
    def schedule(self):
        while True:
            spare = [0] * len(self.manager.groups)
            decodes = self._schedule_decode(spare)
            prefills = self._schedule_prefill(self.max_num_seqs - len(decodes),
                                              self.max_num_tokens - len(decodes), spare)
            plan = decodes + prefills
            if plan or not self.running:
                if not plan and self.waiting:
                    raise RuntimeError("no request can be scheduled although the cache is empty")
                return plan
            # requests hold pages yet none can advance: take the newest one's pages away
            self._preempt(self.running[-1])

    def _schedule_decode(self, spare):
        budget = min(self.max_num_seqs, self.max_num_tokens)
        prefilling = [r for r in self.running if r.is_prefill]
        ready = deque(r for r in self.running if not r.is_prefill)
        scheduled = []
        while ready and len(scheduled) < budget:
            req = ready.popleft()
            fits = self.manager.can_grow(req.request_id, 1, spare)
            while not fits:
                if ready:
                    self._preempt(ready.pop(), keep_in_running=False)   # the newest wastes least
                    fits = self.manager.can_grow(req.request_id, 1, spare)
                else:
                    self._preempt(req, keep_in_running=False)
                    break
            if fits:
                scheduled.append(Scheduled(req, 1, True))
        # those skipped for the budget go first next time
        self.running = deque(prefilling + list(ready) + [s.request for s in scheduled])
        return scheduled

    def _portion(self, req, room):
        """How many of the request's tokens go into a step with `room` left in its token budget:
        all that are left, or as many as the limits allow, cut so that the portion ends at a
        multiple of the portion multiple, counted from the request's first token (a request that
        starts behind shared pages or again after a preemption keeps the same cuts)."""
        left = req.prefill_target - req.computed
        n = min(left, self.chunked_prefill_size, room)
        if n < left:
            n -= (req.computed + n) % self.portion_multiple
        return n

    def _schedule_prefill(self, max_seqs, max_tokens, spare):
        scheduled = []
        tokens = 0
        for req in [r for r in self.running if r.is_prefill]:
            if len(scheduled) >= max_seqs or tokens >= max_tokens:
                break
            n = self._portion(req, max_tokens - tokens)
            if n <= 0 or not self.manager.can_grow(req.request_id, n, spare):
                continue
            scheduled.append(Scheduled(req, n, req.computed + n == req.num_tokens))
            tokens += n
        while self.waiting and len(scheduled) < max_seqs and tokens < max_tokens \
                and len(self.running) < self.max_num_seqs:
            req = self.waiting[0]
            shared = self._share_prefix(req)
            n = self._portion(req, max_tokens - tokens)
            if n <= 0 or not self.manager.can_grow(req.request_id, n, spare):
                if shared:                              # it waits on: what it took over goes back
                    self.manager.prefix_hits -= req.computed
                    self.manager.release(req.request_id)
                    req.computed = req.blocks_offered = 0
                break                                   # no overtaking
            self.waiting.popleft()
            req.status = RequestStatus.RUNNING
            self.running.append(req)
            scheduled.append(Scheduled(req, n, req.computed + n == req.num_tokens))
            tokens += n
        return scheduled

    def _share_prefix(self, req):
        """A waiting request that holds nothing yet is admitted to the cache and
        takes over what the prefix index has of its tokens. True if it did."""
        m = self.manager
        if not getattr(m, "prefix_cache", False) or req.computed or m.has(req.request_id):
            return False
        try:
            m.admit(req.request_id)
        except OutOfPages:
            return False                                # no slot: can_grow says so next
        req.computed = m.share_prefix(req.request_id, req.tokens[:req.prefill_target])
        req.blocks_offered = req.computed // m.page_size
        if not req.computed:
            m.release(req.request_id)                   # nothing found: the step admits it as usual
            return False
        return True

    def _preempt(self, req, keep_in_running=True):
        self.release(req.request_id)
        if req in self.running:
            self.running.remove(req)
        req.computed = 0
        req.blocks_offered = 0
        req.prefill_target = req.num_tokens
        req.status = RequestStatus.WAITING
        req.preemptions += 1
        self.waiting.appendleft(req)

    # ---- after the step ----
    def after_step(self, plan, sampled):
        """`sampled`: one token per plan entry that samples, in plan order.
        Returns the requests that finished."""
        finished = []
        it = iter(sampled)
        for s in plan:
            req = s.request
            req.computed += s.num_tokens
            full = req.computed // self.manager.page_size
            if full > req.blocks_offered and getattr(self.manager, "prefix_cache", False) \
                    and self.manager.has(req.request_id):
                self.manager.register_prefix(req.request_id, req.tokens)
                req.blocks_offered = full
            if not s.samples:
                continue
            token = int(next(it))
            req.generated.append(token)
            req.last_token_id = token
            hit_eos = (not req.params.ignore_eos) and token in req.eos_ids
            if hit_eos or len(req.generated) >= req.params.max_new_tokens:
                req.status = RequestStatus.FINISHED
                if req in self.running:
                    self.running.remove(req)
                self.release(req.request_id)
                finished.append(req)
        return finished
