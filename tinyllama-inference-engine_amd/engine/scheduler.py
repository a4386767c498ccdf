"""The scheduler: which requests run in the next step, and with how many tokens each.

reference: `Engine` in app/server.cpp.  It admits queued requests first come first served while a
cache slot is free (`Admit`, :360-387), picks up to four rows per step, requests that decode
before requests still in their prompt, from a rotating cursor (`SelectBatch`, :389-408), feeds one
token per row (:432-444), samples when a row was its prompt's last token or a decoded one
(:459-465), and finishes a request when it has `max_tokens` outputs (:468-469; no end-of-sequence
check).  A slot there is a whole-length reservation, so memory cannot run out mid-request.

Here a step has a budget of tokens and of sequences.  Decoding requests come first, one token
each (from a rotating cursor when they exceed the budget); what is left of the budget goes to
prompts, cut into portions.  Pages are taken as a request grows, so they can run out:

  * a request whose prompt plus outputs could never fit the pool, or the model's positions, is
    refused when it is added (`out_of_memory` / `out_of_bounds`; app/reference_cli.cpp:72-75);
  * when a decoding request finds no free page, the request admitted last is preempted: its
    pages and slot are given back and it returns to the front of the queue, to be recomputed
    from its prompt and the tokens it has generated so far (they are kept);  this repeats until
    the step fits;  the choice is deterministic;
  * a prompt portion is cut down to the pages that are free, and waits when none are;
  * a waiting request (new, or preempted) is admitted beside running ones only when the pool has room
    for everything it brings (its prompt and what it has generated so far) after what the running
    requests still need to get through their own tokens, and a page of growth for each of them: a
    request admitted for a first portion that then fights the others for the rest is preempted and
    recomputed again and again when requests outnumber the pool several times (64 requests of up to
    2300 positions on a pool for a fifth of them: 415 preemptions and 31 thousand tokens/s that way,
    against the 107 thousand of an ample pool).  `admit_partial=True` admits as soon as a first
    portion fits.

The scheduler owns no device memory and calls no kernel: it plans with the cache manager's
counts, and the engine loop runs what it plans.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Hashable

from ..cache.manager import CacheManager
from ..errors import invalid_argument, out_of_bounds, out_of_memory


@dataclass
class SamplingParams:
    """Names as the reference's request options (app/server.cpp:601-613): max_tokens,
    temperature (0 = greedy), top_p in (0, 1]; the seed is the request's own."""
    max_tokens: int = 16
    temperature: float = 0.0
    top_p: float = 1.0
    seed: int = 0
    stop_on_eos: bool = False

    def validate(self) -> None:
        if self.max_tokens < 1:
            raise invalid_argument("max_tokens must be an integer >= 1")
        if not self.temperature >= 0.0:
            raise invalid_argument("temperature must be >= 0")
        if not 0.0 < self.top_p <= 1.0:
            raise invalid_argument("top_p must be in (0, 1]")


PENDING = -1        # in a request's generated tokens: sampled, but not yet read from the device


@dataclass
class Request:
    id: Hashable
    prompt: list[int]
    params: SamplingParams
    generated: list[int] = field(default_factory=list)
    state: str = "waiting"            # waiting, running, finished
    finish_reason: str | None = None  # length, eos, aborted
    computed: int = 0                 # tokens of prompt + generated whose keys are in the cache
    order: int = 0                    # admission order (larger = admitted later)
    preemptions: int = 0

    @property
    def tokens(self) -> list[int]:
        return self.prompt + self.generated

    @property
    def total(self) -> int:
        """How many tokens the request has: prompt and generated."""
        return len(self.prompt) + len(self.generated)

    def token_slice(self, first: int, count: int) -> list[int]:
        """tokens[first : first + count] without joining the two lists."""
        split = len(self.prompt)
        if first + count <= split:
            return self.prompt[first:first + count]
        if first >= split:
            return self.generated[first - split:first - split + count]
        return self.prompt[first:] + self.generated[:first + count - split]

    @property
    def pending(self) -> bool:
        """The last generated token has been sampled but is not on the host yet."""
        return bool(self.generated) and self.generated[-1] == PENDING

    @property
    def remaining(self) -> int:
        return len(self.prompt) + len(self.generated) - self.computed


@dataclass
class Scheduled:
    request: Request
    first: int          # index into request.tokens of the first token this step runs
    count: int
    samples: bool       # the portion reaches the end of the known tokens: its last logits are sampled


class Scheduler:
    def __init__(self, cache: CacheManager, max_tokens_per_step: int = 2048, max_seqs_per_step: int = 64,
                 chunk_size: int | None = None, max_positions: int | None = None, eos_token_id: int = -1,
                 prompt_tokens_beside_decodes: int | None = None, admit_partial: bool = False):
        """admit_partial: admit a waiting request beside running ones as soon as pages for a first
        portion of it are free (by default only when all it brings fits, see above).
        prompt_tokens_beside_decodes: in a step that holds decoding requests, prompts get at most
        this many tokens in all (None: whatever the budget leaves).  A step's time grows with its
        prompt tokens, and every decoding request of the step waits for it: the cap trades the
        prompts' throughput for the decoding requests' time between tokens (the reference's steps
        hold one token per row, prompt rows too: app/server.cpp:389-408,432-444)."""
        if max_tokens_per_step < 1 or max_seqs_per_step < 1:
            raise invalid_argument("the step budgets must be positive")
        if prompt_tokens_beside_decodes is not None and prompt_tokens_beside_decodes < 1:
            raise invalid_argument("prompts need at least one token a step beside decoding requests")
        self.prompt_tokens_beside_decodes = prompt_tokens_beside_decodes
        self.admit_partial = admit_partial
        self.cache = cache
        self.max_tokens_per_step = max_tokens_per_step
        self.max_seqs_per_step = max_seqs_per_step
        self.chunk_size = chunk_size or max_tokens_per_step
        self.max_positions = max_positions
        self.eos_token_id = eos_token_id
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []
        self.finished: list[Request] = []
        self._admitted = 0
        self._cursor = 0
        self.stats = {"steps": 0, "prefill_tokens": 0, "decode_tokens": 0, "preemptions": 0}

    # ---- requests in ---------------------------------------------------------------------------
    def add(self, request: Request) -> None:
        request.params.validate()
        if not request.prompt:
            raise invalid_argument("a request needs a prompt of at least one token")
        total = len(request.prompt) + request.params.max_tokens
        # the last sampled token is never fed back, so it needs no position
        if self.max_positions is not None and total > self.max_positions:
            raise out_of_bounds("prompt plus output exceeds context length")
        capacity = min(group.allocator.num_pages for group in self.cache.groups) * self.cache.page_size \
            if self.cache.groups else total
        if total - 1 > capacity:
            raise out_of_memory(f"prompt plus output needs {total - 1} cached positions, the pool holds {capacity}")
        request.state = "waiting"
        self.waiting.append(request)

    def abort(self, request_id: Hashable) -> bool:
        for request in list(self.running) + list(self.waiting):
            if request.id == request_id:
                self._finish(request, "aborted")
                return True
        return False

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- planning a step -------------------------------------------------------------------------
    def schedule(self) -> list[Scheduled]:
        """The next step's plan.  When pages are so short that no running request can take even
        one token (every one of them waits for pages the others hold), the request admitted last
        is preempted and the step is planned again; the oldest request therefore always gets on."""
        while True:
            plan = self._plan()
            if plan or len(self.running) <= 1:
                break
            self._preempt(max(self.running, key=lambda candidate: candidate.order), [], [0] * len(self.cache.groups))
        self.stats["steps"] += 1
        for item in plan:
            self.stats["decode_tokens" if item.count == 1 and item.first > 0 and item.samples else "prefill_tokens"] += item.count
        return plan

    def _plan(self) -> list[Scheduled]:
        budget = self.max_tokens_per_step
        plan: list[Scheduled] = []
        planned_pages = [0] * len(self.cache.groups)

        planned: set = set()                 # ids of the requests that the plan holds

        def needs(request: Request, count: int) -> list[int]:
            return self.cache.pages_needed(request.id, count)

        def fits(needed: list[int]) -> bool:
            return all(held + need <= free for held, need, free in zip(planned_pages, needed, self.cache.free_pages()))

        def take(request: Request, count: int, needed: list[int] | None = None) -> None:
            nonlocal budget
            for group, need in enumerate(needed if needed is not None else needs(request, count)):
                planned_pages[group] += need
            plan.append(Scheduled(request, request.computed, count, request.computed + count == request.total))
            planned.add(request.id)
            budget -= count

        # 1. requests that decode: one token each, from the cursor when they exceed the budget
        decoding = [request for request in self.running if request.remaining == 1 and request.computed > 0]
        limit = min(len(decoding), self.max_seqs_per_step, budget)
        if limit < len(decoding):
            start = self._cursor % len(decoding)
            decoding = (decoding[start:] + decoding[:start])[:limit]
            self._cursor += limit
        for request in decoding:
            if request.state != "running":             # preempted for a request before it in this loop
                continue
            needed = needs(request, 1)
            while request.state == "running" and not fits(needed):
                victim = max(self.running, key=lambda candidate: candidate.order)
                if victim is request and len(self.running) == 1:
                    raise out_of_memory(f"request {request.id!r} does not fit the pool alone")   # add() rules this out
                budget += self._preempt(victim, plan, planned_pages)     # what the victim had planned is free for others
                planned.discard(victim.id)
            if request.state == "running":
                take(request, 1, needed)

        if plan and self.prompt_tokens_beside_decodes is not None:
            budget = min(budget, self.prompt_tokens_beside_decodes)    # the decoding requests wait for the whole step

        # 2. running requests still in their prompt (or being recomputed), in admission order
        for request in sorted(self.running, key=lambda candidate: candidate.order):
            if budget <= 0 or len(plan) >= self.max_seqs_per_step:
                break
            if request.id in planned or request.remaining == 0:
                continue
            count = self._portion(request, budget, planned_pages)
            if count > 0:
                take(request, count)

        # 3. new requests, first come first served, while a slot, budget and pages allow
        while self.waiting and budget > 0 and len(plan) < self.max_seqs_per_step and self.cache.free_slots > 0:
            request = self.waiting[0]
            self.cache.admit(request.id)
            if self.running and not self.admit_partial and not self._fits_whole(request):
                self.cache.release(request.id)
                break
            count = self._portion(request, budget, planned_pages)
            if count <= 0:
                self.cache.release(request.id)
                break
            self.waiting.popleft()
            request.state = "running"
            self._admitted += 1
            request.order = self._admitted
            self.running.append(request)
            take(request, count)
        return plan

    def _fits_whole(self, request: Request) -> bool:
        """Whether the pools have room for all of the (just admitted) request's tokens after what the
        running requests still need for theirs, with a page of growth for each of them and for it."""
        wanted = self.cache.pages_needed(request.id, request.remaining)
        for other in self.running:
            for group, pages in enumerate(self.cache.pages_needed(other.id, other.remaining)):
                wanted[group] += pages
        reserve = len(self.running) + 1
        return all(pages + reserve <= free for pages, free in zip(wanted, self.cache.free_pages()))

    def _portion(self, request: Request, budget: int, planned_pages: list[int]) -> int:
        """How many of the request's next tokens this step can take: bounded by the chunk size,
        the budget, and the pages still free after what the step has planned so far."""
        count = min(request.remaining, self.chunk_size, budget)
        if not self.cache.groups:
            return count
        length = self.cache.length(request.id)
        page_size = self.cache.page_size
        room = count
        for group, free in enumerate(self.cache.free_pages()):
            held = len(self.cache.page_list(request.id, group))
            room = min(room, (held + free - planned_pages[group]) * page_size - length)
        return max(0, min(count, room))

    def _preempt(self, victim: Request, plan: list[Scheduled], planned_pages: list[int]) -> int:
        """Takes the victim out of the plan and out of the cache and puts it back in front of the
        queue; returns the tokens it had in the plan."""
        removed = 0
        for item in list(plan):
            if item.request is victim:
                # its planned pages were counted against free pages that its release now returns
                needed = self.cache.pages_needed(victim.id, item.count)
                for group, need in enumerate(needed):
                    planned_pages[group] -= need
                plan.remove(item)
                removed += item.count
        self.cache.release(victim.id)
        self.running.remove(victim)
        victim.state = "waiting"
        victim.computed = 0
        victim.preemptions += 1
        self.stats["preemptions"] += 1
        self.waiting.appendleft(victim)
        return removed

    # ---- after the step ----------------------------------------------------------------------------
    def update(self, plan: list[Scheduled], sampled: list[int] | None) -> list[Request]:
        """`sampled` holds one token for each planned item with `samples`, in plan order.
        Returns the requests that finished.

        `sampled` may be None when the tokens are not on the host yet: PENDING stands in their
        place, and `resolve` writes them later.  Everything a plan depends on is known without
        them (a request ends by its count of tokens), except the end of a request that stops at
        the end-of-sequence token: `can_defer` says whether a plan has such a request."""
        done = []
        cursor = 0
        for item in plan:
            request = item.request
            request.computed += item.count
            if not item.samples:
                continue
            token = PENDING if sampled is None else int(sampled[cursor])
            cursor += 1
            request.generated.append(token)
            if len(request.generated) >= request.params.max_tokens:
                self._finish(request, "length")
                done.append(request)
            elif request.params.stop_on_eos and token == self.eos_token_id:
                self._finish(request, "eos")
                done.append(request)
        return done

    @staticmethod
    def can_defer(plan: list[Scheduled]) -> bool:
        """Whether `update` can do without the tokens of this plan's step for now."""
        return all(not item.request.params.stop_on_eos for item in plan if item.samples)

    @staticmethod
    def resolve(plan: list[Scheduled], sampled: list[int]) -> None:
        """The tokens of a plan that `update` took without them.  Item i's token is the one it
        appended: at index first + count - len(prompt) of the request's generated tokens."""
        cursor = 0
        for item in plan:
            if not item.samples:
                continue
            request = item.request
            index = item.first + item.count - len(request.prompt)
            if not (0 <= index < len(request.generated)) or request.generated[index] != PENDING:
                raise invalid_argument(f"request {request.id!r} has no token pending at {index}")
            request.generated[index] = int(sampled[cursor])
            cursor += 1

    def _finish(self, request: Request, reason: str) -> None:
        if request.state == "running":
            self.cache.release(request.id)
            self.running.remove(request)
        elif request in self.waiting:
            self.waiting.remove(request)
        request.state = "finished"
        request.finish_reason = reason
        self.finished.append(request)
