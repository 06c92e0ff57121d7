"""Continuous-batching scheduler with chunked prefill.  Pure host logic: it decides, the engine runs.

Each call to :meth:`Scheduler.plan` makes one step's batch under a token budget:

1. every running request whose prompt is in the cache decodes one token (scheduled first);
2. the rest of the budget goes to prompt portions, first come first served: requests that are
   part-way through their prompt, then new admissions; a prompt may be cut at any token and a
   single request's portion is capped by ``chunk_size``;
3. a request finishes on an end-of-sequence token (not emitted, not counted), when its budget
   of new tokens is used up, when it reaches the longest sequence the cache can hold, or - with
   the error ``invalid_logits`` - when the sampler reports that its logits named no token
   (a negative token id: no logit of the row was finite).

The reference has no chunked prefill (its prefill attention cannot read the cache,
``base/src/engine.cu:730-737``); what it does have is kept: FCFS queue with preempted requests
going back to the FRONT (``paged_attention/src/engine.cu:728-730``), admission only when the
whole prompt's pages are free (``:326-339``), admission closed to new requests while preempted
ones are pending (``:314-321``), and - when pages run out during decoding - preemption of the
newest request first with recomputation: its prompt plus everything it has generated re-enters
as a prompt and nothing is emitted twice (``:640-731, 792-838``).  If a request cannot get its
pages even with nothing else running it fails with ``kv_cache_exhausted`` (``:953-1001``).

Contiguous mode (``base/src/engine.cu:301-355, 411-464``): a request reserves its whole run at
admission by policy - ``max`` (the longest sequence), ``pow2`` (prompt + output budget rounded
up to a power of two), ``oracle`` (prompt + output budget) - the queue head blocks until its
reservation can be placed, nothing is ever preempted, and a request that fills its reservation
finishes with ``sequence_too_long``.

Running ahead of the device.  Booking a step does not need the values of the tokens it sampled,
only their number: :meth:`Scheduler.book` advances every request as if no end-of-sequence token
had come and returns a :class:`Ticket`; the next step can be planned and launched at once, its
decode entries naming the tokens by their row in the previous sampling (they are still on the
device).  :meth:`Scheduler.resolve` later takes the values: it emits the token events, and a
request whose token was end-of-sequence is finished then - the one token computed for it in the
step already in flight is dropped.  Anything that must know the values first (preempting or
failing a request) makes :meth:`plan` raise :class:`UnresolvedTokens` before it changes anything.
:meth:`complete` is ``resolve(book(plan), sampled)``.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Sequence, Tuple

from ..cache.manager import CacheManager

RESERVE_POLICIES = ("max", "pow2", "oracle")


@dataclass
class Request:
    id: int
    tokens: List[int]                 # prompt (plus earlier output when resumed)
    max_new_tokens: int
    seq_index: int = 0
    temperature: float = 0.0
    resumed_tokens: int = 0           # how many of ``tokens`` (at the end) were generated before a preemption
    arrival: int = -1
    preempted: bool = False           # re-entered after a preemption (possibly with nothing generated yet)


@dataclass
class Sequence_:
    request: Request
    seat: int
    prompt: List[int]
    computed: int = 0                 # tokens whose K/V are in the cache
    generated: List[int] = field(default_factory=list)
    remaining: int = 0
    was_preempted: bool = False
    next_token: Optional[int] = None  # sampled, not yet run through the model; negative: row
                                      # ``-1 - next_token`` of the last sampling, value not seen yet
    next_from: object = None          # the Ticket whose sampling ``next_token`` names
    unresolved: int = 0               # placeholders in ``generated``
    dead: bool = False                # finished; entries of it still in flight are dropped

    @property
    def prefilling(self) -> bool:
        return self.computed < len(self.prompt)


@dataclass
class PlanEntry:
    seq: Sequence_
    tokens: List[int]
    start: int
    sample: bool                      # the last token's logits are wanted and a token is sampled


@dataclass
class Event:
    kind: str                         # "token" | "done" | "preempted" | "rejected"
    request_id: int
    seq_index: int = 0
    seat: int = -1
    token: Optional[int] = None
    tokens: int = 0                   # done: tokens generated in total
    reason: Optional[str] = None      # done: "eos" | "length" | error name
    generated: int = 0                # preempted: tokens generated so far


@dataclass
class StepPlan:
    entries: List[PlanEntry]
    events: List[Event]               # what planning itself decided (preemptions, failures)

    @property
    def num_tokens(self) -> int:
        return sum(len(e.tokens) for e in self.entries)


@dataclass
class Ticket:
    """A booked step whose sampled tokens the host has not seen yet."""
    plan: StepPlan
    rows: List[Tuple[Sequence_, int, bool]]   # per sampled entry: sequence, index of its
                                              # placeholder in ``generated``, ends by length


class UnresolvedTokens(RuntimeError):
    """Planning has to finish or preempt a request whose last tokens are not known to the host
    yet: resolve the step in flight, then plan again."""


def reservation_tokens(policy: str, prompt_len: int, max_new_tokens: int, max_seq_len: int) -> int:
    """Tokens a contiguous-mode request reserves (reference: ``base/src/engine.cu:301-330``)."""
    if policy == "max":
        return max_seq_len
    if policy == "pow2":
        p = 1
        while p < max_new_tokens:
            p *= 2
        return min(prompt_len + p, max_seq_len)
    if policy == "oracle":
        return min(prompt_len + max_new_tokens, max_seq_len)
    raise ValueError(f"reservation policy {policy!r} is not one of {RESERVE_POLICIES}")


class Scheduler:
    def __init__(self, cache: CacheManager, *, max_batch_tokens: int = 3072, chunk_size: Optional[int] = None,
                 eos_token_ids: Sequence[int] = (), ignore_eos: bool = False,
                 reserve_policy: str = "max", portion_multiple: int = 1):
        if max_batch_tokens < 1:
            raise ValueError("max_batch_tokens must be at least 1")
        if portion_multiple < 1 or portion_multiple > max_batch_tokens:
            raise ValueError(f"portions that end on multiples of {portion_multiple} positions do not fit "
                             f"steps of {max_batch_tokens} tokens")
        if reserve_policy not in RESERVE_POLICIES:
            raise ValueError(f"reservation policy {reserve_policy!r} is not one of {RESERVE_POLICIES}")
        self.cache = cache
        self.max_batch_tokens = int(max_batch_tokens)
        self.chunk_size = int(chunk_size) if chunk_size else self.max_batch_tokens
        # every portion but a prompt's last ends at a multiple of this many positions (what the
        # model's mixers ask for: parts.base.Mixer.portion_multiple)
        self.portion_multiple = int(portion_multiple)
        if self.chunk_size < self.portion_multiple:
            raise ValueError(f"chunk_size {self.chunk_size} is smaller than the {self.portion_multiple} positions "
                             f"a portion must be a multiple of")
        self.eos = frozenset(int(e) for e in eos_token_ids)
        self.ignore_eos = bool(ignore_eos)
        self.reserve_policy = reserve_policy
        self.waiting: Deque[Request] = deque()
        self.running: List[Sequence_] = []
        self.closing: List[Sequence_] = []     # out of tokens, waiting for their last value
        self._arrivals = 0
        self.preemption_pending = False
        self._preempted_in_flight = 0
        self.preemptions = 0
        self.on_admit = None          # callback(seq) when a request takes a seat
        self.on_release = None        # callback(seq) when a seat is given back

    # ------------------------------------------------------------------ queue
    def add(self, request: Request) -> None:
        if request.arrival < 0:
            request.arrival = self._arrivals
            self._arrivals += 1
        self.waiting.append(request)

    def idle(self) -> bool:
        return not self.waiting and not self.running and not self.closing

    def cancel(self, request_id: int) -> List[Event]:
        """Drops every sequence of a request, wherever it is: waiting ones leave the queue, seated
        ones give back their seat and pages at once.  Each ends with reason ``cancelled`` and the
        number of tokens it had emitted.  Tokens of a booked step that are still to be resolved
        are dropped when they arrive.  The caller resolves the step in flight first if it wants
        the tokens that step produced."""
        events: List[Event] = []
        kept: Deque[Request] = deque()
        for r in self.waiting:
            if r.id != request_id:
                kept.append(r)
                continue
            events.append(Event("done", r.id, r.seq_index, tokens=r.resumed_tokens, reason="cancelled"))
            if r.preempted:
                self._preempted_gone()
        self.waiting = kept
        for seq in [s for s in self.running + self.closing if s.request.id == request_id]:
            del seq.generated[len(seq.generated) - seq.unresolved:]      # placeholders of tokens never seen
            seq.unresolved = 0
            self._finish(seq, "cancelled", events)
        return events

    # ------------------------------------------------------------------ helpers
    def _release(self, seq: Sequence_) -> None:
        if self.on_release:
            self.on_release(seq)
        self.cache.free(seq.seat)
        seq.dead = True
        (self.running if seq in self.running else self.closing).remove(seq)

    def _finish(self, seq: Sequence_, reason: str, events: List[Event]) -> None:
        events.append(Event("done", seq.request.id, seq.request.seq_index, seq.seat,
                            tokens=seq.request.resumed_tokens + len(seq.generated), reason=reason))
        if seq.was_preempted:
            self._preempted_gone()
        self._release(seq)

    def _preempted_gone(self) -> None:
        """A request that had been preempted has left for good; admission opens again with the last."""
        self._preempted_in_flight -= 1
        if self._preempted_in_flight <= 0:
            self._preempted_in_flight = 0
            self.preemption_pending = False

    def _preempt(self, seq: Sequence_, events: List[Event]) -> None:
        """Recompute-style preemption: everything so far becomes the prompt of a request that
        re-enters at the front of the queue."""
        done_before = seq.request.resumed_tokens + len(seq.generated)
        tokens = list(seq.prompt) + list(seq.generated)
        events.append(Event("preempted", seq.request.id, seq.request.seq_index, seq.seat,
                            generated=done_before, reason="recompute"))
        resumed = Request(seq.request.id, tokens, seq.remaining, seq.request.seq_index,
                          seq.request.temperature, resumed_tokens=done_before,
                          arrival=seq.request.arrival, preempted=True)
        if not seq.was_preempted:
            self._preempted_in_flight += 1
        self.preemption_pending = True
        self.preemptions += 1
        self._release(seq)
        self.waiting.appendleft(resumed)

    def _free_pages(self) -> List[int]:
        return [g.free_pages() for g in self.cache.groups]

    # ------------------------------------------------------------------ planning
    def plan(self) -> StepPlan:
        events: List[Event] = []
        cache = self.cache
        paged = cache.mode == "paged"

        # finishing or preempting a request needs all its tokens' values: refuse before any change
        pending = [s for s in self.running if s.unresolved]
        if pending:
            if any(not s.prefilling and s.computed + 1 > cache.capacity_tokens(s.seat) for s in pending):
                raise UnresolvedTokens("a request with unseen tokens has filled its room in the cache")
            if paged:
                need = [0] * len(cache.groups)
                for s in self.running:
                    if not s.prefilling:
                        for i, n in enumerate(cache.pages_needed(s.seat, s.computed + 1)):
                            need[i] += n
                if any(n > f for n, f in zip(need, self._free_pages())):
                    raise UnresolvedTokens("pages run out while tokens of running requests are unseen")

        # a request that has filled what the cache can hold for it ends before the forward
        for seq in list(self.running):
            if not seq.prefilling and seq.computed + 1 > cache.capacity_tokens(seq.seat):
                self._finish(seq, "sequence_too_long", events)

        # 1. decoding requests, one token each; preempt the newest until their pages fit
        def decode_need() -> List[int]:
            need = [0] * len(cache.groups)
            for s in self.running:
                if not s.prefilling:
                    for i, n in enumerate(cache.pages_needed(s.seat, s.computed + 1)):
                        need[i] += n
            return need

        if paged:
            while any(n > f for n, f in zip(decode_need(), self._free_pages())):
                victims = sorted(self.running, key=lambda s: s.request.arrival)
                if len(victims) <= 1:
                    self._finish(victims[0], "kv_cache_exhausted", events)
                    break
                self._preempt(victims[-1], events)

        entries: List[PlanEntry] = []
        committed = [0] * len(cache.groups)     # pages promised to entries planned so far
        for seq in sorted(self.running, key=lambda s: s.request.arrival):
            if seq.prefilling:
                continue
            if len(entries) >= self.max_batch_tokens:
                break
            for i, n in enumerate(cache.pages_needed(seq.seat, seq.computed + 1)):
                committed[i] += n
            entries.append(PlanEntry(seq, [seq.next_token], seq.computed, sample=True))
        budget = self.max_batch_tokens - len(entries)
        decode_pages = list(committed)          # pages the decoding requests take in this step

        def prompt_pages_outstanding() -> List[int]:
            """Pages the admitted requests still need to finish their prompts: a prompt is mapped
            portion by portion, so what is free now is not all free for a newcomer."""
            need = [0] * len(cache.groups)
            for s in self.running:
                if s.prefilling:
                    for i, n in enumerate(cache.pages_outstanding(s.seat, len(s.prompt), self.chunk_size)):
                        need[i] += n
            return need

        def fit_tokens(seq: Sequence_, want: int) -> int:
            """Largest portion <= want whose pages are still free."""
            if not paged:
                return want
            free = [f - c for f, c in zip(self._free_pages(), committed)]
            n = want
            while n > 0:
                need = cache.pages_needed(seq.seat, seq.computed + n)
                if all(x <= f for x, f in zip(need, free)):
                    return n
                # drop back to the previous page edge
                edge = (seq.computed + n - 1) // cache.page_size * cache.page_size
                n = edge - seq.computed
            return 0

        def add_portion(seq: Sequence_) -> None:
            nonlocal budget
            want = min(len(seq.prompt) - seq.computed, self.chunk_size, budget)
            n = fit_tokens(seq, want)
            if self.portion_multiple > 1 and seq.computed + n < len(seq.prompt):
                n = (seq.computed + n) // self.portion_multiple * self.portion_multiple - seq.computed
            if n <= 0:
                return
            for i, x in enumerate(cache.pages_needed(seq.seat, seq.computed + n)):
                committed[i] += x
            last = seq.computed + n == len(seq.prompt)
            entries.append(PlanEntry(seq, seq.prompt[seq.computed:seq.computed + n], seq.computed,
                                     sample=last))
            budget -= n

        # 2. requests part-way through their prompt
        for seq in sorted(self.running, key=lambda s: s.request.arrival):
            if seq.prefilling and budget > 0:
                add_portion(seq)

        # 3. admissions, first come first served
        while self.waiting and budget > 0 and cache.free_seats > 0:
            head = self.waiting[0]
            if self.preemption_pending and not head.preempted:
                break
            plen = len(head.tokens)
            if plen == 0 or head.max_new_tokens < 1:
                self.waiting.popleft()
                events.append(Event("rejected", head.id, head.seq_index, reason="empty_request"))
                continue
            if plen + 1 > cache.max_seq_len:
                self.waiting.popleft()
                events.append(Event("rejected", head.id, head.seq_index, reason="prompt_too_long"))
                continue
            reserve = None
            if paged:
                # every group says what a prompt of this length needs of it (all its pages where
                # all keys stay, a window's worth where only a window is kept, nothing where a
                # model keeps no keys at all)
                pages = [g.pages_for(plen, self.chunk_size) for g in cache.groups]
                free = [f - d - o for f, d, o in zip(self._free_pages(), decode_pages, prompt_pages_outstanding())]
                if any(p > f for p, f in zip(pages, free)):
                    if not self.running and not entries and any(p > g.num_pages for p, g in zip(pages, cache.groups)):
                        self.waiting.popleft()
                        events.append(Event("done", head.id, head.seq_index, tokens=head.resumed_tokens,
                                            reason="kv_cache_exhausted"))
                        if head.preempted:
                            self._preempted_gone()
                        continue
                    break
            else:
                reserve = reservation_tokens(self.reserve_policy, plen - head.resumed_tokens,
                                             head.max_new_tokens + head.resumed_tokens, cache.max_seq_len)
            seat = cache.admit(head.id, reserve)
            if seat is None:
                # given up only when nothing can still free room: a request that waits for its
                # last token's value (``closing``) holds its run one more step and then leaves
                if not paged and not self.running and not self.closing:
                    self.waiting.popleft()
                    events.append(Event("done", head.id, head.seq_index, tokens=head.resumed_tokens,
                                        reason="kv_cache_exhausted"))
                    if head.preempted:
                        self._preempted_gone()
                    continue
                break       # the queue head waits for room (head-of-line, as in the reference)
            self.waiting.popleft()
            seq = Sequence_(head, seat, list(head.tokens), remaining=head.max_new_tokens,
                            was_preempted=head.preempted)
            self.running.append(seq)
            if self.on_admit:
                self.on_admit(seq)
            add_portion(seq)

        # Nothing to run although requests hold seats: every one of them is part-way through its
        # prompt and no page is free (decoding neighbours that have since left took the pages their
        # prompts were admitted against; requests that wait for their last token's value, which
        # will free theirs, are excluded).  The newest gives its pages back and re-enters at the
        # front of the queue; one alone that cannot go on does not fit the cache at all.
        if paged and not entries and self.running and not self.closing \
                and all(s.prefilling for s in self.running):
            victims = sorted(self.running, key=lambda s: s.request.arrival)
            if len(victims) > 1:
                self._preempt(victims[-1], events)
            else:
                self._finish(victims[0], "kv_cache_exhausted", events)
        return StepPlan(entries, events)

    # ------------------------------------------------------------------ after the forward
    def complete(self, plan: StepPlan, sampled: Sequence[int]) -> List[Event]:
        """Books the step: ``sampled`` holds one token per entry with ``sample`` set, in order."""
        return self.resolve(self.book(plan), sampled)

    def book(self, plan: StepPlan) -> Ticket:
        """The part of booking that does not need the sampled values: lengths, counts, and a
        placeholder per sampled token.  A request that has used up its budget of new tokens
        leaves the running set (it is not scheduled again) and keeps its seat until
        :meth:`resolve`."""
        ticket = Ticket(plan, [])
        for e in plan.entries:
            seq = e.seq
            seq.computed += len(e.tokens)
            self.cache.commit(seq.seat, seq.computed)
            if not e.sample:
                continue
            seq.generated.append(None)
            seq.unresolved += 1
            seq.next_token = -1 - len(ticket.rows)
            seq.next_from = ticket
            seq.remaining -= 1
            ending = seq.remaining <= 0
            if ending:
                self.running.remove(seq)
                self.closing.append(seq)
            ticket.rows.append((seq, len(seq.generated) - 1, ending))
        return ticket

    def resolve(self, ticket: Ticket, sampled: Sequence[int]) -> List[Event]:
        """Takes the values of a booked step's sampled tokens, one per row of the ticket."""
        events: List[Event] = []
        if len(sampled) != len(ticket.rows):
            raise ValueError(f"{len(sampled)} tokens for {len(ticket.rows)} sampled entries")
        for (seq, idx, ending), tok in zip(ticket.rows, sampled):
            if seq.dead:
                continue            # ended by an earlier token while this step was in flight
            tok = int(tok)
            seq.unresolved -= 1
            if tok < 0:
                # the sampler found no token in this row's logits (none of them finite): the request
                # ends with an error instead of going on from a token nobody chose
                del seq.generated[idx:]
                seq.unresolved = 0
                self._finish(seq, "invalid_logits", events)
                continue
            if tok in self.eos and not self.ignore_eos:
                del seq.generated[idx:]
                seq.unresolved = 0
                self._finish(seq, "eos", events)
                continue
            seq.generated[idx] = tok
            if seq.next_from is ticket:
                seq.next_token, seq.next_from = tok, None
            events.append(Event("token", seq.request.id, seq.request.seq_index, seq.seat, token=tok))
            if ending:
                self._finish(seq, "length", events)
        return events
