"""Scheduler + step function + sampler in one loop; the Python entry point ``LLM.generate``."""
from __future__ import annotations

from dataclasses import dataclass, replace
from typing import Dict, Iterable, List, Optional, Sequence

from ..sampling.sampler import SampleRow, Sampler
from .batch import StepEntry
from .engine import Engine, EngineOptions
from .scheduler import Event, Request, Scheduler, StepPlan, UnresolvedTokens


# A request may ask for up to this many sequences (reference: base/src/config.h:97); the random
# stream of sequence i of request r is keyed r * MAX_PARALLEL_SEQUENCES + i (base/src/engine.cu:892-907).
MAX_PARALLEL_SEQUENCES = 8


def engine_key(request: Request):
    """The name a scheduled sequence goes by in the engine (a preempted request that re-enters is
    the same sequence again: same id, index and arrival)."""
    return ("sched", request.id, request.seq_index, request.arrival)


@dataclass
class ServeOptions:
    """Options of the serving loop; names follow the reference's environment variables
    (``base/src/main.cu:52-105``) and limits (``base/src/config.h:80-136``)."""

    temperature: float = 0.0            # TEMPERATURE: <= 0 is greedy
    sampling_seed: int = 0              # SAMPLING_SEED
    ignore_eos: bool = False            # IGNORE_EOS
    repetition_penalty: float = 1.0     # REPETITION_PENALTY (the reference fixes 1.15)
    max_batch_tokens: int = 3072        # MAX_BATCH_TOKENS: a step's token budget
    chunk_size: Optional[int] = None    # most prompt tokens of one request per step
    reserve_policy: str = "max"         # ORCA_POLICY: max | pow2 | oracle (contiguous mode)
    run_ahead: bool = True              # launch a step before the host has seen the previous step's tokens


class Runner:
    """Drives requests to completion, one batch per call to :meth:`step`."""

    def __init__(self, engine: Engine, options: Optional[ServeOptions] = None):
        self.engine = engine
        self.options = options = options or ServeOptions()
        # the engine refuses a step above its own bound, so the scheduler never plans one
        self.scheduler = Scheduler(
            engine.cache, max_batch_tokens=min(options.max_batch_tokens, engine.max_batch_tokens),
            chunk_size=options.chunk_size,
            eos_token_ids=engine.spec.eos_token_ids, ignore_eos=options.ignore_eos,
            reserve_policy=options.reserve_policy, portion_multiple=engine.model.portion_multiple)
        self.sampler = Sampler(engine.vocab_size, engine.cache.max_seqs, engine.device,
                               seed=options.sampling_seed, repetition_penalty=options.repetition_penalty)
        self.scheduler.on_admit = self._on_admit
        self.scheduler.on_release = self._on_release
        self._next_id = 0
        self._in_flight = None        # (ticket, pending tokens) of the step launched last

    # the scheduler owns seats; the engine only needs to know which request sits where
    def _on_admit(self, seq) -> None:
        self.engine.bind_request(engine_key(seq.request), seq.seat)
        emitted = seq.prompt[len(seq.prompt) - seq.request.resumed_tokens:] if seq.request.resumed_tokens else ()
        self.sampler.reset_seat(seq.seat, emitted)

    def _on_release(self, seq) -> None:
        self.engine.unbind_request(engine_key(seq.request))

    def submit(self, tokens: Sequence[int], max_new_tokens: int, *, request_id: Optional[int] = None,
               n_seqs: int = 1, temperature: Optional[float] = None) -> int:
        """Queues ``n_seqs`` copies of a request (reference wire format:
        ``<id> <max_tokens> <n_seqs> <tok> ...``, ``base/src/request_queue.cpp:11-61``)."""
        if not 1 <= n_seqs <= MAX_PARALLEL_SEQUENCES:
            raise ValueError(f"n_seqs {n_seqs} is not in 1..{MAX_PARALLEL_SEQUENCES}")
        if request_id is None:
            request_id = self._next_id
        self._next_id = max(self._next_id, request_id + 1)
        t = self.options.temperature if temperature is None else temperature
        for i in range(n_seqs):
            self.scheduler.add(Request(request_id, [int(x) for x in tokens], int(max_new_tokens),
                                       seq_index=i, temperature=float(t)))
        return request_id

    def idle(self) -> bool:
        return self.scheduler.idle() and self._in_flight is None

    def cancel(self, request_id: int) -> List[Event]:
        """Ends a request now, whatever it was doing: the tokens of the step in flight are taken
        first (they are returned as events, before the ``done`` events with reason ``cancelled``),
        then its sequences leave the queue or give back their seats and pages."""
        events = self._resolve_in_flight()
        events.extend(self.scheduler.cancel(request_id))
        return events

    def live_requests(self) -> List[int]:
        """Ids of the requests that are waiting or hold a seat."""
        sched = self.scheduler
        ids = [r.id for r in sched.waiting] + [s.request.id for s in sched.running + sched.closing]
        return sorted(set(ids))

    def _launch(self, plan: StepPlan):
        """Queues the forward pass and the sampling of a planned step; nothing is waited for."""
        entries, rows = [], []
        for e in plan.entries:
            rid = engine_key(e.seq.request)
            entries.append(StepEntry(rid, e.tokens, [len(e.tokens) - 1] if e.sample else []))
            if e.sample:
                req = e.seq.request
                emitted_before = req.resumed_tokens + len(e.seq.generated)
                rows.append(SampleRow(e.seq.seat, req.temperature, req.id * MAX_PARALLEL_SEQUENCES + req.seq_index,
                                      e.start + len(e.tokens), apply_penalty=emitted_before > 0))
        logits = self.engine.step_planned(entries, [e.seq.seat for e in plan.entries],
                                          [e.start for e in plan.entries])
        # the tokens also stay on the device, where the next step's entries can name them
        return self.sampler.sample_async(logits, rows, out=self.engine.feedback)

    def _resolve_in_flight(self) -> List[Event]:
        if self._in_flight is None:
            return []
        ticket, pending = self._in_flight
        self._in_flight = None
        return self.scheduler.resolve(ticket, pending.wait())

    def step(self) -> List[Event]:
        """Plans and launches one step.  With ``run_ahead`` the events of a step are returned by
        the call after the one that launched it (the device works on a step while the host
        prepares the next); without it every call waits for its own tokens."""
        events: List[Event] = []
        try:
            plan = self.scheduler.plan()
        except UnresolvedTokens:
            events.extend(self._resolve_in_flight())
            plan = self.scheduler.plan()
        launched = None
        if plan.entries:
            if len([e for e in plan.entries if e.sample]) > self.engine.feedback.shape[0]:
                raise RuntimeError("more sampled rows than the engine's feedback buffer holds")
            pending = self._launch(plan)
            launched = (self.scheduler.book(plan), pending)
        events.extend(self._resolve_in_flight())      # the step before the one just launched
        events.extend(plan.events)
        self._in_flight = launched
        if launched is not None and not self.options.run_ahead:
            events.extend(self._resolve_in_flight())
        return events

    def run_until_idle(self) -> Iterable[Event]:
        while not self.idle():
            for ev in self.step():
                yield ev


class LLM:
    """Python entry point: ``LLM(model_dir).generate(prompts, max_new_tokens=...)``."""

    def __init__(self, model_dir: str, engine_options: Optional[EngineOptions] = None,
                 serve_options: Optional[ServeOptions] = None):
        options = engine_options or EngineOptions()
        if options.max_logit_rows is None:
            # generation samples one token per request and step: logits for that many rows, not for
            # every token a step may bring (at a vocabulary of 128,256 that is 4 GB of a step's memory)
            options = replace(options, max_logit_rows=max(1, options.max_seqs))
        self.engine = Engine(model_dir, options)
        self.serve_options = serve_options or ServeOptions()

    def generate(self, prompts: Sequence[Sequence[int]], max_new_tokens: int = 16, *,
                 temperature: Optional[float] = None, seed: Optional[int] = None,
                 ignore_eos: Optional[bool] = None, repetition_penalty: Optional[float] = None,
                 return_reasons: bool = False):
        """Generates for every prompt (token ids in, token ids out), batched continuously."""
        opts = ServeOptions(**vars(self.serve_options))
        if temperature is not None:
            opts.temperature = temperature
        if seed is not None:
            opts.sampling_seed = seed
        if ignore_eos is not None:
            opts.ignore_eos = ignore_eos
        if repetition_penalty is not None:
            opts.repetition_penalty = repetition_penalty
        runner = Runner(self.engine, opts)
        ids = [runner.submit(p, max_new_tokens) for p in prompts]
        out: Dict[int, List[int]] = {i: [] for i in ids}
        reasons: Dict[int, str] = {}
        for ev in runner.run_until_idle():
            if ev.kind == "token":
                out[ev.request_id].append(ev.token)
            elif ev.kind in ("done", "rejected"):
                reasons[ev.request_id] = ev.reason
        self.last_runner = runner
        results = [out[i] for i in ids]
        return (results, [reasons.get(i) for i in ids]) if return_reasons else results
