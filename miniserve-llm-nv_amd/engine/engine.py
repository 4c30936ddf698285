"""The engine: requests in, tokens out.  ``add_request`` admits, ``step`` runs one
scheduled batch through the step function and samples, ``generate`` loops until
every request has finished (reference: miniserve/engine/core.py:193-265 submit,
:278-439 the step, :568-591 the synchronous loop).
"""

from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Callable, Sequence

from ..cache import CacheError, OutOfPagesError
from ..sampling import Sampler
from .batch import StepEntry
from .plan import ExecutionPlan
from .request import Request, SamplingParams
from .scheduler import Scheduler
from .sequence import TERMINAL, RequestStatus, SequenceState


@dataclass(frozen=True)
class StepOutput:
    """A token that a step produced for a request, and whether the request ended with it."""

    request_id: str
    token_id: int
    finished: bool
    finish_reason: str | None


@dataclass(frozen=True)
class GenerationResult:
    request_id: str
    prompt_token_ids: tuple[int, ...]
    token_ids: tuple[int, ...]
    finish_reason: str | None
    num_preemptions: int = 0


def _longest_first(decode_items):
    """The rows of single tokens in the order in which the step runs them: the longest
    context first (equal ones stay in the scheduler's order).  The attention kernel's
    workgroups start in row order, and a step takes as long as its last workgroup: a long
    row that starts late would run on after the others (64 rows of 128 to 2,200 keys:
    75 us a layer in random order, 69 us longest first)."""

    return sorted(decode_items, key=lambda item: -item.position)


@dataclass(frozen=True)
class _StepAhead:
    version: int            # of the engine's request set when the step was planned
    plan: ExecutionPlan
    prepared: object        # the runner's handle: an open cache transaction


class Engine:
    """``runner`` offers ``step(entries) -> logits``, ``admit``, ``release``,
    ``cache.capacity()``, ``spec``, ``max_model_len``, ``block_size`` and
    ``engine_config`` (the ``ModelRunner``; tests may pass a stand-in)."""

    def __init__(self, runner, *, sampler=None, clock_ns: Callable[[], int] = time.monotonic_ns) -> None:
        self.runner = runner
        config = runner.engine_config
        max_positions = runner.spec.max_positions
        self.max_model_len = runner.max_model_len
        self.max_num_batched_tokens = config.resolved_max_num_batched_tokens(max_positions)
        self.enable_chunked_prefill = config.enable_chunked_prefill
        self.max_pending_requests = config.max_pending_requests
        self.vocab_size = runner.spec.vocab_size
        self.scheduler = Scheduler(
            max_num_seqs=config.max_num_seqs,
            max_num_batched_tokens=self.max_num_batched_tokens,
            enable_chunked_prefill=config.enable_chunked_prefill,
            prefill_chunk_size=config.prefill_chunk_size,
        )
        self.sampler = sampler if sampler is not None else Sampler()
        self._clock_ns = clock_ns
        self._sequences: dict[str, SequenceState] = {}
        self._results: dict[str, GenerationResult] = {}
        self.last_plan: ExecutionPlan | None = None
        self._version = 0                       # goes up when requests are added or cancelled
        self._ahead: _StepAhead | None = None
        self.counters = {"steps": 0, "prefill_tokens": 0, "decode_tokens": 0, "preemptions": 0, "empty_plans": 0}

    # ---- admission --------------------------------------------------------------------
    def add_request(
        self,
        request_id: str,
        prompt_token_ids: Sequence[int],
        sampling_params: SamplingParams | None = None,
        *,
        arrival_ns: int | None = None,
    ) -> None:
        """Checks of the reference's ``submit`` (core.py:193-236), before any state exists."""

        params = sampling_params if sampling_params is not None else SamplingParams()
        request = Request(
            request_id,
            tuple(prompt_token_ids),
            params,
            self._clock_ns() if arrival_ns is None else arrival_ns,
        )
        if request_id in self._sequences or request_id in self._results:
            raise ValueError(f"Duplicate request_id: {request_id}")
        active = sum(1 for state in self._sequences.values() if state.status not in TERMINAL)
        if active >= self.max_pending_requests:
            raise RuntimeError("QUEUE_FULL: max_pending_requests reached.")
        total = len(request.prompt_token_ids) + params.max_new_tokens
        if total > self.max_model_len:
            raise ValueError(
                f"CONTEXT_LENGTH_EXCEEDED: prompt {len(request.prompt_token_ids)} + max_new_tokens "
                f"{params.max_new_tokens} exceeds max_model_len {self.max_model_len}."
            )
        capacity = self.runner.cache.capacity()
        # (a preempted request runs all it holds again, so a step may bring up to total - 1 tokens or the budget)
        step_tokens = self.max_num_batched_tokens if self.enable_chunked_prefill else total
        needed = capacity.most_pages_held(total, step_tokens)
        if any(pages > pool for pages, pool in zip(needed, capacity.total_blocks)):
            raise ValueError("CONTEXT_CAPACITY_EXCEEDED: the request alone needs more pages than the pool holds.")
        if any(token >= self.vocab_size for token in request.prompt_token_ids):
            raise ValueError("prompt token id is outside the vocabulary.")
        if params.top_k > self.vocab_size:
            raise ValueError("top_k must not exceed the vocabulary size.")
        if any(token >= self.vocab_size for token in params.stop_token_ids):
            raise ValueError("stop token id is outside the vocabulary.")
        if not self.enable_chunked_prefill and total - 1 > self.max_num_batched_tokens:
            # without portions, a preempted request must be able to run all its tokens in one step
            raise ValueError(
                "CHUNKED_PREFILL_DISABLED: the request does not fit max_num_batched_tokens in one step; "
                "enable chunked prefill."
            )
        self._sequences[request_id] = SequenceState.from_request(request)
        self._version += 1

    def cancel(self, request_id: str) -> None:
        state = self._sequences[request_id]
        self._version += 1
        self._drop_prepared_step()
        state.cancel()
        self._finalize(state)

    def _drop_prepared_step(self) -> None:
        ahead, self._ahead = self._ahead, None
        if ahead is not None:
            self.runner.discard(ahead.prepared)

    def has_unfinished(self) -> bool:
        return bool(self._sequences)

    # ---- one step ---------------------------------------------------------------------
    def step(self) -> list[StepOutput]:
        ahead = self._take_prepared_step()
        if ahead is not None:
            plan = ahead.plan
        else:
            views = [state.snapshot() for state in self._sequences.values()]
            plan = self.scheduler.schedule(views, self.runner.cache.capacity())
        self.last_plan = plan
        for request_id in plan.preempted:
            self.runner.release(request_id)
            self._sequences[request_id].preempt()
            self.counters["preemptions"] += 1
        if plan.empty:
            self.counters["empty_plans"] += 1
            return []

        entries: list[StepEntry] = []
        sampled: list[SequenceState] = []
        for item in _longest_first(plan.decode_items):
            state = self._sequences[item.request_id]
            # (a step planned ahead did not know the token yet)
            entries.append(StepEntry(item.request_id, (state.token_at(state.computed_tokens),), (0,)))
            sampled.append(state)
        for item in plan.prefill_items:
            state = self._sequences[item.request_id]
            if state.status is RequestStatus.WAITING:
                if not self.runner.cache.is_live(item.request_id):       # (a step planned ahead admitted it)
                    self.runner.admit(item.request_id)
                state.admitted()
            tokens = state.tokens_between(item.token_start, item.token_end)
            final = item.token_end == state.prefill_target
            entries.append(StepEntry(item.request_id, tuple(tokens), (len(tokens) - 1,) if final else ()))
            if final:
                sampled.append(state)

        next_ahead = None
        try:
            if ahead is not None:
                logits = self.runner.step(entries, prepared=ahead.prepared)
            else:
                logits = self.runner.step(entries)
            staged = ()
            if sampled:
                requests = [(s.request_id, s.sampling_params) for s in sampled]
                if hasattr(self.sampler, "launch"):
                    launched = self.sampler.launch(logits, requests)
                    # while the GPU runs the step: the next one, if it can be foreseen
                    next_ahead = self._prepare_step_ahead(plan, sampled)
                    self._launch_chained(next_ahead, sampled, launched)
                    staged = self.sampler.finish(launched)
                else:
                    staged = self.sampler.stage(logits, requests)
        except Exception as exc:
            # the step left no trace in the cache; its requests fail (reference: core.py:396-406)
            if next_ahead is not None:
                self.runner.discard(next_ahead.prepared)
            for entry in entries:
                state = self._sequences[entry.request_id]
                state.fail(f"{type(exc).__name__}: {exc}")
                self._finalize(state)
            raise
        self.sampler.commit(staged)

        self.counters["steps"] += 1
        self.counters["decode_tokens"] += len(plan.decode_items)
        self.counters["prefill_tokens"] += plan.scheduled_tokens - len(plan.decode_items)
        for item in plan.decode_items:
            self._sequences[item.request_id].ran_pending_token()
        for item in plan.prefill_items:
            self._sequences[item.request_id].ran_to(item.token_end)
        outputs: list[StepOutput] = []
        planned = set() if next_ahead is None else {item.request_id for item in next_ahead.plan.decode_items}
        # (the requests of its prompt portions are not sampled now and cannot end now)
        for state, sample in zip(sampled, staged):
            state.take_token(sample.token_id)
            reason = state.ending()
            if reason is not None:
                if next_ahead is not None and state.request_id in planned:
                    # a request of the step that was planned ahead ends (a stop token): that
                    # step's reservation goes back before the request's pages can
                    self.runner.discard(next_ahead.prepared)
                    next_ahead = None
                state.finish(reason)
                self._finalize(state)
            outputs.append(StepOutput(state.request_id, sample.token_id, reason is not None, reason))
        self._ahead = next_ahead
        return outputs

    # ---- the next step, planned while the GPU runs this one -------------------------------
    def _take_prepared_step(self) -> "_StepAhead | None":
        """The step planned ahead, if nothing has happened since that it did not foresee."""

        ahead, self._ahead = self._ahead, None
        if ahead is not None and ahead.version != self._version:
            self.runner.discard(ahead.prepared)
            return None
        return ahead

    def _prepare_step_ahead(self, plan: ExecutionPlan, sampled: Sequence[SequenceState]) -> "_StepAhead | None":
        """The step after the running one, as far as it can be foreseen: every request as
        the running step will leave it, each sampled one a token further (the token itself
        not known yet) and without those that end by length now.  It is scheduled from
        views that say so, its cache transaction is opened and its numbers are written
        now; only the sampled token ids are left for when they are known.  A step of
        single tokens goes to the recorded step's second host buffer, any other has its
        tensors built.  A plan that would preempt is left to the next call, and so is one
        that could make use of what a request that ends now gives back."""

        prepare_decode = getattr(self.runner, "prepare_decode", None)
        prepare_step = getattr(self.runner, "prepare_step", None)
        if prepare_decode is None or plan.preempted:
            return None
        sampled_ids = {state.request_id for state in sampled}
        prefill_end = {item.request_id: item.token_end for item in plan.prefill_items}
        decoded = {item.request_id for item in plan.decode_items}
        views = []
        ending = False
        for state in self._sequences.values():
            is_sampled = state.request_id in sampled_ids
            if is_sampled and len(state.generated_token_ids) + 1 >= state.sampling_params.max_new_tokens:
                ending = True           # ends with the token sampled now
                continue
            views.append(
                state.view_after(
                    prefill_end=prefill_end.get(state.request_id),
                    decoded=state.request_id in decoded,
                    sampled=is_sampled,
                )
            )
        if not views:
            return None
        next_plan = self.scheduler.schedule(views, self.runner.cache.capacity())
        if next_plan.preempted or next_plan.empty:
            return None
        if ending and (next_plan.prefill_items or len(next_plan.decode_items) != len(views)):
            # the pages and the slot of a request that ends now are not free yet; a plan
            # made without them may hold less than the one made when they are
            return None
        try:
            if not next_plan.prefill_items:
                prepared = prepare_decode([item.request_id for item in _longest_first(next_plan.decode_items)])
            elif prepare_step is not None:
                entries, admit = [], []
                for item in _longest_first(next_plan.decode_items):
                    state = self._sequences[item.request_id]
                    token = 0 if item.request_id in sampled_ids else state.token_at(state.computed_tokens)
                    entries.append(StepEntry(item.request_id, (token,), (0,)))
                for item in next_plan.prefill_items:
                    state = self._sequences[item.request_id]
                    if not self.runner.cache.is_live(item.request_id):
                        admit.append(item.request_id)
                    tokens = state.tokens_between(item.token_start, item.token_end)
                    final = item.token_end == state.prefill_target
                    entries.append(StepEntry(item.request_id, tuple(tokens), (len(tokens) - 1,) if final else ()))
                prepared = prepare_step(entries, admit)
            else:
                prepared = None
        except (OutOfPagesError, CacheError):
            return None                # the plan's page and slot counts were estimates; the next call decides
        if prepared is None:
            return None
        return _StepAhead(self._version, next_plan, prepared)

    def _launch_chained(self, ahead: "_StepAhead | None", sampled: Sequence[SequenceState], launched) -> None:
        """A recorded step of single tokens that was planned ahead is launched at once,
        behind the running step, when each of its rows is a request that the running step
        samples: the sampling kernel's tokens go into its token ids on the device (row by
        row, or through a map of rows when a request of the running step ends by length
        now or the order differs), and the GPU does not wait while the host reads them and
        advances the requests.  Should a request of it turn out to have ended (a stop
        token), or the set of requests change before the next call, the step is thrown
        away like any step planned ahead; it has then run for nothing."""

        launch = getattr(self.runner, "launch_chained", None)
        if ahead is None or launch is None or ahead.plan.prefill_items or not hasattr(ahead.prepared, "launched"):
            return
        tokens = launched[0]
        if not getattr(tokens, "is_cuda", False):
            return
        rows = [item.request_id for item in _longest_first(ahead.plan.decode_items)]
        sampled_ids = [state.request_id for state in sampled]
        if rows == sampled_ids[: len(rows)]:
            launch(ahead.prepared, tokens)          # the same rows, or the first of them (the last ones end now)
            return
        place = {request_id: row for row, request_id in enumerate(sampled_ids)}
        if all(request_id in place for request_id in rows):
            launch(ahead.prepared, tokens, [place[request_id] for request_id in rows])

    def _finalize(self, state: SequenceState) -> None:
        """A request that ended gives back its pages, its state slot and its random stream."""

        if self.runner.cache.is_live(state.request_id):
            self.runner.release(state.request_id)
        self.sampler.release(state.request_id)
        self._results[state.request_id] = GenerationResult(
            state.request_id,
            state.prompt_token_ids,
            tuple(state.generated_token_ids),
            state.finish_reason,
            state.num_preemptions,
        )
        del self._sequences[state.request_id]

    def pop_result(self, request_id: str) -> GenerationResult:
        return self._results.pop(request_id)

    # ---- the synchronous loop ---------------------------------------------------------
    def generate(
        self,
        prompts: Sequence[Sequence[int]],
        sampling_params: SamplingParams | Sequence[SamplingParams] | None = None,
    ) -> list[list[int]]:
        """Token ids in, generated token ids out, one list per prompt."""

        if isinstance(sampling_params, SamplingParams) or sampling_params is None:
            params = [sampling_params or SamplingParams()] * len(prompts)
        else:
            params = list(sampling_params)
            if len(params) != len(prompts):
                raise ValueError("one SamplingParams per prompt is needed.")
        base = len(self._results) + len(self._sequences)
        request_ids = [f"generate-{base + index}" for index in range(len(prompts))]
        for index, (request_id, prompt, p) in enumerate(zip(request_ids, prompts, params)):
            self.add_request(request_id, prompt, p, arrival_ns=index)
        idle = 0
        while any(request_id in self._sequences for request_id in request_ids):
            produced = self.step()
            idle = 0 if (produced or not self.last_plan.empty) else idle + 1
            if idle > 2:
                raise RuntimeError("the scheduler made no progress: no request fits the cache.")
        return [list(self.pop_result(request_id).token_ids) for request_id in request_ids]
