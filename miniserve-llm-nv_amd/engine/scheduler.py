"""The scheduler: which requests run in the next step, and with how many tokens.

Policy of the reference's ``ContinuousBatchScheduler`` (miniserve/engine/scheduler.py:129-227):
oldest first by ``(arrival, id)``; requests that decode go first, one token each;
then prompts, whole, or in portions under the token budget when chunked prefill
is on; when chunked prefill is on and a prompt can move, one token of the budget
is held back for it so decoding cannot starve it.

What happens when pages run out is decided here, where the reference only skips
the request (scheduler.py:167-172, 203-210) and can stall for good: a running
request that needs a page and finds none takes the pages of the YOUNGEST running
request that is younger than itself, which is *preempted* (it loses its cache and
waits; its tokens are run again later).  The oldest running request is never
preempted, so it always finishes.  A running request that finds no younger one to
preempt waits for a step.  Waiting requests never preempt anyone; they are
admitted only while a state slot is free.

The function is pure: it reads views and a capacity snapshot and returns a plan.
"""

from __future__ import annotations

from collections.abc import Sequence

from ..cache.manager import CapacitySnapshot
from .plan import DecodeItem, ExecutionPlan, PrefillItem
from .sequence import RequestStatus, SequenceView


class Scheduler:
    def __init__(
        self,
        *,
        max_num_seqs: int,
        max_num_batched_tokens: int,
        enable_chunked_prefill: bool = False,
        prefill_chunk_size: int | None = None,
    ) -> None:
        if max_num_seqs <= 0 or max_num_batched_tokens <= 0:
            raise ValueError("The scheduler requires positive sequence and token budgets.")
        if prefill_chunk_size is not None:
            if not isinstance(prefill_chunk_size, int) or isinstance(prefill_chunk_size, bool) or prefill_chunk_size <= 0:
                raise ValueError("prefill_chunk_size must be a positive integer or None.")
            if not enable_chunked_prefill:
                raise ValueError("prefill_chunk_size requires enable_chunked_prefill=True.")
            if prefill_chunk_size > max_num_batched_tokens:
                raise ValueError("prefill_chunk_size cannot exceed max_num_batched_tokens.")
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens
        self.enable_chunked_prefill = enable_chunked_prefill
        self.prefill_chunk_size = prefill_chunk_size
        self._next_step_id = 0

    def schedule(self, sequences: Sequence[SequenceView], capacity: CapacitySnapshot) -> ExecutionPlan:
        step_id = self._next_step_id
        self._next_step_id += 1
        ordered = sorted(sequences, key=lambda view: (view.arrival_ns, view.request_id))
        running = [v for v in ordered if v.status in (RequestStatus.PREFILLING, RequestStatus.DECODING)]
        block_size = capacity.block_size
        free = list(capacity.free_blocks)            # estimated free pages per group
        free_slots = capacity.free_slots
        token_budget = self.max_num_batched_tokens
        preempted: list[str] = []
        preempted_set: set[str] = set()
        decode_items: list[DecodeItem] = []
        prefill_items: list[PrefillItem] = []
        scheduled: set[str] = set()

        def fits(pages: int) -> bool:
            return all(pages <= count for count in free)

        def take(pages: int) -> None:
            for group in range(len(free)):
                free[group] -= pages

        def make_room(view: SequenceView, pages: int) -> bool:
            """Preempt the youngest running requests younger than ``view`` until
            ``pages`` fit; False when none is left to preempt."""

            nonlocal free_slots
            while not fits(pages):
                victim = next(
                    (
                        v
                        for v in reversed(running)
                        if v.request_id not in preempted_set
                        and v.request_id not in scheduled
                        and (v.arrival_ns, v.request_id) > (view.arrival_ns, view.request_id)
                    ),
                    None,
                )
                if victim is None:
                    return False
                preempted.append(victim.request_id)
                preempted_set.add(victim.request_id)
                held = capacity.held_blocks.get(victim.request_id, (0,) * len(free))
                for group in range(len(free)):
                    free[group] += held[group]
                free_slots += 1
            return True

        prefill_candidates = [v for v in ordered if v.status in (RequestStatus.WAITING, RequestStatus.PREFILLING)]
        can_admit_waiting = free_slots > 0 and capacity.min_free_blocks > 0
        has_progressable_prefill = any(
            v.status is RequestStatus.PREFILLING or can_admit_waiting for v in prefill_candidates
        )
        reserved_token = 1 if self.enable_chunked_prefill and has_progressable_prefill else 0

        # Requests that decode go first: one token each.
        for view in ordered:
            if view.status is not RequestStatus.DECODING or view.request_id in preempted_set:
                continue
            if token_budget <= reserved_token:
                break
            if view.next_input_token_id is None:
                raise RuntimeError("DECODING view has no pending input token.")
            pages = capacity.pages_for(view.computed_tokens, view.computed_tokens + 1)
            if not fits(pages) and not make_room(view, pages):
                continue     # the oldest blocked request waits for a page
            decode_items.append(DecodeItem(view.request_id, view.next_input_token_id, view.computed_tokens))
            scheduled.add(view.request_id)
            token_budget -= 1
            take(pages)

        # Then prompts: running ones continue, waiting ones are admitted while a slot is free.
        live_count = len(running) - len(preempted)
        for view in prefill_candidates:
            if view.request_id in preempted_set or token_budget <= 0:
                continue
            remaining = view.prefill_target - view.prefill_cursor
            if remaining <= 0:
                raise RuntimeError("Prefillable sequence has no remaining prompt tokens.")
            waiting = view.status is RequestStatus.WAITING
            if waiting and (free_slots <= 0 or live_count >= self.max_num_seqs):
                continue
            tokens = min(remaining, token_budget) if self.enable_chunked_prefill else remaining
            if self.prefill_chunk_size is not None:
                tokens = min(tokens, self.prefill_chunk_size)
            if tokens > token_budget:
                continue
            before = view.computed_tokens
            pages = capacity.pages_for(before, before + tokens)
            if not fits(pages) and not (not waiting and make_room(view, pages)):
                if not self.enable_chunked_prefill:
                    continue
                # the largest portion that the free pages hold: the rest of the
                # partly filled page plus whole free pages
                room = (-before) % block_size + max(min(free, default=0), 0) * block_size
                tokens = min(tokens, room)
                if tokens <= 0:
                    continue
                pages = capacity.pages_for(before, before + tokens)
            prefill_items.append(PrefillItem(view.request_id, view.prefill_cursor, view.prefill_cursor + tokens))
            scheduled.add(view.request_id)
            token_budget -= tokens
            take(pages)
            if waiting:
                free_slots -= 1
                live_count += 1

        return ExecutionPlan(
            step_id=step_id,
            prefill_items=tuple(prefill_items),
            decode_items=tuple(decode_items),
            scheduled_tokens=self.max_num_batched_tokens - token_budget,
            preempted=tuple(preempted),
        )
