"""The scheduler: which requests run in the next step, and with how many tokens.

Policy (that of the reference's ``ContinuousBatchScheduler``,
miniserve/engine/scheduler.py:129-227): oldest first by ``(arrival, id)``; requests
that decode go first, one token each; then prompts, whole, or in portions under the
token budget when chunked prefill is on; when chunked prefill is on and a prompt
can move, one token of the budget is held back for it so that decoding cannot starve it.

What happens when pages run out is decided here, where the reference only skips the
request (scheduler.py:167-172, 203-210) and can stall for good: a running request
that needs a page and finds none takes the pages of the YOUNGEST running request
that is younger than itself, which is *preempted* (it loses its cache and waits; its
tokens are run again later).  The oldest running request is never preempted, so it
always finishes.  A running request that finds no younger one to preempt waits for a
step.  Waiting requests never preempt anyone; they are admitted only while a state
slot is free.

``schedule`` is a pure function of views and a capacity snapshot.  Its bookkeeping
for one call lives in a ``_Ledger``: what the step has taken so far of the three
budgets (tokens, live requests, pages per group) and who was preempted for it.
"""

from __future__ import annotations

from collections.abc import Sequence

from ..cache.manager import CapacitySnapshot
from .plan import DecodeItem, ExecutionPlan, PrefillItem
from .sequence import RUNNING, RequestStatus, SequenceView


class _Ledger:
    """The budgets of one call of ``schedule``, as they shrink."""

    def __init__(self, capacity: CapacitySnapshot, running: list[SequenceView], tokens: int, max_live: int) -> None:
        self.capacity = capacity
        self.running = running                       # oldest first
        self.tokens = tokens
        self.free_pages = list(capacity.free_blocks)  # an estimate per group: the cache manager has the last word
        self.free_slots = capacity.free_slots
        self.live = len(running)
        self.max_live = max_live
        self.preempted: list[str] = []
        self.planned: set[str] = set()

    def holds(self, pages: Sequence[int]) -> bool:
        return all(wanted <= free for wanted, free in zip(pages, self.free_pages))

    def spend(self, view: SequenceView, tokens: int, pages: Sequence[int]) -> None:
        self.planned.add(view.request_id)
        self.tokens -= tokens
        self.free_pages = [free - wanted for free, wanted in zip(self.free_pages, pages)]

    def preempt_for(self, view: SequenceView, pages: Sequence[int]) -> bool:
        """Takes the caches of the youngest running requests that are younger than
        ``view`` and not part of this step, one by one, until ``pages`` fit.  False
        when there is nobody left to take from (what was taken stays taken: those
        requests were the youngest, and the next step finds the room)."""

        while not self.holds(pages):
            victim = None
            for candidate in reversed(self.running):
                if candidate.age_key <= view.age_key:
                    break
                if candidate.request_id not in self.planned and candidate.request_id not in self.preempted:
                    victim = candidate
                    break
            if victim is None:
                return False
            self.preempted.append(victim.request_id)
            held = self.capacity.held_blocks.get(victim.request_id, ())
            self.free_pages = [free + (held[group] if group < len(held) else 0) for group, free in enumerate(self.free_pages)]
            self.free_slots += 1
            self.live -= 1
        return True


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
            raise ValueError("max_num_seqs and max_num_batched_tokens must be positive.")
        if prefill_chunk_size is not None:
            if type(prefill_chunk_size) is not int or prefill_chunk_size <= 0:
                raise ValueError("prefill_chunk_size is a positive whole number or None.")
            if not enable_chunked_prefill:
                raise ValueError("prefill_chunk_size has a meaning only with enable_chunked_prefill.")
            if prefill_chunk_size > max_num_batched_tokens:
                raise ValueError("a portion of prefill_chunk_size tokens would not fit max_num_batched_tokens.")
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens
        self.enable_chunked_prefill = enable_chunked_prefill
        self.prefill_chunk_size = prefill_chunk_size
        self._steps_planned = 0

    def schedule(self, sequences: Sequence[SequenceView], capacity: CapacitySnapshot) -> ExecutionPlan:
        step_id = self._steps_planned
        self._steps_planned += 1
        by_age = sorted(sequences, key=lambda view: view.age_key)
        ledger = _Ledger(
            capacity, [view for view in by_age if view.status in RUNNING], self.max_num_batched_tokens, self.max_num_seqs
        )
        decoding = [view for view in by_age if view.status is RequestStatus.DECODING]
        prompts = [view for view in by_age if view.status in (RequestStatus.WAITING, RequestStatus.PREFILLING)]

        decode_items = self._plan_decoding(decoding, ledger, held_back=self._token_held_back(prompts, capacity))
        prefill_items = self._plan_prompts(prompts, ledger)
        return ExecutionPlan(
            step_id=step_id,
            prefill_items=tuple(prefill_items),
            decode_items=tuple(decode_items),
            scheduled_tokens=self.max_num_batched_tokens - ledger.tokens,
            preempted=tuple(ledger.preempted),
        )

    def _token_held_back(self, prompts: list[SequenceView], capacity: CapacitySnapshot) -> int:
        """With chunked prefill, one token of the budget belongs to the prompts as long
        as one of them can move at all: one that is running, or a waiting one while a
        slot and a page are free."""

        if not self.enable_chunked_prefill:
            return 0
        a_waiting_one_fits = capacity.free_slots > 0 and capacity.min_free_blocks > 0
        can_move = any(view.status is RequestStatus.PREFILLING or a_waiting_one_fits for view in prompts)
        return 1 if can_move else 0

    def _plan_decoding(self, decoding: list[SequenceView], ledger: _Ledger, *, held_back: int) -> list[DecodeItem]:
        items = []
        for view in decoding:
            if view.request_id in ledger.preempted:
                continue
            if ledger.tokens <= held_back:
                break
            if view.next_input_token_id is None:
                raise RuntimeError(f"request {view.request_id!r} decodes but names no pending token.")
            pages = ledger.capacity.pages_for(view.computed_tokens, view.computed_tokens + 1)
            if not ledger.holds(pages) and not ledger.preempt_for(view, pages):
                continue            # nobody younger to take a page from: it waits a step
            items.append(DecodeItem(view.request_id, view.next_input_token_id, view.computed_tokens))
            ledger.spend(view, 1, pages)
        return items

    def _plan_prompts(self, prompts: list[SequenceView], ledger: _Ledger) -> list[PrefillItem]:
        items = []
        for view in prompts:
            if view.request_id in ledger.preempted or ledger.tokens <= 0:
                continue
            start = view.computed_tokens
            left = view.prefill_target - start
            if left <= 0:
                raise RuntimeError(f"request {view.request_id!r} has no tokens left to run before sampling.")
            newcomer = view.status is RequestStatus.WAITING
            if newcomer and (ledger.free_slots <= 0 or ledger.live >= ledger.max_live):
                continue
            tokens = left
            if self.enable_chunked_prefill:
                tokens = min(tokens, ledger.tokens, self.prefill_chunk_size or tokens)
            if tokens > ledger.tokens:
                continue            # whole prompts only, and this one does not fit the step
            pages = ledger.capacity.pages_for(start, start + tokens)
            if not ledger.holds(pages) and (newcomer or not ledger.preempt_for(view, pages)):
                if not self.enable_chunked_prefill:
                    continue
                # as much as the free pages hold: the rest of its last page and every free page
                tokens = min(tokens, ledger.capacity.room_for(start, ledger.free_pages))
                if tokens <= 0:
                    continue
                pages = ledger.capacity.pages_for(start, start + tokens)
            items.append(PrefillItem(view.request_id, start, start + tokens))
            ledger.spend(view, tokens, pages)
            if newcomer:
                ledger.free_slots -= 1
                ledger.live += 1
        return items
