"""What the scheduler decides for one step, as plain integers
(reference: miniserve/engine/plan.py:8-84)."""

from __future__ import annotations

from dataclasses import dataclass


def _is_int(value: object) -> bool:
    return isinstance(value, int) and not isinstance(value, bool)


@dataclass(frozen=True)
class PrefillItem:
    """Run tokens ``[token_start, token_end)`` of the request's sequence."""

    request_id: str
    token_start: int
    token_end: int

    def __post_init__(self) -> None:
        if (
            not self.request_id
            or not _is_int(self.token_start)
            or not _is_int(self.token_end)
            or self.token_start < 0
            or self.token_end <= self.token_start
        ):
            raise ValueError("Invalid prefill item.")


@dataclass(frozen=True)
class DecodeItem:
    """Run the pending sampled token ``input_token_id`` at ``position``."""

    request_id: str
    input_token_id: int
    position: int

    def __post_init__(self) -> None:
        if (
            not self.request_id
            or not _is_int(self.input_token_id)
            or not _is_int(self.position)
            or self.input_token_id < 0
            or self.position < 0
        ):
            raise ValueError("Invalid decode item.")


@dataclass(frozen=True)
class ExecutionPlan:
    step_id: int
    prefill_items: tuple[PrefillItem, ...] = ()
    decode_items: tuple[DecodeItem, ...] = ()
    scheduled_tokens: int = 0
    preempted: tuple[str, ...] = ()      # requests that lose their cache before the step runs

    def __post_init__(self) -> None:
        if not _is_int(self.step_id) or not _is_int(self.scheduled_tokens) or self.step_id < 0 or self.scheduled_tokens < 0:
            raise ValueError("step_id and scheduled_tokens must be non-negative.")
        if not isinstance(self.prefill_items, tuple) or not isinstance(self.decode_items, tuple):
            raise TypeError("ExecutionPlan items must be immutable tuples.")
        if any(not isinstance(item, PrefillItem) for item in self.prefill_items) or any(
            not isinstance(item, DecodeItem) for item in self.decode_items
        ):
            raise TypeError("ExecutionPlan contains an invalid item type.")
        request_ids = [item.request_id for item in (*self.prefill_items, *self.decode_items)]
        if len(request_ids) != len(set(request_ids)):
            raise ValueError("A request may appear only once in one ExecutionPlan.")
        if set(request_ids) & set(self.preempted):
            raise ValueError("A preempted request cannot run in the same step.")
        expected = sum(item.token_end - item.token_start for item in self.prefill_items) + len(self.decode_items)
        if self.scheduled_tokens != expected:
            raise ValueError("scheduled_tokens does not match plan items.")

    @property
    def empty(self) -> bool:
        return not self.prefill_items and not self.decode_items
