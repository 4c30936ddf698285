"""What the scheduler decides for one step, as plain integers: which requests run
a portion of their prompt, which run their pending sampled token, and which lose
their cache first.  The plan carries no tensors and no references into the engine,
so it can be made from views, logged, compared and replayed
(the reference's counterpart: miniserve/engine/plan.py:8-84).
"""

from __future__ import annotations

from dataclasses import dataclass


def _whole_number(value: object) -> bool:
    """A Python int that is not a bool and not negative."""

    return type(value) is int and value >= 0


def _named(request_id: object, what: str) -> None:
    if not isinstance(request_id, str) or not request_id:
        raise ValueError(f"a {what} needs the id of its request, got {request_id!r}.")


@dataclass(frozen=True)
class PrefillItem:
    """Run tokens ``[token_start, token_end)`` of the request's sequence."""

    request_id: str
    token_start: int
    token_end: int

    def __post_init__(self) -> None:
        _named(self.request_id, "prompt portion")
        if not (_whole_number(self.token_start) and _whole_number(self.token_end) and self.token_start < self.token_end):
            raise ValueError(
                f"prompt portion of {self.request_id!r}: [{self.token_start!r}, {self.token_end!r}) is no run of tokens."
            )

    @property
    def num_tokens(self) -> int:
        return self.token_end - self.token_start


@dataclass(frozen=True)
class DecodeItem:
    """Run the pending sampled token ``input_token_id`` at ``position``."""

    request_id: str
    input_token_id: int
    position: int

    def __post_init__(self) -> None:
        _named(self.request_id, "decode item")
        if not (_whole_number(self.input_token_id) and _whole_number(self.position)):
            raise ValueError(
                f"decode item of {self.request_id!r}: token {self.input_token_id!r} at position {self.position!r} "
                "must both be whole numbers."
            )

    num_tokens = 1


@dataclass(frozen=True)
class ExecutionPlan:
    """One step.  ``preempted`` requests give their pages and their slot back before
    the step runs and take no part in it; ``scheduled_tokens`` is the number of tokens
    the step runs, kept beside the items so that a reader need not add them up and a
    writer cannot get it wrong unnoticed."""

    step_id: int
    prefill_items: tuple[PrefillItem, ...] = ()
    decode_items: tuple[DecodeItem, ...] = ()
    scheduled_tokens: int = 0
    preempted: tuple[str, ...] = ()

    def __post_init__(self) -> None:
        for name, kind in (("prefill_items", PrefillItem), ("decode_items", DecodeItem)):
            items = getattr(self, name)
            if type(items) is not tuple:
                raise TypeError(f"ExecutionPlan.{name} is a {type(items).__name__}; a plan is immutable and takes tuples.")
            strangers = [type(item).__name__ for item in items if type(item) is not kind]
            if strangers:
                raise TypeError(f"ExecutionPlan.{name} holds {strangers[0]} where {kind.__name__} belongs.")
        if not _whole_number(self.step_id) or not _whole_number(self.scheduled_tokens):
            raise ValueError(f"step {self.step_id!r} with {self.scheduled_tokens!r} tokens: both must be whole numbers.")
        running = self.request_ids
        twice = {request_id for request_id in running if running.count(request_id) > 1}
        if twice:
            raise ValueError(f"requests {sorted(twice)} stand more than once in step {self.step_id}.")
        both = set(running) & set(self.preempted)
        if both:
            raise ValueError(f"requests {sorted(both)} are preempted and run in the same step {self.step_id}.")
        counted = sum(item.num_tokens for item in self.prefill_items) + len(self.decode_items)
        if counted != self.scheduled_tokens:
            raise ValueError(f"step {self.step_id} says {self.scheduled_tokens} tokens, its items hold {counted}.")

    @property
    def request_ids(self) -> tuple[str, ...]:
        """The requests that run, decoding ones first (the order of the batch)."""

        return tuple(item.request_id for item in (*self.decode_items, *self.prefill_items))

    @property
    def empty(self) -> bool:
        return not self.prefill_items and not self.decode_items
