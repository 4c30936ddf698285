"""What a caller hands to the engine: sampling parameters and a tokenised request.

The option names, their defaults and their bounds are those of the reference's
request schema (miniserve/engine/request.py:9-89), since a user of one should find
the other familiar; values are taken as given, never coerced (``True`` is no
integer, ``"0.7"`` no number).  Each field's rule is one row of a table, and a
refused value is named in the error.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, fields
from typing import Any, Callable

MAX_SEED = 2**63 - 1


def _integer(value: Any) -> bool:
    return type(value) is int


def _real(value: Any) -> bool:
    return type(value) in (int, float) and math.isfinite(value)


def _token_tuple(value: Any) -> bool:
    return type(value) is tuple and all(_integer(token) and token >= 0 for token in value)


# field -> (rule, what the rule asks for)
_SAMPLING_RULES: dict[str, tuple[Callable[[Any], bool], str]] = {
    "temperature": (lambda v: _real(v) and 0 <= v <= 2, "a finite number from 0 (greedy) to 2"),
    "top_p": (lambda v: _real(v) and 0 < v <= 1, "a number above 0 and at most 1 (1 switches it off)"),
    "top_k": (lambda v: _integer(v) and v >= 0, "a whole number (0 switches it off)"),
    "max_new_tokens": (lambda v: _integer(v) and v > 0, "a positive whole number"),
    "stop_token_ids": (
        lambda v: _token_tuple(v) and len(set(v)) == len(v),
        "a tuple of distinct token ids (whole numbers)",
    ),
    "seed": (lambda v: v is None or (_integer(v) and 0 <= v <= MAX_SEED), "None or a whole number below 2^63"),
}

_REQUEST_RULES: dict[str, tuple[Callable[[Any], bool], str]] = {
    "request_id": (lambda v: isinstance(v, str) and bool(v.strip()), "a string that is not blank"),
    "prompt_token_ids": (lambda v: _token_tuple(v) and len(v) > 0, "a tuple of at least one token id (whole numbers)"),
    "sampling_params": (lambda v: isinstance(v, SamplingParams), "a SamplingParams"),
    "arrival_ns": (lambda v: _integer(v) and v >= 0, "a whole number of nanoseconds"),
}


def _apply(rules: dict, record: Any) -> None:
    for spec in fields(record):
        rule, asks_for = rules[spec.name]
        value = getattr(record, spec.name)
        if not rule(value):
            raise ValueError(f"{type(record).__name__}.{spec.name} = {value!r}: it must be {asks_for}.")


@dataclass(frozen=True)
class SamplingParams:
    """How the next token is chosen.  ``temperature == 0``: the largest logit, lowest
    id among equals.  Above zero: divide the logits by it, keep the ``top_k``
    largest, then the smallest set whose probability reaches ``top_p``, and draw
    once.  ``seed``: the request's own random stream; None draws a fresh seed."""

    temperature: float = 0.0
    top_p: float = 1.0
    top_k: int = 0
    max_new_tokens: int = 4
    stop_token_ids: tuple[int, ...] = ()
    seed: int | None = None

    def __post_init__(self) -> None:
        _apply(_SAMPLING_RULES, self)

    @property
    def greedy(self) -> bool:
        return self.temperature == 0


@dataclass(frozen=True)
class Request:
    """A prompt as token ids (the tokenizer stays outside the engine), its sampling
    parameters and the time it arrived, which orders the queue."""

    request_id: str
    prompt_token_ids: tuple[int, ...]
    sampling_params: SamplingParams
    arrival_ns: int

    def __post_init__(self) -> None:
        _apply(_REQUEST_RULES, self)
