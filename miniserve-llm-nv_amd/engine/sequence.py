"""One request's tokens and where it stands (reference: miniserve/engine/state.py:11-290).

The invariant of the reference is kept: a DECODING request always holds exactly
one sampled token that has not been run yet, ``total_tokens == computed_tokens + 1``.
Beyond the reference a running request can be *preempted*: it loses its cache and
goes back to WAITING; everything it holds so far (prompt and generated tokens) is
then run again as one prefill of ``prefill_target`` tokens.
"""

from __future__ import annotations

from dataclasses import dataclass
from enum import Enum, auto

from .request import Request, SamplingParams


class RequestStatus(Enum):
    WAITING = auto()
    PREFILLING = auto()
    DECODING = auto()
    FINISHED = auto()
    FAILED = auto()
    CANCELLED = auto()


TERMINAL = frozenset({RequestStatus.FINISHED, RequestStatus.FAILED, RequestStatus.CANCELLED})


@dataclass(frozen=True)
class SequenceView:
    """What the scheduler may read; it cannot change the request through it."""

    request_id: str
    status: RequestStatus
    prefill_target: int        # tokens to run before the next token can be sampled
    prefill_cursor: int
    computed_tokens: int
    total_tokens: int
    num_generated: int
    max_new_tokens: int
    arrival_ns: int
    next_input_token_id: int | None
    num_preemptions: int = 0


@dataclass
class SequenceState:
    request_id: str
    prompt_token_ids: tuple[int, ...]
    generated_token_ids: list[int]
    status: RequestStatus
    prefill_target: int
    prefill_cursor: int
    computed_tokens: int
    sampling_params: SamplingParams
    arrival_ns: int
    finish_reason: str | None = None
    error_message: str | None = None
    num_preemptions: int = 0

    @classmethod
    def from_request(cls, request: Request) -> "SequenceState":
        state = cls(
            request_id=request.request_id,
            prompt_token_ids=request.prompt_token_ids,
            generated_token_ids=[],
            status=RequestStatus.WAITING,
            prefill_target=len(request.prompt_token_ids),
            prefill_cursor=0,
            computed_tokens=0,
            sampling_params=request.sampling_params,
            arrival_ns=request.arrival_ns,
        )
        state.assert_invariants()
        return state

    @property
    def all_tokens(self) -> tuple[int, ...]:
        return self.prompt_token_ids + tuple(self.generated_token_ids)

    def token_at(self, index: int) -> int:
        """``all_tokens[index]`` without building the whole tuple (this is asked every step)."""

        prompt = len(self.prompt_token_ids)
        return self.prompt_token_ids[index] if index < prompt else self.generated_token_ids[index - prompt]

    def tokens_between(self, start: int, end: int) -> tuple[int, ...]:
        """``all_tokens[start:end]``."""

        prompt = len(self.prompt_token_ids)
        if end <= prompt:
            return self.prompt_token_ids[start:end]
        if start >= prompt:
            return tuple(self.generated_token_ids[start - prompt : end - prompt])
        return self.prompt_token_ids[start:] + tuple(self.generated_token_ids[: end - prompt])

    @property
    def total_tokens(self) -> int:
        return len(self.prompt_token_ids) + len(self.generated_token_ids)

    def snapshot(self) -> SequenceView:
        self.assert_invariants()
        return SequenceView(
            request_id=self.request_id,
            status=self.status,
            prefill_target=self.prefill_target,
            prefill_cursor=self.prefill_cursor,
            computed_tokens=self.computed_tokens,
            total_tokens=self.total_tokens,
            num_generated=len(self.generated_token_ids),
            max_new_tokens=self.sampling_params.max_new_tokens,
            arrival_ns=self.arrival_ns,
            next_input_token_id=(
                self.token_at(self.computed_tokens) if self.status is RequestStatus.DECODING else None
            ),
            num_preemptions=self.num_preemptions,
        )

    def view_after(self, *, prefill_end: int | None = None, decoded: bool = False, sampled: bool = False) -> SequenceView:
        """What :meth:`snapshot` will give once a running step is done: a step that ran
        this request's prompt up to ``prefill_end``, or its pending token
        (``decoded``), and that samples a token for it (``sampled``) which is not
        known yet, so ``next_input_token_id`` is 0 in its place."""

        computed = self.computed_tokens + 1 if decoded else self.computed_tokens if prefill_end is None else prefill_end
        if sampled:
            status = RequestStatus.DECODING
        elif prefill_end is not None:
            status = RequestStatus.PREFILLING
        else:
            status = self.status
        return SequenceView(
            request_id=self.request_id,
            status=status,
            prefill_target=self.prefill_target,
            prefill_cursor=self.prefill_cursor if prefill_end is None else prefill_end,
            computed_tokens=computed,
            total_tokens=self.total_tokens + int(sampled),
            num_generated=len(self.generated_token_ids) + int(sampled),
            max_new_tokens=self.sampling_params.max_new_tokens,
            arrival_ns=self.arrival_ns,
            next_input_token_id=(
                0 if sampled else self.token_at(self.computed_tokens) if status is RequestStatus.DECODING else None
            ),
            num_preemptions=self.num_preemptions,
        )

    # ---- transitions ------------------------------------------------------------------
    def begin_prefill(self) -> None:
        if self.status is not RequestStatus.WAITING:
            raise RuntimeError("Only a waiting sequence can begin prefill.")
        self.status = RequestStatus.PREFILLING
        self.assert_invariants()

    def commit_prefill(self, token_end: int) -> None:
        """A portion of the prefill has run; a portion that does not end the prefill samples nothing."""

        if self.status is not RequestStatus.PREFILLING:
            raise RuntimeError("Prompt completion requires PREFILLING state.")
        if not self.prefill_cursor < token_end <= self.prefill_target:
            raise RuntimeError("Prefill commit must advance within the prompt.")
        self.prefill_cursor = token_end
        self.computed_tokens = token_end
        self.assert_invariants()

    def mark_decode_input_computed(self) -> None:
        if self.status is not RequestStatus.DECODING or self.computed_tokens != self.total_tokens - 1:
            raise RuntimeError("Decode must consume exactly the pending sampled token.")
        self.computed_tokens += 1

    def append_sampled_token(self, token_id: int) -> None:
        if self.status is not RequestStatus.PREFILLING and self.status is not RequestStatus.DECODING:
            raise RuntimeError("A token can only be sampled after model execution.")
        if self.computed_tokens != self.total_tokens:
            raise RuntimeError("All current tokens must be computed before sampling the next token.")
        if not isinstance(token_id, int) or isinstance(token_id, bool) or token_id < 0:
            raise ValueError("token_id must be a non-negative integer.")
        self.generated_token_ids.append(token_id)
        self.status = RequestStatus.DECODING
        self.assert_invariants()

    def should_finish(self) -> str | None:
        """"stop" when the last token is a stop token (it stays in the output but is
        never run), else "length" at ``max_new_tokens`` (reference: state.py:148-155)."""

        if not self.generated_token_ids:
            return None
        if self.generated_token_ids[-1] in self.sampling_params.stop_token_ids:
            return "stop"
        if len(self.generated_token_ids) >= self.sampling_params.max_new_tokens:
            return "length"
        return None

    def finish(self, reason: str) -> None:
        if self.status is not RequestStatus.DECODING:
            raise RuntimeError("Only a decoding sequence can finish normally.")
        if reason not in {"stop", "length"}:
            raise ValueError("Normal finish reason must be 'stop' or 'length'.")
        self.status = RequestStatus.FINISHED
        self.finish_reason = reason
        self.assert_invariants()

    def preempt(self) -> None:
        """Lose the cache, keep the tokens: back to WAITING, all tokens to be run again."""

        if self.status not in {RequestStatus.PREFILLING, RequestStatus.DECODING}:
            raise RuntimeError("Only a running sequence can be preempted.")
        self.status = RequestStatus.WAITING
        self.prefill_target = self.total_tokens
        self.prefill_cursor = 0
        self.computed_tokens = 0
        self.num_preemptions += 1
        self.assert_invariants()

    def cancel(self, reason: str = "cancelled") -> None:
        if self.status in TERMINAL:
            raise RuntimeError("Terminal sequence cannot be cancelled again.")
        self.status = RequestStatus.CANCELLED
        self.finish_reason = reason

    def fail(self, message: str) -> None:
        if self.status in TERMINAL:
            raise RuntimeError("Terminal sequence cannot transition to FAILED.")
        if not isinstance(message, str) or not message.strip():
            raise ValueError("failure message must not be empty.")
        self.status = RequestStatus.FAILED
        self.finish_reason = "error"
        self.error_message = message

    # ---- invariants -------------------------------------------------------------------
    def assert_invariants(self) -> None:
        if not self.request_id or not self.prompt_token_ids:
            raise AssertionError("Sequence identity and prompt must be non-empty.")
        if not len(self.prompt_token_ids) <= self.prefill_target <= self.total_tokens:
            raise AssertionError("prefill_target lies outside the sequence.")
        if not 0 <= self.prefill_cursor <= self.prefill_target:
            raise AssertionError("prefill_cursor is outside the prefill.")
        if not 0 <= self.computed_tokens <= self.total_tokens:
            raise AssertionError("computed_tokens is outside all_tokens.")
        if len(self.generated_token_ids) > self.sampling_params.max_new_tokens:
            raise AssertionError("generated tokens exceed max_new_tokens.")
        status = self.status          # identity tests: hashing an enum member costs a Python call
        if status is RequestStatus.WAITING or status is RequestStatus.PREFILLING:
            if self.computed_tokens != self.prefill_cursor or self.prefill_target != self.total_tokens:
                raise AssertionError("WAITING/PREFILLING only advances the prefill of all current tokens.")
            if status is RequestStatus.WAITING and self.computed_tokens != 0:
                raise AssertionError("WAITING holds no computed tokens.")
        elif status is RequestStatus.DECODING or status is RequestStatus.FINISHED:
            if not self.generated_token_ids or self.computed_tokens != self.total_tokens - 1:
                raise AssertionError("Decode/finish must retain one sampled, uncomputed token.")
        if status is RequestStatus.FINISHED and self.finish_reason not in {"stop", "length"}:
            raise AssertionError("FINISHED state requires a normal finish reason.")
        if status is RequestStatus.FAILED and (self.finish_reason != "error" or not self.error_message):
            raise AssertionError("FAILED state requires a separate diagnostic message.")
