"""One request inside the engine: the tokens it holds and how far they have run.

Two numbers carry the whole state machine.  ``computed_tokens`` counts the tokens
whose keys and values lie in the cache; ``prefill_target`` is how many must lie
there before the next token may be sampled (the prompt; after a preemption,
everything the request holds).  From them:

    WAITING      nothing computed, no cache held
    PREFILLING   computed <= target == all tokens held; nothing sampled is pending
    DECODING     exactly one sampled token is held that has not run: computed == held - 1
    FINISHED     as DECODING, with a reason ("stop" or "length"); the last token never runs
    FAILED / CANCELLED   terminal, whatever the numbers were

The phases and the rule of the one pending token are the reference's
(miniserve/engine/state.py:11-290); preemption (back to WAITING with all tokens to
run again) is this engine's own.
"""

from __future__ import annotations

from dataclasses import dataclass, field
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
RUNNING = frozenset({RequestStatus.PREFILLING, RequestStatus.DECODING})
NORMAL_ENDS = ("stop", "length")


class TransitionError(RuntimeError):
    """A step asked a request for something its phase does not allow."""


@dataclass(frozen=True)
class SequenceView:
    """The numbers of a request that the scheduler decides by.  A view is a copy: the
    scheduler cannot change a request through it, and a view may describe a request as
    a running step will leave it."""

    request_id: str
    status: RequestStatus
    prefill_target: int
    computed_tokens: int
    total_tokens: int
    num_generated: int
    max_new_tokens: int
    arrival_ns: int
    next_input_token_id: int | None        # DECODING: the pending token (0 where it is not known yet)
    num_preemptions: int = 0

    @property
    def age_key(self) -> tuple[int, str]:
        """Older requests sort first; the id breaks ties of the clock."""

        return (self.arrival_ns, self.request_id)


@dataclass
class SequenceState:
    request: Request
    generated_token_ids: list[int] = field(default_factory=list)
    status: RequestStatus = RequestStatus.WAITING
    computed_tokens: int = 0
    prefill_target: int = 0
    finish_reason: str | None = None
    error_message: str | None = None
    num_preemptions: int = 0

    @classmethod
    def from_request(cls, request: Request) -> "SequenceState":
        return cls(request=request, prefill_target=len(request.prompt_token_ids))

    # ---- what it holds ----------------------------------------------------------------
    @property
    def request_id(self) -> str:
        return self.request.request_id

    @property
    def prompt_token_ids(self) -> tuple[int, ...]:
        return self.request.prompt_token_ids

    @property
    def sampling_params(self) -> SamplingParams:
        return self.request.sampling_params

    @property
    def arrival_ns(self) -> int:
        return self.request.arrival_ns

    @property
    def total_tokens(self) -> int:
        return len(self.request.prompt_token_ids) + len(self.generated_token_ids)

    @property
    def all_tokens(self) -> tuple[int, ...]:
        return self.request.prompt_token_ids + tuple(self.generated_token_ids)

    def token_at(self, index: int) -> int:
        """Token ``index`` of prompt + generated, without joining the two."""

        prompt = self.request.prompt_token_ids
        return prompt[index] if index < len(prompt) else self.generated_token_ids[index - len(prompt)]

    def tokens_between(self, start: int, end: int) -> tuple[int, ...]:
        """Tokens ``[start, end)`` of prompt + generated."""

        prompt = self.request.prompt_token_ids
        from_prompt = prompt[start:end] if start < len(prompt) else ()
        if end <= len(prompt):
            return from_prompt
        return from_prompt + tuple(self.generated_token_ids[max(start - len(prompt), 0) : end - len(prompt)])

    # ---- views ------------------------------------------------------------------------
    def _view(self, status: RequestStatus, computed: int, sampled_ahead: bool) -> SequenceView:
        pending = None
        if status is RequestStatus.DECODING:
            pending = 0 if sampled_ahead else self.token_at(computed)
        return SequenceView(
            request_id=self.request_id,
            status=status,
            prefill_target=self.prefill_target,
            computed_tokens=computed,
            total_tokens=self.total_tokens + int(sampled_ahead),
            num_generated=len(self.generated_token_ids) + int(sampled_ahead),
            max_new_tokens=self.sampling_params.max_new_tokens,
            arrival_ns=self.arrival_ns,
            next_input_token_id=pending,
            num_preemptions=self.num_preemptions,
        )

    def snapshot(self) -> SequenceView:
        """The request as it stands."""

        self.check()
        return self._view(self.status, self.computed_tokens, False)

    def view_after(self, *, prefill_end: int | None = None, decoded: bool = False, sampled: bool = False) -> SequenceView:
        """The request as a step that is still running will leave it: a step that runs
        its tokens up to ``prefill_end``, or its pending token (``decoded``), and that
        samples a token for it (``sampled``) whose id is not known yet."""

        if decoded:
            computed = self.computed_tokens + 1
        elif prefill_end is not None:
            computed = prefill_end
        else:
            computed = self.computed_tokens
        if sampled:
            status = RequestStatus.DECODING
        elif prefill_end is not None:
            status = RequestStatus.PREFILLING
        else:
            status = self.status
        return self._view(status, computed, sampled)

    # ---- what a step does to it -----------------------------------------------------------
    def _expect(self, *phases: RequestStatus, to: str) -> None:
        if self.status not in phases:
            names = " or ".join(phase.name for phase in phases)
            raise TransitionError(f"request {self.request_id!r} is {self.status.name}; only a {names} request can {to}.")

    def admitted(self) -> None:
        """Admitted: it holds a cache slot and starts running its tokens."""

        self._expect(RequestStatus.WAITING, to="be admitted")
        self.status = RequestStatus.PREFILLING

    def ran_to(self, token_end: int) -> None:
        """A step ran its tokens up to ``token_end``.  Nothing is sampled unless that is the target."""

        self._expect(RequestStatus.PREFILLING, to="run a portion of its tokens")
        if not self.computed_tokens < token_end <= self.prefill_target:
            raise TransitionError(
                f"request {self.request_id!r}: a portion ending at {token_end} does not move it forward from "
                f"{self.computed_tokens} within its {self.prefill_target} tokens."
            )
        self.computed_tokens = token_end

    def ran_pending_token(self) -> None:
        """A step ran the one pending token."""

        self._expect(RequestStatus.DECODING, to="run its pending token")
        if self.computed_tokens != self.total_tokens - 1:
            raise TransitionError(f"request {self.request_id!r} holds no single pending token to run.")
        self.computed_tokens += 1

    def take_token(self, token_id: int) -> None:
        """The token sampled from the logits of its last computed position."""

        self._expect(*RUNNING, to="take a sampled token")
        if self.computed_tokens != self.total_tokens:
            raise TransitionError(
                f"request {self.request_id!r}: {self.total_tokens - self.computed_tokens} of its tokens have not run; "
                "a token is sampled only after all of them."
            )
        if type(token_id) is not int or token_id < 0:
            raise ValueError(f"a sampled token id is a whole number, not {token_id!r}.")
        self.generated_token_ids.append(token_id)
        self.status = RequestStatus.DECODING
        self.check()

    def ending(self) -> str | None:
        """Why the request ends with the token it took last, if it does: ``"stop"``
        for a stop token (which stays in the output and never runs), ``"length"`` at
        ``max_new_tokens``; a stop token at the length limit counts as ``"stop"``."""

        if not self.generated_token_ids:
            return None
        params = self.sampling_params
        if self.generated_token_ids[-1] in params.stop_token_ids:
            return "stop"
        return "length" if len(self.generated_token_ids) >= params.max_new_tokens else None

    def finish(self, reason: str) -> None:
        self._expect(RequestStatus.DECODING, to="end normally")
        if reason not in NORMAL_ENDS:
            raise ValueError(f"a request ends normally by one of {NORMAL_ENDS}, not {reason!r}.")
        self.status, self.finish_reason = RequestStatus.FINISHED, reason

    def preempt(self) -> None:
        """It loses its cache and keeps its tokens: all of them run again, later, as one
        prefill, after which the next token is sampled as if nothing had happened."""

        self._expect(*RUNNING, to="be preempted")
        self.status = RequestStatus.WAITING
        self.prefill_target = self.total_tokens
        self.computed_tokens = 0
        self.num_preemptions += 1

    def cancel(self, reason: str = "cancelled") -> None:
        if self.status in TERMINAL:
            raise TransitionError(f"request {self.request_id!r} has ended ({self.status.name}) and cannot be cancelled.")
        self.status, self.finish_reason = RequestStatus.CANCELLED, reason

    def fail(self, message: str) -> None:
        if self.status in TERMINAL:
            raise TransitionError(f"request {self.request_id!r} has ended ({self.status.name}) and cannot fail.")
        if not isinstance(message, str) or not message.strip():
            raise ValueError("a failed request needs a message that says why.")
        self.status, self.finish_reason, self.error_message = RequestStatus.FAILED, "error", message

    # ---- consistency ------------------------------------------------------------------------
    def problems(self) -> list[str]:
        """Everything about the numbers that does not fit the phase (empty when all is well)."""

        found = []
        held, done, target = self.total_tokens, self.computed_tokens, self.prefill_target
        prompt = len(self.request.prompt_token_ids)
        if not prompt <= target <= held:
            found.append(f"target {target} lies outside prompt {prompt} .. held {held}")
        if not 0 <= done <= held:
            found.append(f"{done} tokens computed of {held} held")
        if len(self.generated_token_ids) > self.sampling_params.max_new_tokens:
            found.append(f"{len(self.generated_token_ids)} tokens generated, {self.sampling_params.max_new_tokens} allowed")
        status = self.status
        if status is RequestStatus.WAITING and done != 0:
            found.append(f"waiting with {done} tokens computed")
        if status is RequestStatus.WAITING or status is RequestStatus.PREFILLING:
            if target != held or done > target:
                found.append(f"{status.name}: target {target}, held {held}, computed {done}")
        elif status is RequestStatus.DECODING or status is RequestStatus.FINISHED:
            if not self.generated_token_ids or done != held - 1:
                found.append(f"{status.name}: {done} computed of {held} held; exactly one sampled token must be pending")
        if status is RequestStatus.FINISHED and self.finish_reason not in NORMAL_ENDS:
            found.append(f"finished by {self.finish_reason!r}")
        if status is RequestStatus.FAILED and (self.finish_reason != "error" or not self.error_message):
            found.append("failed without a message")
        return found

    def check(self) -> None:
        found = self.problems()
        if found:
            raise AssertionError(f"request {self.request_id!r} is inconsistent: " + "; ".join(found))

