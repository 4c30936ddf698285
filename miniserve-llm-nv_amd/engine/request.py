"""What a caller hands to the engine: sampling parameters and a tokenised request
(reference: miniserve/engine/request.py:9-89; same names, defaults and bounds)."""

from __future__ import annotations

import math
from dataclasses import dataclass


def _is_int(value: object) -> bool:
    return isinstance(value, int) and not isinstance(value, bool)


def _is_number(value: object) -> bool:
    return isinstance(value, (int, float)) and not isinstance(value, bool) and math.isfinite(value)


@dataclass(frozen=True)
class SamplingParams:
    """``temperature == 0`` is greedy; above zero the order is temperature, top-k,
    top-p, one draw.  ``seed`` None means a fresh random seed per request."""

    temperature: float = 0.0
    top_p: float = 1.0
    top_k: int = 0
    max_new_tokens: int = 4
    stop_token_ids: tuple[int, ...] = ()
    seed: int | None = None

    def __post_init__(self) -> None:
        if not _is_number(self.temperature) or not 0 <= self.temperature <= 2:
            raise ValueError("temperature must be finite and in [0, 2].")
        if not _is_number(self.top_p) or not 0 < self.top_p <= 1:
            raise ValueError("top_p must be in (0, 1].")
        if not _is_int(self.top_k) or self.top_k < 0:
            raise ValueError("top_k must be non-negative.")
        if not _is_int(self.max_new_tokens) or self.max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be positive.")
        if not isinstance(self.stop_token_ids, tuple):
            raise ValueError("stop_token_ids must be an immutable tuple.")
        if any(not _is_int(token) or token < 0 for token in self.stop_token_ids):
            raise ValueError("stop_token_ids must contain non-negative integers.")
        if len(set(self.stop_token_ids)) != len(self.stop_token_ids):
            raise ValueError("stop_token_ids must not contain duplicates.")
        if self.seed is not None and (not _is_int(self.seed) or not 0 <= self.seed <= 2**63 - 1):
            raise ValueError("seed must be an integer in [0, 2^63-1] or None.")


@dataclass(frozen=True)
class Request:
    request_id: str
    prompt_token_ids: tuple[int, ...]
    sampling_params: SamplingParams
    arrival_ns: int

    def __post_init__(self) -> None:
        if not isinstance(self.request_id, str) or not self.request_id.strip():
            raise ValueError("request_id must not be empty.")
        if not isinstance(self.prompt_token_ids, tuple) or not self.prompt_token_ids:
            raise ValueError("prompt_token_ids must not be empty.")
        if any(not _is_int(token) or token < 0 for token in self.prompt_token_ids):
            raise ValueError("prompt_token_ids must contain non-negative integers.")
        if not isinstance(self.sampling_params, SamplingParams):
            raise ValueError("sampling_params must be a SamplingParams instance.")
        if not _is_int(self.arrival_ns) or self.arrival_ns < 0:
            raise ValueError("arrival_ns must be non-negative.")
