"""Choosing the next token: greedy, or temperature -> top-k -> top-p -> one draw,
with one random stream per request (reference: miniserve/model/sampling.py:61-242).

The choice itself is made on the device by ``ops.sample_rows``; the host keeps
the per-request generators and draws ONE uniform number per sampled token from
them.  As in the reference, a draw is *staged*: the generator advances only when
the step that produced the logits is committed.
"""

from __future__ import annotations

import os
from dataclasses import dataclass
from typing import TYPE_CHECKING, Sequence

import numpy as np
import torch

if TYPE_CHECKING:       # for the annotations only: the engine package imports this one
    from ..engine.request import SamplingParams

_BELOW_ONE = 1.0 - 2.0**-24      # largest float32 below 1


@dataclass(frozen=True)
class StagedSample:
    request_id: str
    token_id: int
    generator_state: torch.Tensor | None      # None: greedy, no randomness used


class NonFiniteLogitsError(ValueError):
    pass


class Sampler:
    def __init__(self) -> None:
        self._generators: dict[str, torch.Generator] = {}
        # pinned host buffers that the chosen tokens are copied into, used in turn (a launch's
        # tokens are read before the launch after the next one reuses its buffer)
        self._token_buffers: list[torch.Tensor | None] = [None] * 4
        self._token_turn = 0

    def _token_buffer(self, rows: int) -> torch.Tensor:
        index = self._token_turn = (self._token_turn + 1) % len(self._token_buffers)
        buffer = self._token_buffers[index]
        if buffer is None or buffer.numel() < rows:
            buffer = self._token_buffers[index] = torch.empty(max(rows, 64), dtype=torch.int32, pin_memory=True)
        return buffer[:rows]

    # ---- random streams ---------------------------------------------------------------
    @staticmethod
    def _new_generator(params: SamplingParams) -> torch.Generator:
        generator = torch.Generator(device="cpu")
        seed = params.seed if params.seed is not None else int.from_bytes(os.urandom(8), "little") & (2**63 - 1)
        generator.manual_seed(seed)
        return generator

    @staticmethod
    def draw_uniform(generator: torch.Generator) -> float:
        """One number in [0, 1) that float32 represents below 1."""

        value = float(torch.rand((), generator=generator, dtype=torch.float64))
        return min(value, _BELOW_ONE)

    # ---- sampling ---------------------------------------------------------------------
    def stage(
        self, logits: torch.Tensor, requests: Sequence[tuple[str, SamplingParams]]
    ) -> tuple[StagedSample, ...]:
        """One token per row of float32 ``logits [R, V]`` (on the GPU) for the R
        requests, without advancing any generator."""

        return self.finish(self.launch(logits, requests))

    def launch(self, logits: torch.Tensor, requests: Sequence[tuple[str, SamplingParams]]):
        """The first half of :meth:`stage`: the draws are made and the choice is launched
        on the device; nothing waits for it.  The caller may do host work before
        :meth:`finish` fetches the tokens."""

        from .. import ops

        if logits.ndim != 2 or logits.shape[0] != len(requests) or logits.shape[1] == 0:
            raise ValueError(f"{len(requests)} requests need logits [{len(requests)}, vocab], not {tuple(logits.shape)}.")
        if not logits.is_floating_point():
            raise TypeError(f"logits are floating-point numbers, not {logits.dtype}.")
        vocab = logits.shape[1]
        states: list[torch.Tensor | None] = []
        uniforms: list[float] = []
        for request_id, params in requests:
            if params.top_k > vocab:
                raise ValueError(f"request {request_id!r}: top_k {params.top_k} is more than the {vocab} tokens of the vocabulary.")
            if params.temperature == 0:
                states.append(None)
                uniforms.append(0.0)
                continue
            known = self._generators.get(request_id)
            scratch = torch.Generator(device="cpu")
            scratch.set_state((known or self._new_generator(params)).get_state())
            uniforms.append(self.draw_uniform(scratch))
            states.append(scratch.get_state())
        logits = logits.float().contiguous()
        if all(state is None for state in states):
            tokens = ops.sample_rows(logits)
        else:
            # the four numbers of every row in one pinned buffer and one copy that nothing waits for
            # (a copy from pageable memory would wait for the step that is still running)
            host = torch.empty((4, len(requests)), dtype=torch.float32, pin_memory=logits.is_cuda)
            numbers = host.numpy()
            numbers[0] = [p.temperature for _, p in requests]
            numbers[1] = [p.top_p for _, p in requests]
            numbers[2] = uniforms
            numbers[3].view(np.int32)[:] = [p.top_k for _, p in requests]
            sent = host.to(logits.device, non_blocking=True)
            # (a top-k of the whole vocabulary cuts nothing: the kernel treats it as off)
            alone = any(p.temperature > 0 and p.top_p < 1 and (p.top_k == 0 or p.top_k >= vocab) for _, p in requests)
            tokens = ops.sample_rows(
                logits, temperature=sent[0], top_p=sent[1], uniform=sent[2], top_k=sent[3].view(torch.int32),
                top_p_alone=alone,
            )
        # The copy to the host is asked for now, and an event marks its end: what the caller
        # launches between here and finish() (the next step, fed from `tokens` on the device)
        # lies behind the copy in the stream, and finish() does not wait for it.
        arrived = None
        if tokens.is_cuda:
            on_host = self._token_buffer(tokens.numel())
            on_host.copy_(tokens, non_blocking=True)
            arrived = torch.cuda.Event()
            arrived.record()
        else:
            on_host = tokens
        return tokens, tuple(requests), states, on_host, arrived

    def finish(self, launched) -> tuple[StagedSample, ...]:
        """The second half of :meth:`stage`: waits for the tokens of :meth:`launch`."""

        _, requests, states, on_host, arrived = launched
        if arrived is not None:
            arrived.synchronize()
        token_ids = on_host.tolist()
        if any(token < 0 for token in token_ids):
            raise NonFiniteLogitsError("a row of logits holds a value that is not finite; no token can be chosen from it.")
        return tuple(
            StagedSample(request_id, int(token), state)
            for (request_id, _), token, state in zip(requests, token_ids, states)
        )

    def commit(self, samples: Sequence[StagedSample]) -> None:
        for sample in samples:
            if sample.generator_state is None:
                continue
            generator = self._generators.get(sample.request_id)
            if generator is None:
                generator = torch.Generator(device="cpu")
                self._generators[sample.request_id] = generator
            generator.set_state(sample.generator_state)

    def sample(self, logits: torch.Tensor, requests: Sequence[tuple[str, SamplingParams]]) -> list[int]:
        staged = self.stage(logits, requests)
        self.commit(staged)
        return [sample.token_id for sample in staged]

    def release(self, request_id: str) -> None:
        self._generators.pop(request_id, None)

    @property
    def active_request_ids(self) -> tuple[str, ...]:
        return tuple(sorted(self._generators))
