"""A stand-in for the model runner, for testing the engine loop on the CPU: a real
cache manager (without storage) and "logits" that depend only on a request's
token prefix, so what a request generates cannot depend on scheduling."""

from __future__ import annotations

import hashlib
from types import SimpleNamespace

import torch

from miniserve_amd.cache import CacheLayout, CacheManager, StepItem
from miniserve_amd.config import EngineConfig
from miniserve_amd.parts import KVCacheNeed


def next_token(prefix: tuple[int, ...], vocab: int) -> int:
    digest = hashlib.sha256(repr(prefix).encode()).digest()
    return int.from_bytes(digest[:4], "little") % vocab


class FakeRunner:
    def __init__(self, engine_config: EngineConfig, *, vocab_size=97, max_positions=256, fail_on_step=None):
        self.spec = SimpleNamespace(vocab_size=vocab_size, max_positions=max_positions)
        self.engine_config = engine_config.validate(max_positions=max_positions)
        self.max_model_len = engine_config.resolved_max_model_len(max_positions)
        self.block_size = engine_config.kv_block_size
        need = SimpleNamespace(call=0, need=KVCacheNeed(1, 8), cache_from=None)
        self.cache = CacheManager(
            CacheLayout.from_needs([need]), block_size=self.block_size, num_blocks=engine_config.num_kv_blocks,
            max_num_seqs=engine_config.max_num_seqs, max_model_len=self.max_model_len,
        )
        self.tokens: dict[str, list[int]] = {}
        self.steps: list[list[tuple[str, int, int]]] = []     # per step: (request, start, end)
        self.fail_on_step = fail_on_step
        self.prepare_ahead = False          # tests switch it on
        self.chain = False                  # tests switch it on: steps of single tokens are launched ahead
        self.prepared_ahead = self.used_ahead = self.discarded_ahead = self.prepared_mixed = 0
        self.chained = self.voided_chained = self.mapped = 0

    def admit(self, request_id):
        self.tokens[request_id] = []
        return self.cache.admit(request_id)

    def release(self, request_id):
        self.tokens.pop(request_id, None)
        self.cache.release(request_id)

    def prepare_decode(self, request_ids):
        """As the real runner's: the next step's cache transaction, opened ahead."""

        if not self.prepare_ahead:
            return None
        items = []
        for request_id in request_ids:
            start = self.cache.committed_tokens(request_id)
            items.append(StepItem(request_id, start, start + 1))
        self.prepared_ahead += 1
        prepared = SimpleNamespace(request_ids=tuple(request_ids), reservation=self.cache.prepare_step(items))
        if self.chain:
            prepared.launched = False
        return prepared

    def launch_chained(self, prepared, tokens, source_rows=None):
        """As the real runner's: the prepared step of single tokens runs now, on the tokens
        that the "device" holds (``tokens.values``, which the host has not read yet), row
        by row or through the map of rows."""

        assert not prepared.launched and tokens.is_cuda
        rows = len(prepared.request_ids)
        if source_rows is None:
            assert len(tokens.values) >= rows
            source_rows = range(rows)
        else:
            assert len(source_rows) == rows and all(0 <= row < len(tokens.values) for row in source_rows)
            # (a map comes only when it is needed: the rows are not the first of the sampled ones in their order)
            assert list(source_rows) != list(range(rows))
            self.mapped += 1
        prepared.launched = True
        prepared.ran = tuple(int(tokens.values[row]) for row in source_rows)
        self.chained += 1

    def prepare_step(self, entries, admit=()):
        """As the real runner's: any other step's cache transaction, opened ahead; the
        single tokens it is given are placeholders."""

        if not self.prepare_ahead:
            return None
        admitted = []
        try:
            for request_id in admit:
                self.admit(request_id)
                admitted.append(request_id)
            items = []
            for entry in entries:
                start = self.cache.committed_tokens(entry.request_id)
                items.append(StepItem(entry.request_id, start, start + len(entry.token_ids)))
            reservation = self.cache.prepare_step(items)
        except BaseException:
            for request_id in admitted:
                self.release(request_id)
            raise
        self.prepared_ahead += 1
        self.prepared_mixed += 1
        return SimpleNamespace(
            request_ids=tuple(entry.request_id for entry in entries), reservation=reservation, admitted=tuple(admitted),
            lengths=tuple(len(entry.token_ids) for entry in entries),
            known={e.request_id: e.token_ids for e in entries if len(e.token_ids) > 1},
        )

    def discard(self, prepared):
        self.discarded_ahead += 1
        self.voided_chained += bool(getattr(prepared, "launched", False))
        self.cache.abort_step(prepared.reservation)
        for request_id in getattr(prepared, "admitted", ()):
            self.release(request_id)

    def step(self, entries, prepared=None):
        items = []
        for entry in entries:
            start = self.cache.committed_tokens(entry.request_id)
            assert start == len(self.tokens[entry.request_id]), "the engine skipped or repeated tokens"
            items.append(StepItem(entry.request_id, start, start + len(entry.token_ids)))
        if prepared is not None:
            assert tuple(entry.request_id for entry in entries) == prepared.request_ids
            if hasattr(prepared, "lengths"):
                assert tuple(len(entry.token_ids) for entry in entries) == prepared.lengths
                assert all(entry.token_ids == prepared.known[entry.request_id] for entry in entries if len(entry.token_ids) > 1)
            else:
                assert all(len(entry.token_ids) == 1 for entry in entries)
            if getattr(prepared, "launched", False):
                # what ran is what the engine now says the step is
                assert tuple(entry.token_ids[0] for entry in entries) == prepared.ran
            reservation = prepared.reservation
            self.used_ahead += 1
        else:
            reservation = self.cache.prepare_step(items)
        if self.fail_on_step is not None and len(self.steps) == self.fail_on_step:
            self.fail_on_step = None
            self.cache.abort_step(reservation)
            raise RuntimeError("injected kernel failure")
        rows = []
        for entry in entries:
            base = self.tokens[entry.request_id]
            for place in entry.want:
                prefix = tuple(base) + tuple(entry.token_ids[: place + 1])
                row = torch.zeros(self.spec.vocab_size)
                row[next_token(prefix, self.spec.vocab_size)] = 1.0
                rows.append(row)
            base.extend(entry.token_ids)
        self.cache.commit_step(reservation)
        self.cache.assert_invariants()
        self.steps.append([(i.request_id, i.start, i.end) for i in items])
        return torch.stack(rows) if rows else None


class DeviceTokens:
    """Stands for the sampling kernel's output on the device: the engine may hand it to a
    chained launch but reads token values only from what ``finish`` returns."""

    is_cuda = True

    def __init__(self, values):
        self.values = values


class ArgmaxSampler:
    """Greedy on the host; the engine's sampler interface.  ``on_device``: ``launch`` returns
    its tokens as the real sampler does, as a tensor on the device, first."""

    def __init__(self, on_device: bool = False) -> None:
        self.on_device = on_device

    def stage(self, logits, requests):
        return self.finish(self.launch(logits, requests))

    def launch(self, logits, requests):
        if self.on_device:
            return DeviceTokens([int(torch.argmax(row)) for row in logits]), tuple(requests)
        return logits, tuple(requests)

    def finish(self, launched):
        from miniserve_amd.sampling import StagedSample

        first, requests = launched
        tokens = first.values if isinstance(first, DeviceTokens) else [int(torch.argmax(row)) for row in first]
        return tuple(StagedSample(rid, token, None) for (rid, _), token in zip(requests, tokens))

    def commit(self, samples):
        pass

    def release(self, request_id):
        pass


def expected_generation(prompt, max_new_tokens, vocab, stop=()):
    tokens = list(prompt)
    out = []
    for _ in range(max_new_tokens):
        token = next_token(tuple(tokens), vocab)
        out.append(token)
        tokens.append(token)
        if token in stop:
            break
    return out
