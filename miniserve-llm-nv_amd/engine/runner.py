"""The step function: a batch of (request, its next tokens) in, logits at the
wanted places out.  It runs only the tokens it is given, as one batch, from the
cache that earlier steps left, inside a cache transaction
(reference for the transaction: miniserve/engine/core.py:317-434; for executing a
plan: miniserve/engine/executor.py:239-255, which runs one forward per request
where this runs one for all).
"""

from __future__ import annotations

from pathlib import Path
from typing import Sequence

import torch

from ..cache import CacheLayout, CacheManager, StepItem
from ..config import EngineConfig, load_config
from ..parts.model import TORCH_DTYPES, DecoderModel
from ..weights import WeightLoadReport, load_weights, random_device_tensors
from .batch import StepEntry, build_step_context


def _require_gpu(device: torch.device) -> None:
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("the engine runs on the GPU only (HIP kernels); no CPU path exists.")


class ModelRunner:
    """Owns the model, its weights and the cache; offers ``step``."""

    def __init__(
        self,
        model: DecoderModel,
        tensors: dict[str, torch.Tensor],
        engine_config: EngineConfig,
        *,
        device: torch.device | str = "cuda:0",
    ) -> None:
        self.device = torch.device(device)
        _require_gpu(self.device)
        from .. import ops

        ops.load()
        self.model = model
        self.spec = model.spec
        self.engine_config = engine_config.validate(max_positions=self.spec.max_positions)
        self.dtype = model.dtype
        if TORCH_DTYPES[self.engine_config.dtype] != self.dtype:
            raise ValueError("the model and the engine configuration disagree on the dtype.")
        model.load_weights(tensors)
        self.max_model_len = self.engine_config.resolved_max_model_len(self.spec.max_positions)
        self.block_size = self.engine_config.kv_block_size
        layout = CacheLayout.from_needs(model.cache_needs())
        num_blocks = self.engine_config.num_kv_blocks
        if num_blocks is None:
            num_blocks = self._blocks_from_free_memory(layout)
        if num_blocks * self.block_size >= 2**31:
            raise ValueError("the cache pool is too large for 32-bit slot numbers.")
        self.cache = CacheManager(
            layout,
            block_size=self.block_size,
            num_blocks=num_blocks,
            max_num_seqs=self.engine_config.max_num_seqs,
            max_model_len=self.max_model_len,
        )
        self.cache.allocate_storage(self.dtype, self.device)
        self._call_views = self.cache.call_views()
        self.steps_run = 0
        self.tokens_run = 0

    # ---- construction -----------------------------------------------------------------
    @classmethod
    def from_folder(
        cls, model_dir: str | Path, engine_config: EngineConfig, *, device: torch.device | str = "cuda:0"
    ) -> "ModelRunner":
        """A folder with ``config.json`` and safetensors; the model class is chosen
        by ``config.json: architectures``."""

        _require_gpu(torch.device(device))
        config = load_config(model_dir)
        model = DecoderModel(config.model_spec(), engine_config.dtype)
        tensors, report = load_weights(model_dir, model.weight_specs(), dtype=model.dtype, device=device)
        runner = cls(model, tensors, engine_config, device=device)
        runner.config = config
        runner.load_report = report
        return runner

    @classmethod
    def from_random(
        cls, config, engine_config: EngineConfig, *, seed: int = 0, device: torch.device | str = "cuda:0"
    ) -> "ModelRunner":
        """Random weights drawn on the device (for sizes that should not pass through a file)."""

        _require_gpu(torch.device(device))
        model = DecoderModel(config.model_spec(), engine_config.dtype)
        tensors = random_device_tensors(model.weight_specs(), seed=seed, dtype=model.dtype, device=device)
        runner = cls(model, tensors, engine_config, device=device)
        runner.config = config
        runner.load_report = WeightLoadReport(model_dir="<random>")
        return runner

    def _blocks_from_free_memory(self, layout: CacheLayout) -> int:
        """Pages that fit into 80% of the memory that is free after the weights,
        but no more than ``max_num_seqs`` full-length requests need."""

        free_bytes, _ = torch.cuda.mem_get_info(self.device)
        itemsize = torch.empty((), dtype=self.dtype).element_size()
        per_block = max(layout.bytes_per_token(itemsize) * self.block_size, 1)
        by_memory = int(free_bytes * 0.8) // per_block
        by_need = self.engine_config.max_num_seqs * -(-self.max_model_len // self.block_size)
        blocks = max(1, min(by_memory, by_need))
        return blocks

    # ---- requests -------------------------------------------------------------------
    def admit(self, request_id: str) -> int:
        return self.cache.admit(request_id)

    def release(self, request_id: str) -> None:
        self.cache.release(request_id)

    # ---- the step ---------------------------------------------------------------------
    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor | None:
        """Run one batch.  Every request of ``entries`` must be admitted; its tokens
        continue where its committed tokens end.  Returns float32 logits
        ``[wanted, vocab]`` in the order of the entries and of their ``want``, or
        None when nothing is wanted.  On an exception the step leaves no trace in
        the cache manager."""

        if not entries:
            raise ValueError("a step needs at least one entry.")
        items = []
        for entry in entries:
            start = self.cache.committed_tokens(entry.request_id)
            items.append(StepItem(entry.request_id, start, start + len(entry.token_ids)))
        reservation = self.cache.prepare_step(items)
        try:
            ctx, rows = build_step_context(
                entries,
                reservation,
                block_size=self.block_size,
                pool_pages=self.cache.num_blocks,
                vocab_size=self.spec.vocab_size,
                device=self.device,
            )
            logits = self.model.forward(ctx, self._call_views, rows)
        except BaseException:
            self.cache.abort_step(reservation)
            raise
        self.cache.commit_step(reservation)
        self.steps_run += 1
        self.tokens_run += ctx.num_tokens
        return logits
