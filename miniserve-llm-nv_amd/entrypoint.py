"""The Python entry point: a model folder to generated token ids.

Option names and meanings are those of the reference's launcher
(miniserve/api/server.py:350-397) where it has them: ``max_model_len``,
``num_kv_blocks``, ``max_num_seqs``, ``max_pending_requests``,
``max_num_batched_tokens``, ``kv_block_size``, ``enable_chunked_prefill``,
``prefill_chunk_size``.  Token ids in, token ids out; the tokenizer stays outside,
as it does in the reference (miniserve/api/adapter.py:73-80).
"""

from __future__ import annotations

import os
from typing import Sequence

from .config import EngineConfig
from .engine import Engine, ModelRunner, SamplingParams


class LLM:
    def __init__(
        self,
        model,
        *,
        dtype: str = "bfloat16",
        max_model_len: int | None = None,
        num_kv_blocks: int | None = None,
        max_num_seqs: int = 8,
        max_pending_requests: int = 64,
        max_num_batched_tokens: int | None = None,
        kv_block_size: int = 16,
        enable_chunked_prefill: bool = False,
        prefill_chunk_size: int | None = None,
        decode_graphs: bool = True,
        device: str = "cuda:0",
        seed: int = 0,
    ) -> None:
        self.engine_config = EngineConfig(
            dtype=dtype,
            max_model_len=max_model_len,
            max_num_seqs=max_num_seqs,
            max_num_batched_tokens=max_num_batched_tokens,
            kv_block_size=kv_block_size,
            num_kv_blocks=num_kv_blocks,
            enable_chunked_prefill=enable_chunked_prefill,
            prefill_chunk_size=prefill_chunk_size,
            max_pending_requests=max_pending_requests,
            decode_graphs=decode_graphs,
        )
        if isinstance(model, (str, os.PathLike)):
            self.runner = ModelRunner.from_folder(model, self.engine_config, device=device)
        else:
            # a configuration object: random weights from ``seed`` (the model that ``write_random_model``
            # writes for it, unless it is so large that it is drawn on the device)
            self.runner = ModelRunner.from_random(model, self.engine_config, seed=seed, device=device)
        self.engine = Engine(self.runner)

    @classmethod
    def from_random(cls, config, *, seed: int = 0, layers: int | None = None, **options) -> "LLM":
        """An engine over random weights without a file.  ``config`` is a configuration object of a
        registered architecture, the name of a preset (``"qwen3-0.6b"``) or the path
        of a ``config.json``; ``layers`` replaces the number of layers of a preset or
        file.  ``options`` as for the constructor."""

        if isinstance(config, (str, os.PathLike)):
            from .config import config_dict_from_preset_or_file, config_from_dict

            data = config_dict_from_preset_or_file(os.fspath(config))
            if layers is not None:
                data["num_hidden_layers"] = layers
            config = config_from_dict(data)
        elif layers is not None:
            raise ValueError("layers= goes with a preset's name or a config.json; a configuration object names its own.")
        return cls(config, seed=seed, **options)

    def generate(
        self,
        prompts: Sequence[Sequence[int]],
        sampling_params: SamplingParams | Sequence[SamplingParams] | None = None,
    ) -> list[list[int]]:
        """Generated token ids, one list per prompt of token ids."""

        return self.engine.generate(prompts, sampling_params)
