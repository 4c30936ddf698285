"""Engine options.  Names and meanings follow the reference's ``EngineConfig``
(reference: miniserve/config/engine_config.py:16-31); its backend switches are
dropped because this engine has one backend."""

from __future__ import annotations

from dataclasses import dataclass

from .fields import ConfigError

DTYPES = ("bfloat16", "float32")


def _is_int(value: object) -> bool:
    return isinstance(value, int) and not isinstance(value, bool)


@dataclass(frozen=True)
class EngineConfig:
    dtype: str = "bfloat16"
    max_model_len: int | None = None          # None: the model's max positions
    max_num_seqs: int = 8                     # live requests (state slots)
    max_num_batched_tokens: int | None = None # tokens of one step; None: min(4096, max_model_len)
    kv_block_size: int = 16                   # tokens of one page
    num_kv_blocks: int | None = None          # None: derived from free device memory
    enable_chunked_prefill: bool = False
    prefill_chunk_size: int | None = None
    max_pending_requests: int = 64
    decode_graphs: bool = True                # replay decode-only steps as HIP graphs (bfloat16)

    def validate(self, *, max_positions: int) -> "EngineConfig":
        """Cross-field rules of the reference (engine_config.py:253-359,
        runtime_config.py:78-86, model_config.py:204-205)."""

        if self.dtype not in DTYPES:
            raise ConfigError(f"dtype must be one of {DTYPES}.")
        for name in ("max_num_seqs", "kv_block_size", "max_pending_requests"):
            value = getattr(self, name)
            if not _is_int(value) or value <= 0:
                raise ConfigError(f"{name} must be a positive integer.")
        for name in ("max_model_len", "max_num_batched_tokens", "num_kv_blocks", "prefill_chunk_size"):
            value = getattr(self, name)
            if value is not None and (not _is_int(value) or value <= 0):
                raise ConfigError(f"{name} must be a positive integer or None.")
        for name in ("enable_chunked_prefill", "decode_graphs"):
            if not isinstance(getattr(self, name), bool):
                raise ConfigError(f"{name} must be a bool.")
        max_model_len = self.resolved_max_model_len(max_positions)
        if not 0 < max_model_len <= max_positions:
            raise ConfigError("max_model_len exceeds the model position limit.")
        batched = self.resolved_max_num_batched_tokens(max_positions)
        if batched > max_model_len:
            raise ConfigError("max_num_batched_tokens cannot exceed max_model_len.")
        if self.prefill_chunk_size is not None:
            if not self.enable_chunked_prefill:
                raise ConfigError("prefill_chunk_size requires enable_chunked_prefill=True.")
            if self.prefill_chunk_size > batched:
                raise ConfigError("prefill_chunk_size cannot exceed max_num_batched_tokens.")
        return self

    def resolved_max_num_batched_tokens(self, max_positions: int) -> int:
        if self.max_num_batched_tokens is not None:
            return self.max_num_batched_tokens
        return min(4096, self.resolved_max_model_len(max_positions))

    def resolved_max_model_len(self, max_positions: int) -> int:
        return max_positions if self.max_model_len is None else self.max_model_len
