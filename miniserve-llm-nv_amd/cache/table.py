"""A request's map from logical page index to physical page id, for one group
(reference: miniserve/kv/block_table.py:9-53).  Pages that a window has passed
are given back and their entries become ``RETURNED``."""

from __future__ import annotations

from dataclasses import dataclass, field

RETURNED = -1


def _is_int(value: object) -> bool:
    return isinstance(value, int) and not isinstance(value, bool)


@dataclass
class BlockTable:
    block_size: int
    physical_block_ids: list[int] = field(default_factory=list)
    first_live: int = 0          # logical index of the first page still held
    _snapshot: tuple[int, ...] | None = field(default=None, repr=False, compare=False)   # kept until the table changes

    def __post_init__(self) -> None:
        if not _is_int(self.block_size) or self.block_size <= 0:
            raise ValueError("block_size must be a positive integer.")
        if any(not _is_int(page) or page < 0 for page in self.physical_block_ids):
            raise ValueError("Physical block IDs must be non-negative integers.")
        if len(self.physical_block_ids) != len(set(self.physical_block_ids)):
            raise ValueError("One sequence block table cannot duplicate a physical ID.")

    def required_blocks(self, token_count: int) -> int:
        if not _is_int(token_count) or token_count < 0:
            raise ValueError("token_count must be a non-negative integer.")
        return (token_count + self.block_size - 1) // self.block_size

    def append_blocks(self, block_ids: list[int]) -> None:
        if isinstance(block_ids, list) and not block_ids:
            return               # most steps of a decoding request bring no new page
        if not isinstance(block_ids, list) or any(not _is_int(page) or page < 0 for page in block_ids):
            raise ValueError("Appended physical block IDs must be a list of non-negative integers.")
        if len(block_ids) != len(set(block_ids)) or set(block_ids) & set(self.live_pages()):
            raise ValueError("Appended physical block IDs must be unique.")
        self.physical_block_ids.extend(block_ids)
        self._snapshot = None

    def resolve(self, token_position: int) -> tuple[int, int, int]:
        """``(logical page, physical page, offset)`` of a position."""

        if not _is_int(token_position) or token_position < 0:
            raise ValueError("token_position must be a non-negative integer.")
        logical, offset = divmod(token_position, self.block_size)
        if logical >= len(self.physical_block_ids):
            raise IndexError("Token position has no reserved physical block.")
        physical = self.physical_block_ids[logical]
        if physical == RETURNED:
            raise IndexError("Token position lies in a page that was given back.")
        return logical, physical, offset

    def slot(self, token_position: int) -> int:
        _, physical, offset = self.resolve(token_position)
        return physical * self.block_size + offset

    def live_pages(self) -> list[int]:
        return self.physical_block_ids[self.first_live :]

    def live_count(self) -> int:
        return len(self.physical_block_ids) - self.first_live

    def give_back_before(self, token_position: int) -> list[int]:
        """Pages whose every position is below ``token_position`` leave the table."""

        limit = min(max(token_position, 0) // self.block_size, len(self.physical_block_ids))
        returned = []
        for logical in range(self.first_live, limit):
            returned.append(self.physical_block_ids[logical])
            self.physical_block_ids[logical] = RETURNED
        self.first_live = max(self.first_live, limit)
        if returned:
            self._snapshot = None
        return returned

    def snapshot(self) -> tuple[int, ...]:
        """The table as a tuple; the same object until the table changes."""

        if self._snapshot is None:
            self._snapshot = tuple(self.physical_block_ids)
        return self._snapshot
