"""One request's pages in one cache group, in the order of its tokens.

Entry ``i`` names the page that holds positions ``i * block_size`` to
``(i + 1) * block_size - 1``.  The pages need not be neighbours in the pool.  In a
group with a window the oldest entries are given back while the request lives;
they keep their place in the list as ``RETURNED`` so that positions still index it.
(The reference's table maps positions the same way, without giving back:
miniserve/kv/block_table.py:9-53.)
"""

from __future__ import annotations

RETURNED = -1


def _whole(value: object) -> bool:
    return type(value) is int and value >= 0


class BlockTable:
    def __init__(self, block_size: int, pages: list[int] | None = None) -> None:
        if not _whole(block_size) or block_size == 0:
            raise ValueError(f"a page holds a positive whole number of tokens, not {block_size!r}.")
        self.block_size = block_size
        self.pages: list[int] = []
        self.first_live = 0                        # entries below it are RETURNED
        self._tuple: tuple[int, ...] | None = None   # the table as a tuple, made when asked for, dropped on change
        self.extend(list(pages or []))

    def pages_for(self, token_count: int) -> int:
        """Pages that ``token_count`` tokens take."""

        if not _whole(token_count):
            raise ValueError(f"a number of tokens is a whole number, not {token_count!r}.")
        return -(-token_count // self.block_size)

    def extend(self, new_pages: list[int]) -> None:
        """Pages for the positions behind the last one the table covers."""

        if not new_pages:
            return                                  # most steps of a decoding request bring no page
        if not isinstance(new_pages, list) or not all(_whole(page) for page in new_pages):
            raise ValueError(f"pages are named by whole numbers, in a list; got {new_pages!r}.")
        if len(set(new_pages)) != len(new_pages) or not set(new_pages).isdisjoint(self.live_pages()):
            raise ValueError(f"a table names a page once; {new_pages} repeats one.")
        self.pages.extend(new_pages)
        self._tuple = None

    def locate(self, position: int) -> tuple[int, int, int]:
        """``(entry, page, offset inside the page)`` of a token position."""

        if not _whole(position):
            raise ValueError(f"a position is a whole number, not {position!r}.")
        entry, offset = divmod(position, self.block_size)
        if entry >= len(self.pages):
            raise IndexError(f"position {position} lies behind the {len(self.pages)} pages of the table.")
        if self.pages[entry] == RETURNED:
            raise IndexError(f"position {position} lies in a page that was given back.")
        return entry, self.pages[entry], offset

    def slot(self, position: int) -> int:
        """Where a position's key and value lie in the pool: ``page * block_size + offset``."""

        _, page, offset = self.locate(position)
        return page * self.block_size + offset

    def live_pages(self) -> list[int]:
        return self.pages[self.first_live :]

    def live_count(self) -> int:
        return len(self.pages) - self.first_live

    def give_back_before(self, position: int) -> list[int]:
        """The pages that lie wholly below ``position`` leave the table and are returned."""

        end = min(max(position, 0) // self.block_size, len(self.pages))
        gone = self.pages[self.first_live : end]
        if gone:
            self.pages[self.first_live : end] = [RETURNED] * len(gone)
            self.first_live = end
            self._tuple = None
        return gone

    def snapshot(self) -> tuple[int, ...]:
        """The table as a tuple; the same object until the table changes, so a reader
        can tell by identity whether it has seen this table."""

        if self._tuple is None:
            self._tuple = tuple(self.pages)
        return self._tuple
