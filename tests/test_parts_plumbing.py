"""How a block and the model hand norms to the parts around them: pending, prepared by
the part before, or taken from the residual stream.  Stub parts and no kernels: the
decisions alone, on the CPU."""

from __future__ import annotations

import torch

from miniserve_amd.parts import PendingNorm, PreparedNorm
from miniserve_amd.parts.block import PreNormBlock


class StubNorm:
    """Counts the times it is taken from the residual stream."""

    def __init__(self, name: str) -> None:
        self.name, self.eps, self.weight, self.taken = name, 1e-6, torch.ones(4), 0

    def add_forward(self, residual, delta, *, rows=None, write_back=True):
        self.taken += 1
        if delta is not None:
            residual += delta
        return residual.clone()


class StubPart:
    """A mixer or feed-forward that records what it was given.  ``pending``: it accepts a
    pending norm; ``takes``: it has a use for a prepared one beyond 16 rows; ``adds``: it
    adds its output into the residual stream itself; ``prepares``: and prepares the norm
    it is told of."""

    def __init__(self, *, pending=False, takes=False, adds=False, prepares=False) -> None:
        if pending:
            self.accepts_pending_norm = True
        if takes:
            self.takes_prepared_norm = lambda rows: rows > 16
        if adds:
            self.accumulates_residual = True
        if prepares:
            self.prepares_norm = True
        self.seen: list = []
        self.norm_after_seen: list = []

    def forward(self, x, *extra, residual=None, norm_after=None):
        self.seen.append(x)
        self.norm_after_seen.append(norm_after)
        if isinstance(x, PendingNorm) and x.prepared is None:
            x.materialize()                  # nothing prepared: the norm is taken from the residual stream
        if residual is None:
            return torch.ones(tuple(x.shape))
        residual += 1
        if norm_after is not None:
            return PreparedNorm(norm_after, torch.zeros(1), torch.zeros(1))
        return None


def block_of(mixer, feed_forward):
    block = PreNormBlock.__new__(PreNormBlock)
    block.pre_mixer, block.pre_feed_forward = StubNorm("pre_mixer"), StubNorm("pre_feed_forward")
    block.mixer, block.feed_forward = mixer, feed_forward
    return block


def test_a_pending_norm_keeps_only_what_was_prepared_for_it():
    norm, other = StubNorm("a"), StubNorm("b")
    residual = torch.zeros(3, 4)
    mine = PendingNorm(norm, residual, PreparedNorm(norm, torch.zeros(1), torch.zeros(1)))
    assert mine.prepared is not None and mine.delta is None and mine.fusable
    foreign = PendingNorm(norm, residual, PreparedNorm(other, torch.zeros(1), torch.zeros(1)))
    assert foreign.prepared is None and foreign.delta is None
    assert torch.equal(foreign.materialize(), residual) and norm.taken == 1 and other.taken == 0
    with_delta = PendingNorm(norm, residual.clone(), torch.ones(3, 4))
    assert not with_delta.fusable and with_delta.prepared is None
    assert torch.equal(with_delta.materialize(), torch.ones(3, 4)) and with_delta.delta is None


def test_plain_parts_get_tensors_and_no_word_of_the_norms():
    mixer, feed_forward = StubPart(), StubPart()
    block = block_of(mixer, feed_forward)
    residual, delta = block.forward(torch.zeros(20, 4), None, None, None, norm_after=StubNorm("next"))
    assert isinstance(mixer.seen[0], torch.Tensor) and isinstance(feed_forward.seen[0], torch.Tensor)
    assert mixer.norm_after_seen == [None] and feed_forward.norm_after_seen == [None]
    assert isinstance(delta, torch.Tensor) and block.pre_mixer.taken == 1 and block.pre_feed_forward.taken == 1
    assert not block.takes_prepared_norm(20)


def test_a_norm_is_prepared_only_for_a_part_that_takes_it():
    rows = 20
    # the feed-forward takes prepared norms, the mixer can prepare them: the norm between them is named
    mixer = StubPart(pending=True, takes=True, adds=True, prepares=True)
    feed_forward = StubPart(pending=True, takes=True, adds=True, prepares=True)
    block = block_of(mixer, feed_forward)
    following = StubNorm("next")
    residual, delta = block.forward(torch.zeros(rows, 4), None, None, None, norm_after=following)
    assert mixer.norm_after_seen == [block.pre_feed_forward] and feed_forward.norm_after_seen == [following]
    assert isinstance(feed_forward.seen[0], PendingNorm) and feed_forward.seen[0].prepared is not None
    assert feed_forward.seen[0].prepared.norm is block.pre_feed_forward
    assert isinstance(delta, PreparedNorm) and delta.norm is following
    assert block.pre_feed_forward.taken == 0            # never taken from the residual stream
    assert block.takes_prepared_norm(rows) and not block.takes_prepared_norm(8)
    # few rows: the part behind the norm has no use for it, so none is asked for
    mixer.norm_after_seen.clear()
    block.forward(torch.zeros(8, 4), None, None, None)
    assert mixer.norm_after_seen == [None]
    # a mixer that adds into the residual stream but does not prepare norms is not told of them
    plain_adder = StubPart(pending=True, adds=True)
    block = block_of(plain_adder, StubPart(pending=True, takes=True, adds=True, prepares=True))
    block.forward(torch.zeros(rows, 4), None, None, None)
    assert plain_adder.norm_after_seen == [None]
    assert block.feed_forward.seen[0].prepared is None and block.pre_feed_forward.taken == 1


def test_the_model_names_the_next_blocks_first_norm():
    """DecoderModel.forward passes ``norm_after`` to a block that accepts it when the block
    behind it offers ``first_norm`` and takes prepared norms for this many rows; the last
    block is told of none, and a block without the attributes is called as before."""

    from miniserve_amd.parts.model import DecoderModel

    calls = []

    class Block:
        accepts_norm_after = True

        def __init__(self, name, takes):
            self.name, self.first_norm, self._takes = name, StubNorm(name), takes

        def takes_prepared_norm(self, rows):
            return self._takes

        def forward(self, residual, delta, ctx, cache, *, norm_after=None):
            calls.append((self.name, None if norm_after is None else norm_after.name, type(delta).__name__))
            return residual, (PreparedNorm(norm_after, torch.zeros(1), torch.zeros(1)) if norm_after is not None else None)

    class OldBlock:
        def forward(self, residual, delta, ctx, cache):
            calls.append(("old", None, type(delta).__name__))
            return residual, None

    class Embedding:
        def forward(self, token_ids, ctx):
            return torch.zeros(20, 4)

    class Order:
        def __init__(self, layer):
            self.layer = layer

    class Context:
        token_ids = None

    final = StubNorm("final")
    model = DecoderModel.__new__(DecoderModel)
    model.embedding, model.final_norm = Embedding(), final
    model.layers = [Block("a", True), Block("b", True), OldBlock(), Block("c", False), Block("d", True)]
    model.order = [Order(0), Order(1), Order(2), Order(3), Order(4), Order(0)]
    model.head = type("Head", (), {"forward": staticmethod(lambda x: x)})()
    out = model.forward(Context(), [None] * 6, torch.tensor([0], dtype=torch.int32))
    assert calls == [
        ("a", "b", "NoneType"),             # b takes the norm that a prepares
        ("b", None, "PreparedNorm"),        # the block behind b knows nothing of prepared norms
        ("old", None, "NoneType"),
        ("c", "d", "NoneType"),             # c itself takes none, d behind it does
        ("d", "a", "PreparedNorm"),         # the order names layer 0 again
        ("a", None, "PreparedNorm"),        # the last call: the final norm is taken from the residual stream
    ]
    assert final.taken == 1 and out is not None
