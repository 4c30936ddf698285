"""Which of the two bfloat16 matrix products serves a shape: a fixed rule, no GPU needed."""

from __future__ import annotations

import pytest


def test_the_rule_for_the_two_products():
    """The rule is a function of the shape alone: the shapes of the three model sizes
    fall where the timings on MI355X put them."""

    from miniserve_amd import ops

    small = {"qkv": (4096, 1024), "o": (1024, 2048), "gate_up": (6144, 1024), "down": (1024, 3072)}
    for n, k in small.values():
        assert ops.prefers_skinny(1, n, k) and ops.prefers_skinny(16, n, k) and ops.prefers_skinny(32, n, k)
        assert not ops.prefers_skinny(65, n, k)
    assert ops.prefers_skinny(64, *small["qkv"]) and ops.prefers_skinny(64, *small["down"])
    assert ops.prefers_skinny(8, 151936, 1024) and not ops.prefers_skinny(16, 151936, 1024)      # the head
    assert ops.prefers_skinny(16, 4096, 4096) and not ops.prefers_skinny(17, 4096, 4096)         # 32 MiB
    assert not ops.prefers_skinny(8, 24576, 4096) and ops.prefers_skinny(8, 24576, 4096, fused=True)
    assert not ops.prefers_skinny(8, 51200, 5120, fused=True)                                    # 500 MiB
    assert not ops.prefers_skinny(8, 5120, 25600)            # 250 MiB of very long rows: the library's timed choice splits them


def test_the_norm_is_a_prologue_only_of_small_and_middle_matrices(monkeypatch):
    """The norm as the product's prologue pays up to 64 MiB (48 MiB with the gated
    activation); larger matrices get a norm kernel of their own."""

    import torch

    from miniserve_amd import ops

    class Library:
        @staticmethod
        def ms_gemm_skinny_supported(m, n, k, epilogue):
            return 1

    monkeypatch.setattr(ops, "load", lambda: Library)

    def weight(n, k):
        return torch.empty((n, k), dtype=torch.bfloat16, device="meta")

    assert ops.can_fuse_norm(8, weight(4096, 1024)) and ops.can_fuse_norm(8, weight(6144, 1024), gated=True)   # 0.6B
    assert ops.can_fuse_norm(16, weight(4096, 4096)) and not ops.can_fuse_norm(17, weight(4096, 4096))
    assert ops.can_fuse_norm(8, weight(6144, 4096))                     # 48 MiB: the q/k/v matrix of the 8B sizes
    assert not ops.can_fuse_norm(8, weight(10240, 5120))                # 100 MiB: that of the 32B sizes
    assert not ops.can_fuse_norm(8, weight(24576, 4096), gated=True)    # 192 MiB: its gate and up matrix
    assert ops.can_fuse_norm(8, weight(12288, 2048), gated=True)        # 48 MiB, gated
    assert ops.prefers_skinny(8, 24576, 4096, fused=True)               # the activation stays that product's epilogue
    with ops.forced_product("skinny"):
        assert ops.can_fuse_norm(8, weight(10240, 5120))                # tests may still ask for the fused kernel


def test_where_a_product_takes_a_norm_that_the_product_before_prepared(monkeypatch):
    """A norm prepared by the product before it is taken where the norm would otherwise
    be a kernel of its own and this library's product serves both: never where the
    prologue form runs (few rows, small matrix), up to 8 rows against a large matrix, up
    to 64 rows against a small one."""

    import torch

    from miniserve_amd import ops

    class Library:
        @staticmethod
        def ms_gemm_skinny_supported(m, n, k, epilogue):
            return 1

    monkeypatch.setattr(ops, "load", lambda: Library)

    def weight(n, k, dtype=torch.bfloat16):
        return torch.empty((n, k), dtype=dtype, device="meta")

    qkv, gate_up = weight(4096, 1024), weight(6144, 1024)               # 0.6B
    for rows in (1, 8, 16):
        assert not ops.can_use_prepared_norm(rows, qkv) and not ops.can_use_prepared_norm(rows, gate_up, gated=True)
    for rows in (17, 40, 64):
        assert ops.can_use_prepared_norm(rows, qkv) and ops.can_use_prepared_norm(rows, gate_up, gated=True)
        assert ops.can_prepare_norm(rows, weight(1024, 2048)) and ops.can_prepare_norm(rows, weight(1024, 3072))
    assert not ops.can_use_prepared_norm(65, qkv) and not ops.can_prepare_norm(65, weight(1024, 2048))
    big = weight(24576, 4096)                                           # 8B, gate and up: 192 MiB
    assert ops.can_use_prepared_norm(1, big, gated=True) and ops.can_use_prepared_norm(8, big, gated=True)
    assert not ops.can_use_prepared_norm(9, big, gated=True) and not ops.can_use_prepared_norm(16, big, gated=True)
    assert ops.can_use_prepared_norm(8, big)                             # the saved norm kernel pays for this library's product
    assert ops.can_prepare_norm(8, weight(4096, 4096))                   # 8B, o: 32 MiB, this library's product
    assert not ops.can_prepare_norm(8, weight(4096, 12288))              # 8B, down: the library's
    assert not ops.can_use_prepared_norm(8, weight(51200, 5120), gated=True)    # 32B: the library's
    assert not ops.can_use_prepared_norm(40, qkv.to(torch.float32)) and not ops.can_prepare_norm(40, weight(1024, 2048, torch.float32))
    with ops.forced_product("skinny"):
        assert ops.can_use_prepared_norm(8, qkv) and ops.can_use_prepared_norm(16, big)      # tests may ask for the kernel itself
    with ops.forced_product("library"):
        assert not ops.can_use_prepared_norm(40, qkv) and not ops.can_prepare_norm(40, weight(1024, 2048))


def test_a_forced_product_overrides_the_rule_and_is_undone():
    from miniserve_amd import ops

    assert not ops.prefers_skinny(64, 4096, 4096)
    with ops.forced_product("skinny"):
        assert ops.prefers_skinny(64, 4096, 4096) and not ops.prefers_skinny(65, 4096, 4096)
        with ops.forced_product("library"):
            assert not ops.prefers_skinny(1, 4096, 1024)
        assert ops.prefers_skinny(64, 4096, 4096)
    assert not ops.prefers_skinny(64, 4096, 4096) and ops.prefers_skinny(1, 4096, 1024)
    with pytest.raises(ValueError):
        with ops.forced_product("fastest"):
            pass


def test_the_table_of_pinned_library_solutions_is_well_formed():
    """``ops/library_products.json``: the library's build it was measured under and one pin
    for a (matrix, output type, bucket of row counts), each once, all whole numbers; the
    matrices of the three presets are there."""

    import json

    from miniserve_amd import ops

    table = json.loads(ops.LIBRARY_PRODUCTS_TABLE.read_text())
    assert isinstance(table["library"], str) and ":" in table["library"]
    pins = table["pins"]
    assert all(len(pin) == 5 and all(type(v) is int for v in pin) for pin in pins)
    keys = [tuple(pin[:4]) for pin in pins]
    assert len(keys) == len(set(keys)) and all(pin[2] in (0, 1) and pin[3] >= 0 and pin[4] > 0 for pin in pins)
    matrices = {(n, k) for n, k, _, _, _ in pins}
    # q/k/v, o, gate and up, down of the 0.6B, 8B and 32B sizes (o and down add into the 32-bit stream)
    for shape in [(4096, 1024), (1024, 2048), (6144, 1024), (1024, 3072), (6144, 4096), (4096, 4096), (24576, 4096),
                  (4096, 12288), (10240, 5120), (5120, 8192), (51200, 5120), (5120, 25600)]:
        assert shape in matrices, shape
