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
    assert ops.prefers_skinny(16, 5120, 25600) and not ops.prefers_skinny(17, 5120, 25600)       # very long rows


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
