"""Pins of the plain implementation by what fixes it beside the reference's text:
vectors that the reference's own tests hold, special cases that reduce to a
library routine, and invariants - each chosen so that a plausible mistake (a wrong
sign or pairing, a norm in the wrong place, a wrong head mapping) fails it."""

from __future__ import annotations

import math

import plain_qwen3 as plain
import plain_sampling
import pytest
import torch
import torch.nn.functional as F
from helpers import make_model_folder, random_tokens, read_config, read_weights, tiny_a, tiny_b

F64 = torch.float64


# ---- RMSNorm ---------------------------------------------------------------------------

@pytest.mark.parametrize("shape", [(1, 8), (7, 16), (2, 3, 32)])
def test_rmsnorm_equals_the_direct_formula_bit_for_bit(shape):
    # reference: tests/correctness/test_rmsnorm_reference.py:13-20
    generator = torch.Generator().manual_seed(sum(shape) + 17)
    values = torch.randn(shape, generator=generator, dtype=torch.float32)
    weight = torch.linspace(0.5, 1.5, shape[-1], dtype=torch.float32)
    expected = values * torch.rsqrt(values.square().mean(dim=-1, keepdim=True) + 1e-6) * weight
    torch.testing.assert_close(plain.rms_norm(values, weight, 1e-6), expected, atol=0.0, rtol=0.0)


def test_rmsnorm_vector_library_routine_and_invariants():
    # the 8-value vector of the reference (test_rmsnorm_reference.py:23-32)
    values = torch.tensor([[0.0, 1.0, -1.0, 1e-4, -1e-4, 8.0, -8.0, 2.0]], dtype=F64)
    weight = torch.linspace(0.75, 1.25, 8, dtype=F64)
    out = plain.rms_norm(values, weight, 1e-6)
    torch.testing.assert_close(out, F.rms_norm(values, (8,), weight, 1e-6))
    # no mean subtraction (a LayerNorm would map a constant row to zero)
    constant = plain.rms_norm(torch.full((1, 8), 3.0, dtype=F64), torch.ones(8, dtype=F64), 1e-12)
    torch.testing.assert_close(constant, torch.ones(1, 8, dtype=F64))
    # plain w, not 1 + w
    assert torch.all(plain.rms_norm(values, torch.zeros(8, dtype=F64), 1e-6) == 0)
    # unit RMS and scale invariance
    x = torch.randn(5, 48, dtype=F64)
    y = plain.rms_norm(x, torch.ones(48, dtype=F64), 1e-12)
    torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(5, dtype=F64))
    torch.testing.assert_close(plain.rms_norm(7.0 * x, torch.ones(48, dtype=F64), 1e-12), y)
    # eps stands inside the root, added to the mean of squares
    tiny = torch.full((1, 4), 1e-3, dtype=F64)
    torch.testing.assert_close(
        plain.rms_norm(tiny, torch.ones(4, dtype=F64), 1e-5), tiny / math.sqrt(1e-6 + 1e-5)
    )


# ---- RoPE ------------------------------------------------------------------------------

def rope(x, positions, theta=10000.0):
    cos, sin = plain.rope_angles(torch.as_tensor(positions), x.shape[-1], theta)
    return plain.apply_rope(x, cos, sin)


def test_rope_hand_vector_is_half_split_not_interleaved():
    # D = 4, position 1: pairs (0, 2) and (1, 3); inv_freq = [1, theta^-1/2]
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0]]], dtype=F64)
    out = rope(x, [1], theta=100.0)[0, 0]
    a0, a1 = 1.0, 0.1
    expected = [
        1 * math.cos(a0) - 3 * math.sin(a0),
        2 * math.cos(a1) - 4 * math.sin(a1),
        3 * math.cos(a0) + 1 * math.sin(a0),
        4 * math.cos(a1) + 2 * math.sin(a1),
    ]
    torch.testing.assert_close(out, torch.tensor(expected, dtype=F64), atol=1e-6, rtol=0)


def test_rope_identity_norms_complex_form_and_relative_positions():
    generator = torch.Generator().manual_seed(3)
    x = torch.randn(2, 6, 16, generator=generator, dtype=F64)
    positions = torch.tensor([0, 1, 5, 17, 100, 1000])
    out = rope(x, positions)
    torch.testing.assert_close(out[:, 0], x[:, 0])                              # position 0 is the identity
    half = 8
    torch.testing.assert_close(                                                 # each pair keeps its length
        out[..., :half] ** 2 + out[..., half:] ** 2, x[..., :half] ** 2 + x[..., half:] ** 2
    )
    inv_freq = 1.0 / (10000.0 ** (torch.arange(0, 16, 2, dtype=torch.float32) / 16))
    angle = (positions.float()[:, None] * inv_freq).to(F64)
    rotated = torch.complex(x[..., :half], x[..., half:]) * torch.polar(torch.ones_like(angle), angle)
    torch.testing.assert_close(out, torch.cat([rotated.real, rotated.imag], dim=-1), atol=1e-6, rtol=0)
    # <rope(q, m), rope(k, n)> depends on m - n only
    q, k = torch.randn(1, 1, 16, dtype=F64), torch.randn(1, 1, 16, dtype=F64)
    dots = [float((rope(q, [m]) * rope(k, [n])).sum()) for m, n in ((9, 4), (25, 20), (105, 100))]
    assert max(dots) - min(dots) < 1e-4
    # theta matters
    assert not torch.allclose(rope(x, positions, 1e4), rope(x, positions, 1e6))


# ---- attention -------------------------------------------------------------------------

def test_attention_reduces_to_the_library_routine():
    generator = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(4, 9, 16, generator=generator, dtype=F64) for _ in range(3))
    expected = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]
    torch.testing.assert_close(plain.causal_attention(q, k, v, 16**-0.5), expected)
    # one token: the output is V itself
    torch.testing.assert_close(plain.causal_attention(q[:, :1], k[:, :1], v[:, :1], 0.25), v[:, :1])


def test_gqa_maps_consecutive_query_heads_to_one_kv_head():
    generator = torch.Generator().manual_seed(6)
    q = torch.randn(6, 7, 8, generator=generator, dtype=F64)
    k, v = (torch.randn(2, 7, 8, generator=generator, dtype=F64) for _ in range(2))
    out = plain.causal_attention(q, k, v, 8**-0.5)
    for head in range(6):
        single = plain.causal_attention(q[head : head + 1], k[head // 3 : head // 3 + 1], v[head // 3 : head // 3 + 1], 8**-0.5)
        torch.testing.assert_close(out[head : head + 1], single)
    expanded = plain.repeat_kv(k, 3)
    assert torch.equal(expanded[0], k[0]) and torch.equal(expanded[2], k[0]) and torch.equal(expanded[3], k[1])


def test_window_limits_the_keys():
    generator = torch.Generator().manual_seed(7)
    q, k, v = (torch.randn(1, 12, 8, generator=generator, dtype=F64) for _ in range(3))
    out = plain.causal_attention(q, k, v, 1.0, window=4)
    # query 9 sees keys 6..9 only
    torch.testing.assert_close(out[:, 9:10], plain.causal_attention(q[:, 9:10], k[:, 6:10], v[:, 6:10], 1.0)[:, -1:])
    torch.testing.assert_close(plain.causal_attention(q, k, v, 1.0, window=12), plain.causal_attention(q, k, v, 1.0))


# ---- feed-forward, embedding, head ------------------------------------------------------

def test_swiglu_library_routine_and_zero_gate():
    generator = torch.Generator().manual_seed(8)
    w = {
        "m.gate_proj.weight": torch.randn(10, 6, generator=generator, dtype=F64),
        "m.up_proj.weight": torch.randn(10, 6, generator=generator, dtype=F64),
        "m.down_proj.weight": torch.randn(6, 10, generator=generator, dtype=F64),
    }
    x = torch.randn(3, 6, generator=generator, dtype=F64)
    gate, up = x @ w["m.gate_proj.weight"].T, x @ w["m.up_proj.weight"].T
    expected = (gate * torch.sigmoid(gate) * up) @ w["m.down_proj.weight"].T
    torch.testing.assert_close(plain.swiglu(x, w, "m."), expected)
    w["m.gate_proj.weight"].zero_()
    assert torch.all(plain.swiglu(x, w, "m.") == 0)


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    base = tmp_path_factory.mktemp("plain")
    out = {}
    for name, make in (("a", tiny_a), ("b", tiny_b)):
        folder = make_model_folder(base / name, make(), seed=21)
        out[name] = (read_weights(folder), read_config(folder))
    return out


def test_whole_model_causality_and_head(models):
    for name, (weights, config) in models.items():
        tokens = random_tokens(20, config["vocab_size"], 4)
        logits = plain.forward_logits(weights, config, tokens)
        assert logits.shape == (20, config["vocab_size"])
        changed = list(tokens)
        changed[12] = (changed[12] + 1) % config["vocab_size"]
        other = plain.forward_logits(weights, config, changed)
        torch.testing.assert_close(other[:12], logits[:12], atol=0, rtol=0)       # the future does not leak back
        assert not torch.allclose(other[12:], logits[12:])
    weights, config = models["a"]                                                   # tied: the head is the embedding
    moved = dict(weights)
    moved["model.embed_tokens.weight"] = weights["model.embed_tokens.weight"] * 1.5
    assert not torch.allclose(plain.forward_logits(moved, config, [1, 2, 3]), plain.forward_logits(weights, config, [1, 2, 3]))
    weights, config = models["b"]                                                   # untied: the head alone moves the logits
    moved = dict(weights)
    moved["lm_head.weight"] = weights["lm_head.weight"] * 2.0
    torch.testing.assert_close(
        plain.forward_logits(moved, config, [1, 2, 3]), 2.0 * plain.forward_logits(weights, config, [1, 2, 3])
    )


def test_the_attention_block_takes_the_library_routines_own_scale(models):
    """The scale that ``attention_block`` itself chooses (no caller hands it in) is the
    default of the library's attention, 1/sqrt(head_dim): with the output projection
    set to the identity the block is the library routine over the normed, rotated
    heads.  A scale of 1/head_dim, or none, fails."""

    weights, config = models["a"]                     # 4 heads of 16 = the hidden size: the projection can be the identity
    heads, kv_heads, dim = config["num_attention_heads"], config["num_key_value_heads"], config["head_dim"]
    assert heads * dim == config["hidden_size"]
    w = {name: tensor.to(F64) for name, tensor in weights.items()}
    prefix = "model.layers.0.self_attn."
    w[prefix + "o_proj.weight"] = torch.eye(heads * dim, dtype=F64)
    generator = torch.Generator().manual_seed(12)
    x = torch.randn(11, config["hidden_size"], generator=generator, dtype=F64)
    positions = torch.arange(3, 14)
    got, _ = plain.attention_block(x, w, prefix, config, positions)
    cos, sin = plain.rope_angles(positions, dim, config["rope_theta"])
    q = plain.rms_norm((x @ w[prefix + "q_proj.weight"].T).view(11, heads, dim), w[prefix + "q_norm.weight"], config["rms_norm_eps"])
    k = plain.rms_norm((x @ w[prefix + "k_proj.weight"].T).view(11, kv_heads, dim), w[prefix + "k_norm.weight"], config["rms_norm_eps"])
    v = (x @ w[prefix + "v_proj.weight"].T).view(11, kv_heads, dim)
    q, k = plain.apply_rope(q.transpose(0, 1), cos, sin), plain.apply_rope(k.transpose(0, 1), cos, sin)
    k, v = plain.repeat_kv(k, heads // kv_heads), plain.repeat_kv(v.transpose(0, 1), heads // kv_heads)
    expected = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True)[0]     # the library's default scale
    torch.testing.assert_close(got, expected.transpose(0, 1).reshape(11, heads * dim))


def test_layers_that_add_nothing_leave_the_final_norm_and_the_head(models):
    """With every output projection zero each layer adds nothing to the residual
    stream, and the logits are the library's RMSNorm of the embeddings times the head:
    the final norm is there, once, with the model's eps and weight, before the head."""

    for name, (weights, config) in models.items():
        w = {key: (torch.zeros_like(tensor) if key.endswith(("o_proj.weight", "down_proj.weight")) else tensor).to(F64)
             for key, tensor in weights.items()}
        tokens = random_tokens(9, config["vocab_size"], 2)
        embedded = w["model.embed_tokens.weight"][torch.tensor(tokens)]
        normed = F.rms_norm(embedded, (config["hidden_size"],), w["model.norm.weight"], config["rms_norm_eps"])
        head = w["model.embed_tokens.weight"] if config["tie_word_embeddings"] else w["lm_head.weight"]
        torch.testing.assert_close(plain.forward_logits(w, config, tokens), normed @ head.T)


def test_a_layer_norms_before_its_parts_not_after(models):
    """Pre-norm: what a layer adds to the residual stream does not change when the
    stream is scaled, because each part sees the stream through an RMSNorm (the eps
    aside); the stream itself passes unnormed.  A norm after the sum, or a part fed the
    bare stream, fails this."""

    for name, (weights, config) in models.items():
        w = {key: tensor.to(F64) for key, tensor in weights.items()}
        generator = torch.Generator().manual_seed(3)
        h = torch.randn(7, config["hidden_size"], generator=generator, dtype=F64)
        positions = torch.arange(7)
        # the mixer's share alone: the feed-forward adds nothing
        attention_only = dict(w)
        attention_only["model.layers.0.mlp.down_proj.weight"] = torch.zeros_like(w["model.layers.0.mlp.down_proj.weight"])
        added = plain.decoder_layer(h, attention_only, 0, config, positions)[0] - h
        added_scaled = plain.decoder_layer(5.0 * h, attention_only, 0, config, positions)[0] - 5.0 * h
        torch.testing.assert_close(added_scaled, added, atol=1e-6, rtol=1e-4)       # the eps is all that differs
        assert float(added.abs().max()) > 1e-3
        # the feed-forward's share alone: the mixer adds nothing
        mlp_only = dict(w)
        mlp_only["model.layers.0.self_attn.o_proj.weight"] = torch.zeros_like(w["model.layers.0.self_attn.o_proj.weight"])
        added = plain.decoder_layer(h, mlp_only, 0, config, positions)[0] - h
        added_scaled = plain.decoder_layer(5.0 * h, mlp_only, 0, config, positions)[0] - 5.0 * h
        torch.testing.assert_close(added_scaled, added, atol=1e-6, rtol=1e-4)       # the eps is all that differs
        assert float(added.abs().max()) > 1e-3
        # and the whole layer is the stream plus both shares, the second taken of the stream after the first
        after_attention = plain.decoder_layer(h, attention_only, 0, config, positions)[0]
        x = plain.rms_norm(after_attention, w["model.layers.0.post_attention_layernorm.weight"], config["rms_norm_eps"])
        torch.testing.assert_close(plain.decoder_layer(h, w, 0, config, positions)[0],
                                   after_attention + plain.swiglu(x, w, "model.layers.0.mlp."))


def test_only_distances_count(models):
    """A shift of all positions leaves the logits unchanged: the rotation enters
    through q.k alone, which depends on distances."""

    for weights, config in models.values():
        tokens = random_tokens(15, config["vocab_size"], 9)
        base = plain.forward_logits(weights, config, tokens)
        shifted = plain.forward_logits(weights, config, tokens, first_position=37)
        torch.testing.assert_close(shifted, base, atol=2e-4, rtol=0)       # the angle table itself is float32


def test_qk_norm_stands_before_the_rotation_and_v_is_not_normed(models):
    weights, config = models["a"]
    tokens = random_tokens(10, config["vocab_size"], 2)
    base = plain.forward_logits(weights, config, tokens)
    # scaling q_proj rows leaves everything unchanged: the per-head norm removes the scale (eps aside)
    scaled = dict(weights)
    scaled["model.layers.0.self_attn.q_proj.weight"] = weights["model.layers.0.self_attn.q_proj.weight"] * 8.0
    torch.testing.assert_close(plain.forward_logits(scaled, config, tokens), base, atol=1e-5, rtol=0)
    # scaling v_proj does change them: v has no norm
    scaled = dict(weights)
    scaled["model.layers.0.self_attn.v_proj.weight"] = weights["model.layers.0.self_attn.v_proj.weight"] * 8.0
    assert not torch.allclose(plain.forward_logits(scaled, config, tokens), base, atol=1e-3)


def test_order_list_shared_cache_and_windows(models):
    weights, config = models["a"]
    tokens = random_tokens(12, config["vocab_size"], 3)
    base = plain.forward_logits(weights, config, tokens)
    torch.testing.assert_close(plain.forward_logits(weights, config, tokens, order=[(0, None), (1, None)]), base)
    twice = plain.forward_logits(weights, config, tokens, order=[(0, None), (1, None), (0, None)])
    shared = plain.forward_logits(weights, config, tokens, order=[(0, None), (1, None), (0, 0)])
    assert not torch.allclose(twice, base) and not torch.allclose(shared, twice)
    wide = plain.forward_logits(weights, config, tokens, windows=[12, 12])
    torch.testing.assert_close(wide, base)
    narrow = plain.forward_logits(weights, config, tokens, windows=[3, None])
    torch.testing.assert_close(narrow[:3], base[:3])
    assert not torch.allclose(narrow[3:], base[3:])


# ---- sampling --------------------------------------------------------------------------

def test_sampling_vectors_of_the_reference():
    # reference: tests/unit/test_sampling.py:38-49, 123-125
    assert plain_sampling.sample_row(torch.tensor([0.1, 4.0, 3.0]), 0.0, 0, 1.0, 0.3) == 1
    logits = torch.tensor([5.0, 4.0, 3.0, 2.0])
    assert {plain_sampling.sample_row(logits, 1.0, 2, 0.6, u / 20) for u in range(20)} == {0}
    kept = plain_sampling.filter_top_k(torch.tensor([5.0, 5.0, 5.0, 1.0]), 2)
    assert int(torch.isfinite(kept).sum()) == 2
    # top-p keeps the token that crosses the threshold
    probabilities = torch.tensor([0.5, 0.3, 0.15, 0.05])
    kept = plain_sampling.filter_top_p(torch.log(probabilities), 0.6)
    assert torch.isfinite(kept).tolist() == [True, True, False, False]
    # the draw follows the distribution
    counts = torch.zeros(4)
    for u in range(1000):
        counts[plain_sampling.sample_row(torch.log(probabilities), 1.0, 0, 1.0, (u + 0.5) / 1000)] += 1
    torch.testing.assert_close(counts / 1000, probabilities, atol=2e-3, rtol=0)
    # temperature sharpens
    sharp = sum(plain_sampling.sample_row(torch.log(probabilities), 0.25, 0, 1.0, (u + 0.5) / 200) == 0 for u in range(200))
    assert sharp > 170
