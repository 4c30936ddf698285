"""Each part of a layer alone against the plain implementation, and a toy mixer with
state of its own that is registered, built and stepped without a change to the
framework's files."""

from __future__ import annotations

import plain_qwen3 as plain
import pytest
import torch
from helpers import make_model_folder, random_tokens, read_config, read_weights, tiny_a, tiny_b

pytestmark = pytest.mark.gpu

DEVICE = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 1e-5, "bfloat16": 2e-2}


def to_device(weights, dtype):
    return {name: tensor.to(dtype).to(DEVICE).contiguous() for name, tensor in weights.items()}


def oracle_weights(weights, dtype):
    return {name: tensor.to(dtype).double() for name, tensor in weights.items()}


def rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


def step_context(query_lens, starts, block_size, *, tables=None):
    """A StepContext over one cache group, pages handed out in order (or ``tables``)."""

    from miniserve_amd.parts import GroupStepView, StepContext

    token_pos, seq_of, slots, table_rows = [], [], [], []
    next_page = 0
    for index, (qlen, start) in enumerate(zip(query_lens, starts)):
        pages_needed = -(-(start + qlen) // block_size)
        if tables is None:
            row = list(range(next_page, next_page + pages_needed))
            next_page += pages_needed
        else:
            row = tables[index]
        table_rows.append(row)
        for position in range(start, start + qlen):
            token_pos.append(position)
            seq_of.append(index)
            slots.append(row[position // block_size] * block_size + position % block_size)
    width = max(len(r) for r in table_rows)
    table = torch.tensor([r + [0] * (width - len(r)) for r in table_rows], dtype=torch.int32, device=DEVICE)
    i32 = lambda values: torch.tensor(values, dtype=torch.int32, device=DEVICE)
    starts_q = [0]
    for qlen in query_lens:
        starts_q.append(starts_q[-1] + qlen)
    prefix = 0
    while prefix < len(query_lens) and query_lens[prefix] == 1:
        prefix += 1
    tile_seq, tile_token, tile_length, tile_first = [], [], [], []
    for index in range(prefix, len(query_lens)):
        for start in range(0, query_lens[index], 64):
            tile_seq.append(index)
            tile_token.append(starts_q[index] + start)
            tile_length.append(min(64, query_lens[index] - start))
            tile_first.append(starts[index] + start)
    tile_tables = {"attention.tile_seq": i32(tile_seq), "attention.tile_token": i32(tile_token),
                   "attention.tile_length": i32(tile_length), "attention.tile_first": i32(tile_first)}
    return StepContext(
        num_tokens=len(token_pos), num_seqs=len(query_lens), token_ids=i32([0] * len(token_pos)), positions=i32(token_pos),
        seq_of_token=i32(seq_of), query_start=i32(starts_q), context_lens=i32([s + q for s, q in zip(starts, query_lens)]),
        state_slots=i32(list(range(len(query_lens)))), groups=[GroupStepView(table, i32(slots))],
        query_lens=list(query_lens), context_lens_host=[s + q for s, q in zip(starts, query_lens)],
        query_start_host=starts_q, state_slots_host=list(range(len(query_lens))), first_positions_host=list(starts),
        decode_prefix=prefix, tables=tile_tables if tile_seq else {},
    ), table_rows


@pytest.fixture(scope="module", params=["a", "b"])
def model(request, tmp_path_factory):
    make, block = {"a": (tiny_a, 16), "b": (tiny_b, 8)}[request.param]
    folder = make_model_folder(tmp_path_factory.mktemp("parts") / request.param, make(), seed=31)
    from miniserve_amd.config import load_config

    return {"config": read_config(folder), "weights": read_weights(folder), "spec": load_config(folder).model_spec(), "block": block}


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_norm_part(model, dtype):
    from miniserve_amd.parts import build_part

    spec = model["spec"].layers[0].norms["pre_mixer"]
    part = build_part("norm", spec, DTYPES[dtype])
    part.load_weights(to_device(model["weights"], DTYPES[dtype]))
    assert [w.name for w in part.weight_specs()] == ["model.layers.0.input_layernorm.weight"]
    x = rand(9, spec.params["dim"], seed=1).to(DTYPES[dtype])
    expected = plain.rms_norm(x.double(), oracle_weights(model["weights"], DTYPES[dtype])[spec.prefix + "weight"], spec.params["eps"])
    torch.testing.assert_close(part.forward(x.to(DEVICE)).cpu().double(), expected, atol=TOL[dtype], rtol=TOL[dtype])
    residual, delta = rand(9, spec.params["dim"], seed=2).to(DEVICE), x.to(DEVICE)
    total = residual + delta.float()
    out = part.add_forward(residual, delta)
    assert torch.equal(residual, total)
    expected = plain.rms_norm(total.cpu().double(), oracle_weights(model["weights"], DTYPES[dtype])[spec.prefix + "weight"], spec.params["eps"])
    torch.testing.assert_close(out.cpu().double(), expected, atol=TOL[dtype], rtol=TOL[dtype])


def test_position_part(model):
    from miniserve_amd.parts import build_part

    spec = model["spec"].layers[0].mixer.params["position"]
    part = build_part("position", spec, torch.float32)
    assert part.weight_specs() == []
    dim, theta = spec.params["dim"], spec.params["theta"]
    x = rand(6, 3, dim, seed=4)
    positions = torch.tensor([0, 1, 7, 64, 300, 511], dtype=torch.int32, device=DEVICE)
    cos, sin = plain.rope_angles(positions.cpu().long(), dim, theta)
    expected = plain.apply_rope(x.double().transpose(0, 1), cos, sin).transpose(0, 1)
    out = part.apply(x.to(DEVICE), positions)
    torch.testing.assert_close(out.cpu().double(), expected, atol=1e-5, rtol=1e-5)
    # only distances count: <rope(q, m), rope(k, n)> is the same for equal m - n
    q, k = x[:1, :1].to(DEVICE), x[1:2, :1].to(DEVICE)
    at = lambda t, p: part.apply(t, torch.tensor([p], dtype=torch.int32, device=DEVICE))
    dots = [float((at(q, m) * at(k, n)).sum()) for m, n in ((9, 4), (205, 200))]
    assert abs(dots[0] - dots[1]) < 1e-4


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_feed_forward_part(model, dtype):
    from miniserve_amd.parts import build_part

    spec = model["spec"].layers[1].feed_forward
    part = build_part("feed_forward", spec, DTYPES[dtype])
    part.load_weights(to_device(model["weights"], DTYPES[dtype]))
    assert part.w_gate_up.shape == (2 * spec.params["intermediate_size"], spec.params["hidden_size"])
    x = rand(13, spec.params["hidden_size"], seed=5).to(DTYPES[dtype])
    expected = plain.swiglu(x.double(), oracle_weights(model["weights"], DTYPES[dtype]), spec.prefix)
    torch.testing.assert_close(part.forward(x.to(DEVICE)).cpu().double(), expected, atol=TOL[dtype] * 0.1, rtol=TOL[dtype])


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_attention_part_whole_and_in_portions(model, dtype):
    """The mixer alone over its own cache: one request whole, the same request in
    portions beside another request's decoded token, on scattered pages."""

    from miniserve_amd.parts import KVCacheNeed, KVCacheView, build_part

    config, block = model["config"], model["block"]
    spec = model["spec"].layers[0].mixer
    part = build_part("mixer", spec, DTYPES[dtype])
    from miniserve_amd.parts.base import load_part_weights

    load_part_weights(part, to_device(model["weights"], DTYPES[dtype]))
    assert part.cache_need() == KVCacheNeed(config["num_key_value_heads"], config["head_dim"], None)
    assert part.w_qkv.shape[0] == (config["num_attention_heads"] + 2 * config["num_key_value_heads"]) * config["head_dim"]
    hidden, length = config["hidden_size"], 45
    x = rand(length, hidden, seed=6).to(DTYPES[dtype])
    other = rand(20, hidden, seed=7).to(DTYPES[dtype])
    weights = oracle_weights(model["weights"], DTYPES[dtype])
    expected, _ = plain.attention_block(x.double(), weights, spec.prefix, config, torch.arange(length))
    expected_other, _ = plain.attention_block(other.double(), weights, spec.prefix, config, torch.arange(20))

    def fresh_cache(pages):
        heads, dim = config["num_key_value_heads"], config["head_dim"]
        return KVCacheView(0, torch.full((pages, heads, block, dim), float("nan"), dtype=DTYPES[dtype], device=DEVICE),
                           torch.full((pages, heads, dim, block), float("nan"), dtype=DTYPES[dtype], device=DEVICE), block)

    cache = fresh_cache(8)
    ctx, _ = step_context([length], [0], block)
    out = part.forward(x.to(DEVICE), ctx, cache)
    torch.testing.assert_close(out.cpu().double(), expected, atol=TOL[dtype] * 0.1, rtol=TOL[dtype])

    cache = fresh_cache(16)
    tables = [[15, 3, 9, 0, 7, 12], [5, 1, 14]]
    outs, position = [], 0
    ctx, _ = step_context([19], [0], block, tables=[tables[1]])
    part.forward(other[:19].to(DEVICE), ctx, cache)                                    # the other request's history
    for size in (7, 2, 13, 23):
        if position == 9:      # this portion runs beside the other request's decoded token
            ctx, _ = step_context([size, 1], [position, 19], block, tables=tables)
            batch = torch.cat([x[position : position + size], other[19:20]]).to(DEVICE)
            result = part.forward(batch, ctx, cache)
            outs.append(result[:size])
            torch.testing.assert_close(result[size:].cpu().double(), expected_other[19:20], atol=TOL[dtype] * 0.1, rtol=TOL[dtype])
        else:
            ctx, _ = step_context([size], [position], block, tables=[tables[0]])
            outs.append(part.forward(x[position : position + size].to(DEVICE), ctx, cache))
        position += size
    torch.testing.assert_close(torch.cat(outs).cpu().double(), expected, atol=TOL[dtype] * 0.1, rtol=TOL[dtype])


def test_attention_part_composed_from_its_parts_equals_the_fused_kernel(model):
    """With a position part that the fused kernel does not know, the mixer runs the
    norms and the position encoding through their own parts; same result."""

    from miniserve_amd.config import PartSpec
    from miniserve_amd.parts import KVCacheView, Part, build_part, register_part, unregister_part
    from miniserve_amd.parts.base import load_part_weights
    from miniserve_amd.parts.rotary import RotaryHalf

    class WrappedRotary(Part):
        """The same function behind a class that the attention part does not recognise."""

        def __init__(self, spec, dtype):
            self.inner = RotaryHalf(spec, dtype)

        def apply(self, x, positions):
            return self.inner.apply(x, positions)

    register_part("position", "test_wrapped_rotary", WrappedRotary)
    try:
        spec = model["spec"].layers[0].mixer
        params = dict(spec.params)
        params["position"] = PartSpec("test_wrapped_rotary", spec.params["position"].params)
        fused = build_part("mixer", spec, torch.float32)
        composed = build_part("mixer", PartSpec("attention", params, spec.prefix), torch.float32)
        assert fused._fused and not composed._fused
        config, block = model["config"], model["block"]
        weights = to_device(model["weights"], torch.float32)
        x = rand(21, config["hidden_size"], seed=8).to(DEVICE)
        results = []
        for part in (fused, composed):
            load_part_weights(part, dict(weights))     # a part drops what it has stacked from the mapping it gets
            heads, dim = config["num_key_value_heads"], config["head_dim"]
            cache = KVCacheView(0, torch.zeros((4, heads, block, dim), device=DEVICE),
                                torch.zeros((4, heads, dim, block), device=DEVICE), block)
            ctx, _ = step_context([21], [0], block)
            results.append((part.forward(x, ctx, cache), cache.key.clone(), cache.value.clone()))
        for got, want in zip(results[1], results[0]):
            torch.testing.assert_close(got, want, atol=1e-6, rtol=1e-6)
    finally:
        unregister_part("position", "test_wrapped_rotary")


@pytest.mark.parametrize("dtype", list(DTYPES))
def test_block_embedding_and_head(model, dtype):
    from miniserve_amd.parts import KVCacheView, build_block, build_part
    from miniserve_amd.parts.base import load_part_weights

    config, block_size, spec = model["config"], model["block"], model["spec"]
    device_weights = to_device(model["weights"], DTYPES[dtype])
    weights = oracle_weights(model["weights"], DTYPES[dtype])
    tokens = random_tokens(30, config["vocab_size"], 3)
    embedding = build_part("embedding", spec.embedding, DTYPES[dtype])
    embedding.load_weights(device_weights)
    h = embedding.forward(torch.tensor(tokens, dtype=torch.int32, device=DEVICE))
    assert h.dtype == torch.float32
    assert torch.equal(h.cpu().double(), weights["model.embed_tokens.weight"][tokens])

    layer = build_block(spec.layers[1], DTYPES[dtype])
    load_part_weights(layer, device_weights)
    heads, dim = config["num_key_value_heads"], config["head_dim"]
    cache = KVCacheView(0, torch.zeros((4, heads, block_size, dim), dtype=DTYPES[dtype], device=DEVICE),
                        torch.zeros((4, heads, dim, block_size), dtype=DTYPES[dtype], device=DEVICE), block_size)
    ctx, _ = step_context([30], [0], block_size)
    residual, delta = layer.forward(h.clone(), None, ctx, cache)
    expected, _ = plain.decoder_layer(h.cpu().double(), weights, 1, config, torch.arange(30))
    total = residual if delta is None else residual + delta.float()        # a part may have added its output itself
    torch.testing.assert_close(total.cpu().double(), expected, atol=TOL[dtype], rtol=TOL[dtype])

    head = build_part("head", spec.head, DTYPES[dtype])
    head.load_weights(device_weights)
    y = rand(5, config["hidden_size"], seed=9).to(DTYPES[dtype])
    matrix = weights["model.embed_tokens.weight"] if config["tie_word_embeddings"] else weights["lm_head.weight"]
    logits = head.forward(y.to(DEVICE))
    assert logits.dtype == torch.float32 and logits.shape == (5, config["vocab_size"])
    torch.testing.assert_close(logits.cpu().double(), y.double() @ matrix.T, atol=TOL[dtype], rtol=TOL[dtype])
    if config["tie_word_embeddings"]:
        assert head.weight.data_ptr() == embedding.weight.data_ptr()                   # the very same tensor


def test_blocks_that_prepare_the_norm_behind_a_product(model, monkeypatch):
    """bfloat16 and 30 rows, where the norm would be a kernel of its own: each product that
    adds into the residual stream leaves the next norm prepared (between the parts of a
    block, and for the block that follows when it is named), the product behind the norm
    is made from that, and two blocks give what the plain implementation gives.  What was
    prepared for another norm than the one that is taken is left alone."""

    from miniserve_amd import ops
    from miniserve_amd.parts import KVCacheView, PreparedNorm, build_block, build_part
    from miniserve_amd.parts.base import load_part_weights

    config, block_size, spec = model["config"], model["block"], model["spec"]
    dtype = torch.bfloat16
    device_weights = to_device(model["weights"], dtype)
    weights = oracle_weights(model["weights"], dtype)
    rows = 30
    h = rand(rows, config["hidden_size"], seed=12).to(DEVICE)
    layers = [build_block(spec.layers[index], dtype) for index in (0, 1)]
    for layer in layers:
        load_part_weights(layer, device_weights)
    heads, dim = config["num_key_value_heads"], config["head_dim"]
    caches = [KVCacheView(0, torch.zeros((4, heads, block_size, dim), dtype=dtype, device=DEVICE),
                          torch.zeros((4, heads, dim, block_size), dtype=dtype, device=DEVICE), block_size) for _ in layers]
    ctx, _ = step_context([rows], [0], block_size)
    calls = {"made": 0, "used": 0}
    make, use = ops.linear_norm_ahead, ops.linear_prepared

    def counted(function, key):
        def wrapper(*args, **kwargs):
            calls[key] += 1
            return function(*args, **kwargs)
        return wrapper

    monkeypatch.setattr(ops, "linear_norm_ahead", counted(make, "made"))
    monkeypatch.setattr(ops, "linear_prepared", counted(use, "used"))
    assert layers[1].takes_prepared_norm(rows) and not layers[1].takes_prepared_norm(8)   # few rows: the norm as prologue
    expected = h.cpu().double()
    for index in (0, 1):
        expected, _ = plain.decoder_layer(expected, weights, index, config, torch.arange(rows))

    residual, delta = layers[0].forward(h.clone(), None, ctx, caches[0], norm_after=layers[1].first_norm)
    assert isinstance(delta, PreparedNorm) and delta.norm is layers[1].first_norm and calls == {"made": 2, "used": 1}
    residual, delta = layers[1].forward(residual, delta, ctx, caches[1])
    assert delta is None and calls == {"made": 3, "used": 3}
    torch.testing.assert_close(residual.cpu().double(), expected, atol=TOL["bfloat16"], rtol=TOL["bfloat16"])
    prepared_way = residual.clone()

    # prepared for a norm that is not the one taken next: not used, and nothing is lost
    other = build_part("norm", spec.layers[1].norms["pre_mixer"], dtype)
    other.load_weights(device_weights)
    residual, delta = layers[0].forward(h.clone(), None, ctx, caches[0], norm_after=other)
    assert isinstance(delta, PreparedNorm) and delta.norm is other
    residual, delta = layers[1].forward(residual, delta, ctx, caches[1])
    assert calls == {"made": 6, "used": 5}
    torch.testing.assert_close(residual.cpu().double(), expected, atol=TOL["bfloat16"], rtol=TOL["bfloat16"])
    # the norm as a kernel of its own and as prepared scales differ by roundings alone
    torch.testing.assert_close(residual, prepared_way, atol=TOL["bfloat16"], rtol=TOL["bfloat16"])
