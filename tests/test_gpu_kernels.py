"""Each kernel alone against a plain torch reference, at other sizes than the
engine's: around the wave (63/64/65) and workgroup edges, head sizes in steps of
16, widths and vocabularies that are no power of two (the reference tests its op
at 1, 31, 32, 33, 257, 1024, 1031: tests/cuda_extension/test_vector_add.py:23)."""

from __future__ import annotations

import math

import plain_qwen3 as plain
import plain_sampling
import pytest
import torch

pytestmark = pytest.mark.gpu

DEVICE = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def rand(*shape, seed=0, dtype=torch.float32, scale=1.0):
    generator = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=generator) * scale).to(dtype).to(DEVICE)


def tolerance(dtype, f32=2e-5, bf16=4e-3):
    # the reference's own tolerances: 2e-5 float32 / 4e-3 half for the norm
    # (miniserve/toolchain/benchmark_rmsnorm.py:73), 2e-4 / 8e-3 for attention
    return f32 if dtype == torch.float32 else bf16


# Attention in bfloat16: the reference allows 8e-3 for float16 (11 significant bits);
# bfloat16 carries 8, and the weights P are rounded to it before the second product,
# as in the reference's chunk form.  Twice the float16 figure.
ATTENTION_BF16 = 1.6e-2


@pytest.fixture(scope="module")
def ops():
    from miniserve_amd import ops as module

    module.load()
    assert module.library_path().endswith("libminiserve_hip.so")
    return module


# ---- embedding --------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [1, 63, 64, 65, 257, 1031])
def test_embedding_gather(ops, dtype, hidden):
    table = rand(509, hidden, seed=hidden, dtype=dtype)
    ids = torch.tensor([0, 508, 3, 3, 77, 256], dtype=torch.int32, device=DEVICE)
    out = ops.embedding_gather(ids, table)
    assert out.dtype == torch.float32
    assert torch.equal(out, table[ids.long()].float())


# ---- RMSNorm ----------------------------------------------------------------------------

def rmsnorm_reference(x, weight, eps, storage):
    """32-bit statistics, round to storage, multiply by the weight (layers.py:30-34)."""

    values = x.double()
    normed = (values * torch.rsqrt(values.pow(2).mean(-1, keepdim=True) + eps)).to(storage)
    return (weight.double() * normed.double()).to(storage)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 1024), (7, 1024), (33, 1024), (4, 4096), (3, 1), (5, 63), (5, 65), (2, 96), (9, 5120), (2, 1031)])
def test_rmsnorm_shapes_of_the_reference_and_edges(ops, dtype, shape):
    # reference shapes: miniserve/toolchain/benchmark_rmsnorm.py:97, seed 7000 + rows + hidden (:68)
    rows, dim = shape
    x = rand(rows, dim, seed=7000 + rows + dim, dtype=dtype)
    weight = torch.linspace(0.5, 1.5, dim).to(dtype).to(DEVICE)
    out = ops.rmsnorm(x, weight, 1e-6)
    expected = rmsnorm_reference(x, weight, 1e-6, dtype)
    torch.testing.assert_close(out.double(), expected.double(), atol=tolerance(dtype), rtol=tolerance(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("dim", [200, 256, 1028, 2056, 5120, 9000, 16388])      # both kernels, every number of groups a thread
def test_rmsnorm_residual_forms(ops, dtype, dim):
    residual = rand(6, dim, seed=1)
    delta = rand(6, dim, seed=2, dtype=dtype)
    weight = (1 + 0.1 * rand(dim, seed=3)).to(dtype)
    total = residual + delta.float()
    kept = residual.clone()
    out = ops.rmsnorm(kept, weight, 1e-5, delta=delta, write_back=True)
    assert torch.equal(kept, total)                                             # h <- h + delta in 32-bit
    expected = rmsnorm_reference(total, weight, 1e-5, dtype)
    torch.testing.assert_close(out.double(), expected.double(), atol=tolerance(dtype), rtol=tolerance(dtype))
    rows = torch.tensor([5, 0, 3], dtype=torch.int32, device=DEVICE)
    kept = residual.clone()
    picked = ops.rmsnorm(kept, weight, 1e-5, delta=delta, rows=rows)
    assert torch.equal(kept, residual)                                          # gathered rows write nothing back
    assert torch.equal(picked, out[rows.long()])
    # a row's result does not depend on the batch around it
    alone = ops.rmsnorm(residual[2:3].clone(), weight, 1e-5, delta=delta[2:3].contiguous(), write_back=True)
    assert torch.equal(alone[0], out[2])


def test_rmsnorm_vector_of_the_reference(ops):
    # tests/correctness/test_rmsnorm_reference.py:23-32
    values = torch.tensor([[0.0, 1.0, -1.0, 1e-4, -1e-4, 8.0, -8.0, 2.0]], device=DEVICE)
    weight = torch.linspace(0.75, 1.25, 8, device=DEVICE)
    expected = plain.rms_norm(values.cpu().double(), weight.cpu().double(), 1e-6)
    torch.testing.assert_close(ops.rmsnorm(values, weight, 1e-6).cpu().double(), expected, atol=1e-6, rtol=1e-6)


def test_kernels_refuse_what_they_cannot_do(ops):
    from miniserve_amd.ops import KernelError

    x = rand(4, 64)
    with pytest.raises(KernelError, match="GPU"):
        ops.rmsnorm(x.cpu(), torch.ones(64), 1e-6)
    with pytest.raises(KernelError, match="does not match"):
        ops.rmsnorm(x, torch.ones(65, device=DEVICE), 1e-6)
    with pytest.raises(KernelError, match="float32 or bfloat16"):
        ops.silu_mul(x.half())
    with pytest.raises(KernelError, match="eps"):
        ops.rmsnorm(x, torch.ones(64, device=DEVICE), 0.0)
    with pytest.raises(KernelError, match="contiguous"):
        ops.silu_mul(x.t())
    with pytest.raises(KernelError, match="exceeds"):
        ops.qk_norm_rope_append(rand(1, 1026), num_q_heads=1, num_kv_heads=0, head_dim=1026, q_weight=None,
                                k_weight=None, eps=1.0, rope=None)
    with pytest.raises(KernelError, match="even"):
        ops.qk_norm_rope_append(rand(1, 15), num_q_heads=1, num_kv_heads=0, head_dim=15, q_weight=None,
                                k_weight=None, eps=1.0, rope=None)


# ---- q/k norm, rotation, cache write ------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,block", [(4, 2, 16, 16), (8, 1, 32, 8), (3, 3, 48, 5), (16, 8, 128, 16), (2, 1, 256, 4), (5, 1, 80, 3)])
def test_qk_norm_rope_append(ops, dtype, heads, kv_heads, dim, block):
    from miniserve_amd.parts.rotary import inverse_frequencies

    n, pages, theta, eps = 11, 9, 50000.0, 1e-5
    packed = rand(n, (heads + 2 * kv_heads) * dim, seed=dim, dtype=dtype)
    qw = (1 + 0.1 * rand(dim, seed=1)).to(dtype)
    kw = (1 + 0.1 * rand(dim, seed=2)).to(dtype)
    positions = torch.tensor([0, 1, 2, 63, 64, 65, 1000, 4095, 7, 7, 30000], dtype=torch.int32, device=DEVICE)
    slots = torch.randperm(pages * block, generator=torch.Generator().manual_seed(3))[:n].to(torch.int32).to(DEVICE)
    key_pool = torch.zeros(pages, kv_heads, block, dim, dtype=dtype, device=DEVICE)
    value_pool = torch.zeros(pages, kv_heads, dim, block, dtype=dtype, device=DEVICE)     # transposed inside a page
    q = ops.qk_norm_rope_append(
        packed, num_q_heads=heads, num_kv_heads=kv_heads, head_dim=dim, q_weight=qw, k_weight=kw, eps=eps,
        rope=ops.rope_table(positions, inverse_frequencies(dim, theta).to(DEVICE)), slot_mapping=slots,
        key_pool=key_pool, value_pool=value_pool,
    )
    rows = packed.cpu().double().view(n, heads + 2 * kv_heads, dim)
    cos, sin = plain.rope_angles(positions.cpu().long(), dim, theta)

    def prepare(x, weight):
        normed = rmsnorm_reference(x, weight.cpu(), eps, dtype).double()
        return plain.apply_rope(normed.transpose(0, 1), cos, sin).transpose(0, 1)

    expected_q = prepare(rows[:, :heads], qw)
    expected_k = prepare(rows[:, heads : heads + kv_heads], kw)
    expected_v = rows[:, heads + kv_heads :]
    tol = tolerance(dtype, 1e-5, 1.6e-2)         # one bfloat16 rounding of values up to ~4
    torch.testing.assert_close(q.cpu().double(), expected_q, atol=tol, rtol=tol)
    page, offset = slots.cpu().long() // block, slots.cpu().long() % block
    torch.testing.assert_close(key_pool.cpu().double()[page, :, offset], expected_k, atol=tol, rtol=tol)
    values = value_pool.cpu().double().transpose(2, 3)                                     # [page, head, offset, d]
    assert torch.equal(values[page, :, offset], expected_v)
    touched = torch.zeros(pages, block, dtype=torch.bool)
    touched[page, offset] = True
    untouched = lambda pool: pool.permute(0, 2, 1, 3)[~touched]
    assert torch.all(untouched(key_pool.cpu()) == 0) and torch.all(untouched(values) == 0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,block,start", [(4, 2, 128, 16, 5), (2, 1, 80, 8, 0), (3, 3, 16, 12, 7), (2, 2, 64, 4, 3), (1, 1, 512, 16, 9), (16, 8, 128, 16, 2), (5, 2, 32, 16, 0)])
def test_append_of_a_run_of_tokens_beside_single_ones(ops, dtype, heads, kv_heads, dim, block, start):
    """A portion of a prompt that starts in the middle of a page and runs over several
    pages (handed out in reverse), behind three single tokens in pages of their own:
    every key and value lands in its slot and nothing else is touched."""

    from miniserve_amd.parts.rotary import inverse_frequencies

    run, theta, eps = max(150, 4 * 256 * 16 // dim + 40), 1e4, 1e-6     # enough for the many-token kernel
    run_pages = (start + run + block - 1) // block
    pages = run_pages + 3
    table = list(range(run_pages - 1, -1, -1))                                  # logical -> physical page
    run_slots = [table[(start + i) // block] * block + (start + i) % block for i in range(run)]
    single_slots = [(run_pages + i) * block + (3 * i + 1) % block for i in range(3)]
    slots = torch.tensor(single_slots + run_slots, dtype=torch.int32, device=DEVICE)
    n = len(slots)
    positions = torch.tensor([900, 17, 4000] + list(range(start, start + run)), dtype=torch.int32, device=DEVICE)
    packed = rand(n, (heads + 2 * kv_heads) * dim, seed=dim + block, dtype=dtype)
    qw = (1 + 0.1 * rand(dim, seed=1)).to(dtype)
    kw = (1 + 0.1 * rand(dim, seed=2)).to(dtype)
    key_pool = torch.zeros(pages, kv_heads, block, dim, dtype=dtype, device=DEVICE)
    value_pool = torch.zeros(pages, kv_heads, dim, block, dtype=dtype, device=DEVICE)
    q = ops.qk_norm_rope_append(
        packed, num_q_heads=heads, num_kv_heads=kv_heads, head_dim=dim, q_weight=qw, k_weight=kw, eps=eps,
        rope=ops.rope_table(positions, inverse_frequencies(dim, theta).to(DEVICE)), slot_mapping=slots,
        key_pool=key_pool, value_pool=value_pool,
    )
    rows = packed.cpu().double().view(n, heads + 2 * kv_heads, dim)
    cos, sin = plain.rope_angles(positions.cpu().long(), dim, theta)

    def prepare(x, weight):
        normed = rmsnorm_reference(x, weight.cpu(), eps, dtype).double()
        return plain.apply_rope(normed.transpose(0, 1), cos, sin).transpose(0, 1)

    tol = tolerance(dtype, 1e-5, 1.6e-2)
    torch.testing.assert_close(q.cpu().double(), prepare(rows[:, :heads], qw), atol=tol, rtol=tol)
    page, offset = slots.cpu().long() // block, slots.cpu().long() % block
    torch.testing.assert_close(key_pool.cpu().double()[page, :, offset], prepare(rows[:, heads : heads + kv_heads], kw),
                               atol=tol, rtol=tol)
    values = value_pool.cpu().double().transpose(2, 3)
    assert torch.equal(values[page, :, offset], rows[:, heads + kv_heads :])
    touched = torch.zeros(pages, block, dtype=torch.bool)
    touched[page, offset] = True
    untouched = lambda pool: pool.permute(0, 2, 1, 3)[~touched]
    assert torch.all(untouched(key_pool.cpu()) == 0) and torch.all(untouched(values) == 0)


def test_rotation_and_norm_alone(ops):
    """Without weights the kernel is the rotation alone; without frequencies the norm alone."""

    from miniserve_amd.parts.rotary import inverse_frequencies

    x = rand(5, 3 * 32, seed=9)
    positions = torch.tensor([0, 3, 9, 100, 511], dtype=torch.int32, device=DEVICE)
    only_rope = ops.qk_norm_rope_append(x, num_q_heads=3, num_kv_heads=0, head_dim=32, q_weight=None, k_weight=None,
                                        eps=1.0, rope=ops.rope_table(positions, inverse_frequencies(32, 1e4).to(DEVICE)))
    cos, sin = plain.rope_angles(positions.cpu().long(), 32, 1e4)
    expected = plain.apply_rope(x.cpu().double().view(5, 3, 32).transpose(0, 1), cos, sin).transpose(0, 1)
    torch.testing.assert_close(only_rope.cpu().double(), expected, atol=1e-5, rtol=1e-5)
    assert torch.equal(only_rope[0], x.view(5, 3, 32)[0])                       # position 0 is the identity
    weight = 1 + 0.1 * rand(32, seed=4)
    only_norm = ops.qk_norm_rope_append(x, num_q_heads=3, num_kv_heads=0, head_dim=32, q_weight=weight, k_weight=None,
                                        eps=1e-6, rope=None)
    torch.testing.assert_close(only_norm.view(15, 32), ops.rmsnorm(x.view(15, 32), weight, 1e-6), atol=1e-6, rtol=1e-6)


# ---- attention over the paged cache -------------------------------------------------------

def paged_case(batch_contexts, heads, kv_heads, dim, block, dtype, *, query_lens=None, seed=0, reverse=True):
    """Random q and cache for sequences of the given context lengths; each sequence
    brings ``query_lens[i]`` last positions as queries.  Pages are handed out in
    reversed order so that physical order differs from logical order, as the
    reference's own check does (miniserve/toolchain/benchmark_paged_decode.py:26-60)."""

    generator = torch.Generator().manual_seed(seed)
    query_lens = query_lens or [1] * len(batch_contexts)
    blocks_each = [-(-c // block) for c in batch_contexts]
    total = sum(blocks_each) + 2
    order = list(range(total - 1, -1, -1)) if reverse else list(range(total))
    key_pool = torch.full((total, kv_heads, block, dim), float("nan"))
    value_pool = torch.full((total, kv_heads, block, dim), float("nan"))
    table = torch.zeros(len(batch_contexts), max(blocks_each), dtype=torch.int32)
    keys, values, queries, seq_of_token, positions = [], [], [], [], []
    cursor = 0
    for index, (context, qlen) in enumerate(zip(batch_contexts, query_lens)):
        k = torch.randn(context, kv_heads, dim, generator=generator).to(dtype).float()
        v = torch.randn(context, kv_heads, dim, generator=generator).to(dtype).float()
        q = torch.randn(qlen, heads, dim, generator=generator).to(dtype).float()
        for logical in range(blocks_each[index]):
            page = order[cursor]
            cursor += 1
            table[index, logical] = page
            span = slice(logical * block, min((logical + 1) * block, context))
            key_pool[page, :, : span.stop - span.start] = k[span].transpose(0, 1)
            value_pool[page, :, : span.stop - span.start] = v[span].transpose(0, 1)
        keys.append(k)
        values.append(v)
        queries.append(q)
        seq_of_token += [index] * qlen
        positions += list(range(context - qlen, context))
    return {
        "q": torch.cat(queries).to(dtype).to(DEVICE),
        "key_pool": key_pool.to(dtype).to(DEVICE),
        "value_pool": value_pool.transpose(2, 3).contiguous().to(dtype).to(DEVICE),      # [page, head, d, offset]
        "block_table": table.to(DEVICE),
        "seq_of_token": torch.tensor(seq_of_token, dtype=torch.int32, device=DEVICE),
        "positions": torch.tensor(positions, dtype=torch.int32, device=DEVICE),
        "keys": keys, "values": values, "queries": queries, "query_lens": query_lens,
    }


def attention_reference(case, scale, window=None):
    outs = []
    for k, v, q in zip(case["keys"], case["values"], case["queries"]):
        context, qlen = k.shape[0], q.shape[0]
        padded = torch.zeros(context, q.shape[1], q.shape[2], dtype=torch.float64)
        padded[context - qlen :] = q.double()
        full = plain.causal_attention(padded.transpose(0, 1), k.double().transpose(0, 1), v.double().transpose(0, 1), scale, window)
        outs.append(full.transpose(0, 1)[context - qlen :])
    return torch.cat(outs)


def query_tiles(case, first_sequence, by_keys=False):
    """Tiles of at most 64 consecutive tokens for the sequences from ``first_sequence`` on,
    in the order of the batch, or (``by_keys``) as the attention part makes them: in the
    order of the keys they walk."""

    from miniserve_amd.ops import QueryTiles, query_tiles_host

    starts = [0]
    for qlen in case["query_lens"]:
        starts.append(starts[-1] + qlen)
    if starts[first_sequence] == starts[-1]:
        return None
    firsts = [int(case["positions"][start]) for start in starts[:-1]]
    lists = query_tiles_host(case["query_lens"], starts[:-1], first_sequence, firsts, by_keys=by_keys)
    device = case["q"].device
    return QueryTiles(len(lists[0]), *(torch.tensor(values, dtype=torch.int32, device=device) for values in lists),
                      by_keys=by_keys)


def run_attention(ops, case, scale, window=None, splits=None, by_keys=False):
    """As the engine calls it: sequences that bring one token stand first and are
    served as single tokens, the others in tiles."""

    lens = case["query_lens"]
    prefix = 0
    while prefix < len(lens) and lens[prefix] == 1:
        prefix += 1
    return ops.attention(case["q"], case["key_pool"], case["value_pool"], block_table=case["block_table"],
                         seq_of_token=case["seq_of_token"], positions=case["positions"], scale=scale, window=window,
                         decode_prefix=prefix, tiles=query_tiles(case, prefix, by_keys),
                         max_context=int(case["positions"].max()) + 1, splits=splits)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("batch,context", [(1, 1), (1, 17), (2, 33), (4, 65)])
def test_paged_decode_workloads_of_the_reference(ops, dtype, batch, context):
    # Hq16 / Hkv8 / bs16 / D128, reversed tables, seed 8800 + 100 B + C; 2e-4 float32, 8e-3 half
    # (miniserve/toolchain/benchmark_paged_decode.py:26-60, 112-116, 141)
    case = paged_case([context] * batch, 16, 8, 128, 16, dtype, seed=8800 + 100 * batch + context)
    out = run_attention(ops, case, 128**-0.5)
    expected = attention_reference(case, 128**-0.5)
    tol = tolerance(dtype, 2e-4, ATTENTION_BF16)
    torch.testing.assert_close(out.cpu().double(), expected, atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,block", [(4, 2, 16, 16), (8, 1, 32, 8), (6, 3, 48, 5), (5, 5, 80, 7), (2, 1, 256, 32), (12, 4, 64, 16), (3, 1, 112, 1)])
def test_attention_sizes_chunks_and_decode_rows_in_one_batch(ops, dtype, heads, kv_heads, dim, block):
    contexts = [1, 63, 64, 65, 130, 257]
    query_lens = [1, 1, 64, 7, 130, 2]           # decode rows, whole prompts and portions side by side
    case = paged_case(contexts, heads, kv_heads, dim, block, dtype, query_lens=query_lens, seed=dim + block)
    out = run_attention(ops, case, dim**-0.5)
    expected = attention_reference(case, dim**-0.5)
    tol = tolerance(dtype, 2e-4, ATTENTION_BF16)
    torch.testing.assert_close(out.cpu().double(), expected, atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", DTYPES)
def test_one_far_key_among_hundreds_stands_out(ops, dtype):
    """Random keys give near-uniform weights, which would hide a lost page.  Here one
    key, far back, carries almost all the weight, and its value is unlike all others."""

    for far in (0, 15, 16, 17, 300, 511, 512, 700):
        case = paged_case([701], 4, 2, 64, 16, dtype, seed=far)
        k, v = case["keys"][0], case["values"][0]
        q = case["queries"][0]
        page, offset = int(case["block_table"][0, far // 16]), far % 16
        k[far] = 0.0
        q[0] = 0.0
        q[0, :, 0] = 8.0
        k[far, :, 0] = 8.0                                                      # score 64 * scale = 8 above the rest
        v[far] = 100.0
        case["q"] = q.to(dtype).to(DEVICE)
        case["key_pool"][page, :, offset] = k[far].to(dtype).to(DEVICE)
        case["value_pool"][page, :, :, offset] = v[far].to(dtype).to(DEVICE)
        out = run_attention(ops, case, 64**-0.5)
        expected = attention_reference(case, 64**-0.5)
        assert float(expected.min()) > 10.0                                     # the far key dominates
        tol = tolerance(dtype, 2e-4, ATTENTION_BF16)
        torch.testing.assert_close(out.cpu().double(), expected, atol=tol * 100, rtol=tol)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 5, 16, 64, 100])
def test_window_edges(ops, dtype, window):
    """The key just inside the window carries a large value, the key just outside a
    huge one: an edge off by one changes the result beyond any tolerance."""

    contexts, query_lens = [131, 70, 9], [3, 70, 1]
    case = paged_case(contexts, 4, 2, 32, 8, dtype, query_lens=query_lens, seed=window)
    for index, (context, v) in enumerate(zip(contexts, case["values"])):
        last = context - 1
        inside, outside = last - window + 1, last - window
        for position, value in ((inside, 50.0), (outside, -1000.0)):
            if position >= 0:
                v[position] = value
                page = int(case["block_table"][index, position // 8])
                case["value_pool"][page, :, :, position % 8] = value
    out = run_attention(ops, case, 32**-0.5, window=window)
    expected = attention_reference(case, 32**-0.5, window=window)
    tol = tolerance(dtype, 2e-4, ATTENTION_BF16)
    torch.testing.assert_close(out.cpu().double(), expected, atol=tol * 50, rtol=tol)


@pytest.mark.parametrize("heads,kv_heads,dim,block", [(16, 8, 128, 16), (8, 1, 64, 16), (4, 4, 32, 32), (20, 1, 16, 16), (6, 2, 80, 48), (32, 2, 256, 64), (3, 1, 112, 16)])
def test_decode_kernel_sizes_splits_and_windows(ops, heads, kv_heads, dim, block):
    """The matrix-core kernel for single-token rows: groups of 1 to 20 query heads
    (more than 16 take two passes), head sizes in steps of 16, contexts around
    tile (16), pair (32) and split edges, any number of key splits, windows."""

    contexts = [1, 15, 16, 17, 31, 32, 33, 63, 64, 65, 129, 700, 2500]
    case = paged_case(contexts, heads, kv_heads, dim, block, torch.bfloat16, seed=dim + heads)
    assert ops.load().ms_attention_decode_supported(dim, block)
    expected = attention_reference(case, dim**-0.5)
    for splits in (1, 2, 5, 16, 64, None):
        out = run_attention(ops, case, dim**-0.5, splits=splits)
        torch.testing.assert_close(out.cpu().double(), expected, atol=ATTENTION_BF16, rtol=ATTENTION_BF16, msg=lambda m: f"splits {splits}: {m}")
    for window in (1, 16, 17, 100, 1000):
        expected = attention_reference(case, dim**-0.5, window=window)
        for splits in (1, 3, None):
            out = run_attention(ops, case, dim**-0.5, window=window, splits=splits)
            torch.testing.assert_close(out.cpu().double(), expected, atol=ATTENTION_BF16, rtol=ATTENTION_BF16,
                                       msg=lambda m: f"window {window} splits {splits}: {m}")


@pytest.mark.parametrize("heads,kv_heads,dim,block", [(16, 8, 128, 16), (8, 1, 64, 16), (4, 4, 32, 32), (3, 1, 16, 16), (6, 2, 80, 48), (32, 8, 128, 64), (5, 1, 112, 16)])
def test_tiled_kernel_sizes_portions_and_windows(ops, heads, kv_heads, dim, block):
    """The matrix-core kernel for runs of query tokens: whole prompts, portions that
    start and end off the tile and page grid, single tokens after the prefix, groups
    of 1 to 8 heads, head sizes in steps of 16, windows."""

    contexts = [1, 1, 130, 16, 17, 64, 700, 33, 300]
    query_lens = [1, 1, 130, 16, 2, 31, 150, 1, 300]          # two single tokens first, one more later
    case = paged_case(contexts, heads, kv_heads, dim, block, torch.bfloat16, query_lens=query_lens, seed=dim + heads)
    assert ops.load().ms_attention_prefill_supported(dim, block)
    out = run_attention(ops, case, dim**-0.5)
    torch.testing.assert_close(out.cpu().double(), attention_reference(case, dim**-0.5), atol=ATTENTION_BF16, rtol=ATTENTION_BF16)
    for window in (1, 15, 16, 17, 100):
        out = run_attention(ops, case, dim**-0.5, window=window)
        expected = attention_reference(case, dim**-0.5, window=window)
        torch.testing.assert_close(out.cpu().double(), expected, atol=ATTENTION_BF16, rtol=ATTENTION_BF16, msg=lambda m: f"window {window}: {m}")


@pytest.mark.parametrize("by_keys", [False, True])
@pytest.mark.parametrize("contexts,query_lens,heads,kv_heads,dim", [
    ([2048], [2048], 16, 8, 128),                 # a prompt of the served sizes: 32 tiles, the last walks 2,048 keys;
                                                  # one head and four parts a workgroup, a long and a short tile each
    ([1100, 1200], [1100, 1200], 32, 8, 64),      # two prompts, two workgroups of heads to a kv head
    ([700, 300, 40], [500, 33, 40], 4, 1, 32),    # portions with history, an odd tail
    ([1500] * 3, [1000] * 3, 4, 4, 48),           # one head a workgroup
    ([1990, 130], [1990 - 64, 130], 16, 8, 128),  # an odd number of tiles: the middle one has a workgroup to itself
    ([3000], [3000], 40, 8, 128),                 # two heads a workgroup, tiles in pairs
])
def test_tiled_kernel_over_long_prompts(ops, contexts, query_lens, heads, kv_heads, dim, by_keys):
    """Prompts of a thousand tokens and more (dozens of tiles, walks of thousands of
    keys), against the plain attention, with a window as well; the tiles in the order of
    the batch (a tile a workgroup) and in the order of their keys (where the launch is
    small, a long and a short tile a workgroup)."""

    case = paged_case(contexts, heads, kv_heads, dim, 16, torch.bfloat16, query_lens=query_lens, seed=dim)
    for window in (None, 300):
        out = run_attention(ops, case, dim**-0.5, window=window, by_keys=by_keys)
        expected = attention_reference(case, dim**-0.5, window=window)
        torch.testing.assert_close(out.cpu().double(), expected, atol=ATTENTION_BF16, rtol=ATTENTION_BF16,
                                   msg=lambda m: f"window {window}: {m}")


def test_tiled_kernel_ignores_stale_values(ops):
    case = paged_case([37, 70], 8, 2, 64, 16, torch.bfloat16, query_lens=[20, 70], seed=4)   # unused slots hold NaN
    assert torch.isnan(case["value_pool"]).any()
    out = run_attention(ops, case, 0.125)
    assert torch.isfinite(out).all()
    torch.testing.assert_close(out.cpu().double(), attention_reference(case, 0.125), atol=ATTENTION_BF16, rtol=ATTENTION_BF16)


def test_decode_kernel_ignores_stale_values(ops):
    """Slots past the context inside the last page hold NaN (as fresh pages may):
    a zero weight times NaN must not reach the output."""

    case = paged_case([5, 21, 40], 8, 2, 64, 16, torch.bfloat16, seed=1)       # paged_case fills unused slots with NaN
    assert torch.isnan(case["value_pool"]).any() and torch.isnan(case["key_pool"]).any()
    out = run_attention(ops, case, 0.125)
    assert torch.isfinite(out).all()
    torch.testing.assert_close(out.cpu().double(), attention_reference(case, 0.125), atol=ATTENTION_BF16, rtol=ATTENTION_BF16)


@pytest.mark.parametrize("dtype", DTYPES)
def test_pages_whose_offsets_pass_32_bits(ops, dtype):
    """A pool sized for the card's memory has pages that lie more than 2^31 elements into
    it.  The same keys and values at such pages give the results they give at pages 0, 1,
    2, ... to the bit, from the single-token kernel, the tiled kernel, the generic one (32-bit)
    and the kernel that writes the cache: an offset computed in 32 bits would read or write
    elsewhere.  (The pools are not initialised; 9 and 17 GB of the card's 288.)"""

    from miniserve_amd.parts.rotary import inverse_frequencies

    heads, kv_heads, dim, block = 16, 8, 128, 16
    scale = dim**-0.5
    case = paged_case([300, 77, 150], heads, kv_heads, dim, block, dtype, query_lens=[1, 1, 40], seed=5)
    low = run_attention(ops, case, scale)
    small_pages = case["key_pool"].shape[0]
    pages = (1 << 31) // (kv_heads * block * dim) + 600
    key_pool = torch.empty(pages, kv_heads, block, dim, dtype=dtype, device=DEVICE)
    value_pool = torch.empty(pages, kv_heads, dim, block, dtype=dtype, device=DEVICE)
    moved = torch.arange(pages - 1, pages - 1 - small_pages, -1, device=DEVICE)          # page i lies at pages - 1 - i
    assert int(moved.min()) * kv_heads * block * dim > 1 << 31
    key_pool[moved] = case["key_pool"]
    value_pool[moved] = case["value_pool"]
    high_case = dict(case, key_pool=key_pool, value_pool=value_pool,
                     block_table=(pages - 1 - case["block_table"]).to(torch.int32))
    high = run_attention(ops, high_case, scale)
    assert torch.equal(low, high)

    # the write: the same tokens to slots of low pages and to the same places of high ones
    n, region = 150, 12                      # enough tokens for the tiled form; the pages they and two more are written to
    packed = rand(n, (heads + 2 * kv_heads) * dim, seed=3, dtype=dtype)
    weight = (1 + 0.1 * rand(dim, seed=1)).to(dtype)
    positions = torch.arange(5, 5 + n, dtype=torch.int32, device=DEVICE)
    rope = ops.rope_table(positions, inverse_frequencies(dim, 1e6).to(DEVICE))
    slots = torch.arange(3, 3 + n, dtype=torch.int32, device=DEVICE)
    pools = {}
    for name, shift in (("low", 0), ("high", (pages - region) * block)):
        if shift == 0:
            keys = torch.zeros(region, kv_heads, block, dim, dtype=dtype, device=DEVICE)
            values = torch.zeros(region, kv_heads, dim, block, dtype=dtype, device=DEVICE)
        else:
            keys, values = key_pool, value_pool
            keys[pages - region :] = 0
            values[pages - region :] = 0
        for count in (n, 2):                         # many tokens: the tiled form; two: a token a workgroup
            ops.qk_norm_rope_append(packed[:count], num_q_heads=heads, num_kv_heads=kv_heads, head_dim=dim, q_weight=weight,
                                    k_weight=weight, eps=1e-6, rope=(rope[0][:count].contiguous(), rope[1][:count].contiguous()),
                                    slot_mapping=(slots[:count] + shift + (0 if count == n else n)).contiguous(),
                                    key_pool=keys, value_pool=values)
        pools[name] = (keys[-region:].clone(), values[-region:].clone())
    assert torch.equal(pools["low"][0], pools["high"][0]) and torch.equal(pools["low"][1], pools["high"][1])
    assert bool(pools["low"][0].any()) and bool(pools["low"][1].any())
    del key_pool, value_pool, high_case, keys, values
    torch.cuda.empty_cache()


def test_decode_kernel_is_refused_for_other_geometries(ops):
    lib = ops.load()
    assert not lib.ms_attention_decode_supported(128, 8)          # pages of 8 keys
    assert not lib.ms_attention_decode_supported(24, 16)          # head size off the 16 grid
    assert not lib.ms_attention_decode_supported(272, 16)
    assert not lib.ms_attention_prefill_supported(144, 16)        # large heads are served token by token
    assert lib.ms_attention_decode_supported(144, 16)
    big = paged_case([40, 3], 2, 1, 144, 16, torch.bfloat16, query_lens=[40, 1], seed=3)
    torch.testing.assert_close(run_attention(ops, big, 144**-0.5).cpu().double(), attention_reference(big, 144**-0.5),
                               atol=ATTENTION_BF16, rtol=ATTENTION_BF16)
    case = paged_case([30, 9], 8, 1, 32, 8, torch.bfloat16, seed=2)
    out = run_attention(ops, case, 32**-0.5)                       # falls to the generic kernel
    torch.testing.assert_close(out.cpu().double(), attention_reference(case, 32**-0.5), atol=ATTENTION_BF16, rtol=ATTENTION_BF16)


def test_attention_is_bit_identical_across_batches_in_float32(ops):
    case = paged_case([200, 77], 4, 2, 48, 16, torch.float32, query_lens=[200, 1], seed=5)
    together = run_attention(ops, case, 0.2)
    alone = dict(case)                       # the same cache, only the last query of each sequence
    alone["q"] = torch.stack([case["q"][199], case["q"][200]])
    alone["seq_of_token"] = torch.tensor([0, 1], dtype=torch.int32, device=DEVICE)
    alone["positions"] = torch.tensor([199, 76], dtype=torch.int32, device=DEVICE)
    alone["query_lens"] = [1, 1]
    separate = run_attention(ops, alone, 0.2)
    assert torch.equal(separate[0], together[199]) and torch.equal(separate[1], together[200])


# ---- products and activation ---------------------------------------------------------------

@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (1, 509, 96), (63, 65, 17), (64, 64, 16), (65, 63, 33), (130, 200, 257), (7, 1031, 64)])
def test_gemm_f32_is_true_32_bit(ops, m, n, k):
    x, w = rand(m, k, seed=m), rand(n, k, seed=n + 1)
    out = ops.linear(x, w)
    expected = x.cpu().double() @ w.cpu().double().T
    torch.testing.assert_close(out.cpu().double(), expected, atol=1e-5 * math.sqrt(k), rtol=1e-6)
    # sequential accumulation over k in float32, exactly
    if k <= 33:
        acc = torch.zeros(m, n)
        xc, wc = x.cpu(), w.cpu()
        for index in range(k):
            acc = torch.addcmul(acc, xc[:, index : index + 1], wc[:, index].unsqueeze(0))
        assert float((out.cpu() - acc).abs().max()) <= 1e-6
    # a row's result does not depend on the rows around it
    row = ops.linear(x[m // 2 : m // 2 + 1].contiguous(), w)
    assert torch.equal(row[0], out[m // 2])
    target = rand(m, n, seed=5)
    before = target.clone()
    ops.linear(x, w, accumulate_into=target)
    assert torch.equal(target, before + out)


def test_linear_bfloat16_and_fused_projection_rows(ops):
    """One product over stacked q|k|v (or gate|up) rows equals the separate products."""

    x = rand(37, 96, seed=1, dtype=torch.bfloat16)
    parts = [rand(n, 96, seed=10 + n, dtype=torch.bfloat16, scale=0.05) for n in (256, 32, 32)]
    fused = ops.linear(x, torch.cat(parts).contiguous())
    offset = 0
    for part in parts:
        expected = (x.cpu().double() @ part.cpu().double().T)
        torch.testing.assert_close(fused[:, offset : offset + part.shape[0]].cpu().double(), expected, atol=2e-2, rtol=2e-2)
        offset += part.shape[0]
    x32 = x.float()
    fused32 = ops.linear(x32, torch.cat(parts).float().contiguous())
    assert torch.equal(fused32[:, 256:288], ops.linear(x32, parts[1].float()))


@pytest.mark.parametrize("m", [1, 8, 15, 16, 17, 33, 64])
@pytest.mark.parametrize("n,k", [(16, 32), (509, 96), (100, 200), (4096, 1024), (1024, 3072), (72, 2056), (40, 4104), (40000, 64),
                                 (5130, 72), (6144, 2048)])       # from 5120 rows on two blocks a workgroup
def test_skinny_product_for_few_rows(ops, m, n, k, monkeypatch):
    """The matrix-core product that decoding uses (at most 64 rows), with its four
    epilogues, against float64; sizes off the tile grid in every dimension."""

    assert ops.load().ms_gemm_skinny_supported(m, n, k, 0)
    monkeypatch.setattr(ops, "_forced_product", "skinny")                  # the kernel itself, whatever the rule says
    x = rand(m, k, seed=m + k, dtype=torch.bfloat16)
    w = rand(n, k, seed=n, dtype=torch.bfloat16, scale=0.05)
    exact = x.cpu().double() @ w.cpu().double().T
    scale = float(exact.abs().max())
    out = ops.linear(x, w)
    assert out.dtype == torch.bfloat16
    torch.testing.assert_close(out.cpu().double(), exact, atol=scale * 2**-8, rtol=2**-8)
    wide = ops.linear(x, w, out_float32=True)
    assert wide.dtype == torch.float32
    torch.testing.assert_close(wide.cpu().double(), exact, atol=scale * 1e-5, rtol=1e-5)
    assert torch.equal(wide.to(torch.bfloat16), out)                       # one rounding, at the end
    target = rand(m, n, seed=3)
    before = target.clone()
    ops.linear(x, w, accumulate_into=target)
    torch.testing.assert_close(target, before + wide, atol=1e-6, rtol=1e-6)
    # a row's result is the same to the bit whatever rows stand beside it
    alone = ops.linear(x[m // 2 : m // 2 + 1].contiguous(), w, out_float32=True)
    assert torch.equal(alone[0], wide[m // 2])
    if n % 2 == 0:
        fused = ops.linear_silu_mul(x, w)
        assert torch.equal(fused, ops.silu_mul(out))                        # the same as product, rounding, activation


def test_product_beyond_64_rows_uses_the_library(ops):
    assert not ops.load().ms_gemm_skinny_supported(65, 128, 64, 0)
    assert not ops.load().ms_gemm_skinny_supported(8, 128, 60, 0)          # k off the 8 grid
    x, w = rand(65, 60, seed=1, dtype=torch.bfloat16), rand(33, 60, seed=2, dtype=torch.bfloat16)
    exact = x.cpu().double() @ w.cpu().double().T
    torch.testing.assert_close(ops.linear(x, w).cpu().double(), exact, atol=0.1, rtol=2**-7)
    torch.testing.assert_close(ops.linear(x[:8].contiguous(), w, out_float32=True).cpu().double(), exact[:8], atol=0.1, rtol=2**-7)
    torch.testing.assert_close(ops.linear_silu_mul(x, w[:32].contiguous()), ops.silu_mul(ops.linear(x, w[:32].contiguous())))


@pytest.mark.parametrize("m,n,k", [(17, 512, 96), (40, 1024, 1024), (64, 300, 200), (8, 8192, 2048), (33, 4096, 1024)])
def test_either_product_serves_a_shape_that_both_take(ops, m, n, k):
    """Which product serves a shape is a fixed rule; forced to either one, the call
    gives the product, plain, in 32-bit, added into a 32-bit tensor and with the gated
    activation, eagerly and inside a recording alike."""

    x, w = rand(m, k, seed=m, dtype=torch.bfloat16), rand(n, k, seed=n, dtype=torch.bfloat16, scale=0.1)
    exact = x.cpu().double() @ w.cpu().double().T
    scale = float(exact.abs().max())
    by_rule = ops.linear(x, w)
    results = {}
    for which in ("skinny", "library"):
        with ops.forced_product(which):
            before = dict(ops.product_calls)
            results[which] = ops.linear(x, w)
            assert ops.product_calls[which] == before[which] + 1
            assert ops.prefers_skinny(m, n, k) == (which == "skinny")
            assert ops.can_fuse_norm(min(m, 16), w) == (which == "skinny")
            gated = ops.linear_silu_mul(x, w)
            assert torch.equal(gated, ops.silu_mul(results[which]))          # the activation of the rounded product
            torch.testing.assert_close(results[which].cpu().double(), exact, atol=scale * 2**-8, rtol=2**-7)
            wide = ops.linear(x, w, out_float32=True)
            torch.testing.assert_close(wide.cpu().double(), exact, atol=scale * 1e-5, rtol=1e-5)
            total = torch.ones(m, n, device=DEVICE)
            ops.linear(x, w, accumulate_into=total)
            torch.testing.assert_close(total.cpu().double(), 1 + exact, atol=scale * 1e-5, rtol=1e-5)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                recorded = ops.linear(x, w)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(recorded, results[which])                    # a recording takes the same kernel
    assert torch.equal(by_rule, results["skinny" if ops.prefers_skinny(m, n, k) else "library"])
    with pytest.raises(ValueError):
        with ops.forced_product("other"):
            pass


@pytest.mark.parametrize("m,n,k", [(17, 509, 96), (65, 33, 60), (300, 1024, 200), (2048, 4096, 1024), (129, 300, 80)])
def test_library_product_for_many_rows(ops, m, n, k, monkeypatch):
    """The product through hipBLASLt, bound at run time to the copy the process has:
    bfloat16 out, 32-bit out, and += into a 32-bit tensor; sizes off every grid; the
    same shape again takes the kept plan."""

    monkeypatch.setattr(ops, "_forced_product", "library")   # no choice between the two products here
    x, w = rand(m, k, seed=m, dtype=torch.bfloat16), rand(n, k, seed=n, dtype=torch.bfloat16, scale=0.1)
    exact = x.cpu().double() @ w.cpu().double().T
    scale = float(exact.abs().max())
    for _ in range(2):
        torch.testing.assert_close(ops.linear(x, w).cpu().double(), exact, atol=scale * 2**-8, rtol=2**-7)
        wide = ops.linear(x, w, out_float32=True)
        assert wide.dtype == torch.float32
        torch.testing.assert_close(wide.cpu().double(), exact, atol=scale * 1e-5, rtol=1e-5)
        base = rand(m, n, seed=5)
        total = base.clone()
        assert ops.linear(x, w, accumulate_into=total) is total
        torch.testing.assert_close(total.cpu().double(), base.cpu().double() + exact, atol=scale * 1e-5, rtol=1e-5)
    from miniserve_amd.ops import KernelError

    assert ops.can_accumulate(m, w)
    with pytest.raises(KernelError, match="must have shape"):
        ops.linear(x, w, accumulate_into=torch.zeros(m, n + 1, device=DEVICE))


@pytest.mark.parametrize("m,n,k", [(64, 512, 256), (64, 1024, 2048), (33, 1024, 3072), (48, 4096, 1024), (64, 6144, 1024)])
def test_library_product_inside_a_recorded_graph(ops, monkeypatch, m, n, k):
    """Replayed several times with eager work between the replays; every replay gives
    what the eager call gives for the inputs of that moment: plain, and added into a
    32-bit tensor (the shapes of a decode step of 33 to 64 rows among them)."""

    monkeypatch.setattr(ops, "_forced_product", "library")
    x = rand(m, k, seed=1, dtype=torch.bfloat16)
    w = rand(n, k, seed=2, dtype=torch.bfloat16, scale=0.1)
    base = rand(m, n, seed=3)
    ops.linear(x, w)                                        # plan and workspace exist before the recording
    ops.linear(x, w, accumulate_into=base.clone())
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    total = base.clone()
    with torch.cuda.graph(graph):
        out = ops.linear(x, w, out_float32=True)
        ops.linear(x, w, accumulate_into=total)
    for round_index in range(4):
        x.copy_(rand(m, k, seed=10 + round_index, dtype=torch.bfloat16))
        total.copy_(base)
        graph.replay()
        torch.cuda.synchronize()
        expected = ops.linear(x, w, out_float32=True)       # eager work between the replays
        expected_total = ops.linear(x, w, accumulate_into=base.clone())
        torch.cuda.synchronize()
        assert torch.equal(out, expected)
        assert torch.equal(total, expected_total)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,inter", [(1, 1), (3, 63), (5, 200), (64, 3072), (2, 1031)])
def test_silu_mul(ops, dtype, rows, inter):
    gate_up = rand(rows, 2 * inter, seed=inter, dtype=dtype, scale=3.0)
    out = ops.silu_mul(gate_up)
    g, u = gate_up.cpu().double()[:, :inter], gate_up.cpu().double()[:, inter:]
    expected = torch.nn.functional.silu(g) * u
    tol = tolerance(dtype, 1e-6, 8e-3)
    torch.testing.assert_close(out.cpu().double(), expected, atol=tol, rtol=tol)
    zero_gate = gate_up.clone()
    zero_gate[:, :inter] = 0
    assert torch.all(ops.silu_mul(zero_gate) == 0)


def test_residual_add(ops):
    h, delta = rand(5, 77, seed=1), rand(5, 77, seed=2, dtype=torch.bfloat16)
    expected = h + delta.float()
    ops.residual_add(h, delta)
    assert torch.equal(h, expected)


# ---- sampling -------------------------------------------------------------------------------

def test_greedy_is_argmax_with_the_lowest_index_among_equals(ops):
    logits = rand(9, 1031, seed=3)
    logits[2, 700] = logits[2, 30] = 50.0
    logits[5] = 1.25
    out = ops.sample_rows(logits)
    expected = torch.argmax(logits, dim=-1).cpu()
    expected[2], expected[5] = 30, 0
    assert out.cpu().tolist() == expected.tolist()
    assert ops.sample_rows(torch.tensor([[0.1, 4.0, 3.0]], device=DEVICE)).tolist() == [1]     # test_sampling.py:38-41


def test_greedy_over_a_large_vocabulary(ops):
    """From 4096 tokens on the greedy choice runs in two stages over chunks of the row."""

    for vocab in (4096, 4097, 151936):
        logits = rand(5, vocab, seed=vocab)
        logits[1, vocab - 1] = logits[1, 17] = 60.0                      # equal maxima in the first and the last chunk
        logits[2, vocab // 2] = 70.0
        logits[3, :] = -3.5
        logits[4, vocab - 2] = float("inf")
        expected = torch.argmax(logits, dim=-1).cpu().tolist()
        expected[1], expected[3], expected[4] = 17, 0, -1
        assert ops.sample_rows(logits).cpu().tolist() == expected


def test_non_finite_logits_are_reported(ops):
    # reference: tests/unit/test_sampling.py:90-102
    logits = rand(4, 300, seed=1)
    logits[1, 5], logits[2, 7], logits[3, 9] = float("nan"), float("inf"), float("-inf")
    assert ops.sample_rows(logits).tolist()[1:] == [-1, -1, -1]


@pytest.mark.parametrize("vocab", [2, 64, 509, 1031, 151936])
def test_sampling_matches_the_plain_implementation(ops, vocab):
    generator = torch.Generator().manual_seed(vocab)
    rows = 24
    logits = (torch.randn(rows, vocab, generator=generator) * 3).to(DEVICE)
    temperature = torch.tensor([0.0, 0.3, 0.8, 1.0, 1.5, 2.0] * 4)
    top_k = torch.tensor(([0] * 6 + [1] * 6 + [min(5, vocab)] * 6 + [min(50, vocab)] * 6), dtype=torch.int32)
    top_p = torch.tensor([1.0, 0.9, 0.5, 1.0, 0.1, 0.99] * 4)[torch.randperm(rows, generator=generator)]
    uniform = torch.rand(rows, generator=generator)
    out = ops.sample_rows(logits, temperature=temperature.to(DEVICE), top_k=top_k.to(DEVICE),
                          top_p=top_p.to(DEVICE), uniform=uniform.to(DEVICE)).cpu().tolist()
    for row in range(rows):
        expected = plain_sampling.sample_row(
            logits[row].cpu(), float(temperature[row]), int(top_k[row]), float(top_p[row]), float(uniform[row])
        )
        assert out[row] == expected, f"row {row}: T={temperature[row]} k={top_k[row]} p={top_p[row]} u={uniform[row]}"


def test_sampling_from_the_short_list_and_from_the_whole_row(ops):
    """With top-k or top-p the kernels gather the tokens near the maximum into a list and
    choose among them: in LDS when they are few (4096), in device memory when they are
    many (top-k 4097 and 5000 here), and over the whole row when no distance from the
    maximum holds them (top-p 0.9999); all give the plain implementation's token.  Rows
    with a few outstanding tokens (as a model's logits have) and flat rows."""

    vocab, rows = 50021, 36
    generator = torch.Generator().manual_seed(7)
    logits = torch.randn(rows, vocab, generator=generator) * 2
    for row in range(0, rows, 2):                       # every other row: 40 tokens stand out
        chosen = torch.randperm(vocab, generator=generator)[:40]
        logits[row, chosen] += 8 + 6 * torch.rand(40, generator=generator)
    temperature = torch.tensor([0.6, 0.6, 1.0, 1.0, 1.3, 1.3] * 6)
    top_k = torch.tensor([0, 0, 20, 20, 5000, 5000, 0, 0, 1, 1, 4096, 4097] * 3, dtype=torch.int32)
    top_p = torch.tensor([0.5, 0.5, 0.95, 0.95, 0.9, 0.9, 0.9999, 0.9999, 0.3, 0.3, 1.0, 0.8] * 3)
    uniform = torch.rand(rows, generator=generator)
    out = ops.sample_rows(logits.to(DEVICE), temperature=temperature.to(DEVICE), top_k=top_k.to(DEVICE),
                          top_p=top_p.to(DEVICE), uniform=uniform.to(DEVICE)).cpu().tolist()
    for row in range(rows):
        expected = plain_sampling.sample_row(
            logits[row], float(temperature[row]), int(top_k[row]), float(top_p[row]), float(uniform[row])
        )
        assert out[row] == expected, f"row {row}: T={temperature[row]} k={top_k[row]} p={top_p[row]} u={uniform[row]}"


def test_sampling_from_flat_rows_of_the_served_vocabulary(ops):
    """Rows without outstanding tokens (a model with random weights gives such rows), 151,936
    tokens wide: no distance below the maximum holds the tokens that can stay, so the choice
    walks a list as long as the row or the row itself; with a small top-k the list is short
    again.  Every row gives the plain implementation's token."""

    vocab = 151936
    generator = torch.Generator().manual_seed(21)
    options = [(0.8, 0, 0.9), (0.8, 0, 0.5), (1.0, 5000, 1.0), (0.8, 50, 0.9), (1.5, 0, 0.99), (0.7, 20000, 0.7),
               (1.0, 0, 1.0), (0.8, 1, 0.9), (0.8, vocab, 0.9), (0.9, vocab, 0.6)]      # (a top-k of the whole row is no cut)
    rows = len(options)
    logits = torch.randn(rows, vocab, generator=generator) * torch.tensor([0.2, 0.64] * (rows // 2))[:, None]
    temperature = torch.tensor([o[0] for o in options])
    top_k = torch.tensor([o[1] for o in options], dtype=torch.int32)
    top_p = torch.tensor([o[2] for o in options])
    for trial in range(3):
        uniform = torch.rand(rows, generator=generator)
        out = ops.sample_rows(logits.to(DEVICE), temperature=temperature.to(DEVICE), top_k=top_k.to(DEVICE),
                              top_p=top_p.to(DEVICE), uniform=uniform.to(DEVICE)).cpu().tolist()
        # (the rows with top-p alone were searched by their chunks together; without those kernels the one
        # workgroup of the choice searches them, and finds the same)
        alone = ops.sample_rows(logits.to(DEVICE), temperature=temperature.to(DEVICE), top_k=top_k.to(DEVICE),
                                top_p=top_p.to(DEVICE), uniform=uniform.to(DEVICE), top_p_alone=False).cpu().tolist()
        for row in range(rows):
            case = (logits[row], float(temperature[row]), int(top_k[row]), float(top_p[row]), float(uniform[row]))
            expected = plain_sampling.sample_row(*case)
            for got in (out[row], alone[row]):
                if got != expected:
                    # The kernels take every token's share in 32-bit (7 digits) where the plain form has 16,
                    # and a nucleus of up to 130,000 tokens is added up: a draw that lies within that rounding
                    # of the edge between two tokens' shares (some 7e-6 wide here) may fall to the neighbour.
                    running = plain_sampling.running_sums(*case[:4])
                    kept = torch.nonzero(torch.diff(running, prepend=torch.zeros(1, dtype=running.dtype)) > 0).flatten().tolist()
                    assert got in kept and abs(kept.index(got) - kept.index(expected)) == 1, (
                        f"trial {trial} row {row}: {got}, not {expected} nor its neighbour")
                    assert plain_sampling.edge_distance(*case) < 1e-6, (
                        f"trial {trial} row {row}: T={temperature[row]} k={top_k[row]} p={top_p[row]} u={uniform[row]}: "
                        f"{got} != {expected} and the draw is on no edge")


def test_the_sampling_workspace_is_sized_by_the_library(ops):
    """The workspace of the chunked choice is sized by the library's own entry point: it
    grows with the rows and the vocabulary, and a smaller one is refused."""

    from miniserve_amd.ops.library import KernelError, call, load

    wanted = load().ms_sample_rows_workspace_bytes
    assert wanted(1, 8192) < wanted(1, 50021) < wanted(3, 50021) < wanted(64, 151936)
    rows, vocab = 3, 50021
    logits = torch.randn(rows, vocab, device=DEVICE)
    ones = torch.ones(rows, device=DEVICE)
    out = torch.empty(rows, dtype=torch.int32, device=DEVICE)
    small = torch.empty(wanted(rows, vocab) - 8, dtype=torch.uint8, device=DEVICE)
    with pytest.raises(KernelError, match="workspace"):
        call("ms_sample_rows_chunked", logits.data_ptr(), ones.data_ptr(), None, ones.data_ptr(), ones.data_ptr(),
             out.data_ptr(), small.data_ptr(), small.numel(), rows, vocab, 0, torch.cuda.current_stream().cuda_stream)


def test_rmsnorm_refuses_32_bit_rows_that_are_not_aligned(ops):
    """Rows of the 32-bit stream are read 16 bytes at a time; a view that starts inside
    a row is refused, not served by a kernel whose sums have another order."""

    from miniserve_amd.ops.library import KernelError

    dim = 1024
    weight = torch.ones(dim, dtype=torch.bfloat16, device=DEVICE)
    buffer = torch.randn(3 * dim + 1, device=DEVICE)
    aligned = ops.rmsnorm(buffer[: 3 * dim].view(3, dim), weight, 1e-6)
    assert aligned.shape == (3, dim)
    with pytest.raises(KernelError, match="16-byte aligned"):
        ops.rmsnorm(buffer[1:].view(3, dim), weight, 1e-6)
    # a short row is read value by value and may lie anywhere
    assert ops.rmsnorm(buffer[1 : 1 + 3 * 100].view(3, 100), torch.ones(100, dtype=torch.bfloat16, device=DEVICE), 1e-6).shape == (3, 100)


def test_equal_values_at_the_edge_of_top_k_keep_the_lowest_indices(ops):
    """A hundred tokens share the k-th largest value, spread over a long row: exactly k
    tokens stay, the equal ones with the lowest indices, and every one of them can be drawn."""

    vocab, k, rows = 30011, 30, 200
    generator = torch.Generator().manual_seed(11)
    row = torch.randn(vocab, generator=generator) - 6
    above = torch.randperm(vocab, generator=generator)[:110]
    row[above[:10]] = 7.0 + torch.arange(10) * 0.25            # ten tokens above the tie
    tied = torch.sort(above[10:]).values
    row[tied] = 6.5                                             # a hundred equal ones; twenty of them stay
    logits = row.repeat(rows, 1).to(DEVICE)
    out = ops.sample_rows(
        logits, temperature=torch.ones(rows, device=DEVICE), top_k=torch.full((rows,), k, dtype=torch.int32, device=DEVICE),
        top_p=torch.ones(rows, device=DEVICE), uniform=((torch.arange(rows) + 0.5) / rows).to(DEVICE),
    ).cpu().tolist()
    allowed = set(above[:10].tolist()) | set(tied[:20].tolist())
    assert set(out) <= allowed
    assert set(tied[:20].tolist()) <= set(out)                  # 200 evenly spaced draws reach each of the 30


def test_sampling_vectors_of_the_reference(ops):
    # [5,4,3,2], T=1, k=2, p=0.6 -> always 0 (tests/unit/test_sampling.py:44-49)
    logits = torch.tensor([[5.0, 4.0, 3.0, 2.0]] * 20, device=DEVICE)
    out = ops.sample_rows(
        logits, temperature=torch.ones(20, device=DEVICE), top_k=torch.full((20,), 2, dtype=torch.int32, device=DEVICE),
        top_p=torch.full((20,), 0.6, device=DEVICE), uniform=(torch.arange(20, device=DEVICE) / 20.0),
    )
    assert out.tolist() == [0] * 20
    # ties keep exactly k (tests/unit/test_sampling.py:123-125): [5,5,5,1] with k=2 never gives index 2 or 3
    tied = torch.tensor([[5.0, 5.0, 5.0, 1.0]] * 50, device=DEVICE)
    out = ops.sample_rows(
        tied, temperature=torch.ones(50, device=DEVICE), top_k=torch.full((50,), 2, dtype=torch.int32, device=DEVICE),
        top_p=torch.ones(50, device=DEVICE), uniform=(torch.arange(50, device=DEVICE) + 0.5) / 50.0,
    )
    assert set(out.tolist()) == {0, 1}


def test_the_draw_follows_the_distribution(ops):
    probabilities = torch.tensor([0.5, 0.3, 0.15, 0.05])
    n = 4000
    logits = torch.log(probabilities).repeat(n, 1).to(DEVICE)
    out = ops.sample_rows(logits, temperature=torch.ones(n, device=DEVICE), uniform=((torch.arange(n) + 0.5) / n).to(DEVICE))
    counts = torch.bincount(out.cpu().long(), minlength=4).float() / n
    torch.testing.assert_close(counts, probabilities, atol=1e-3, rtol=0)


def test_sampler_stages_without_advancing_the_stream(ops):
    # reference: tests/unit/test_sampling.py:71-87
    from miniserve_amd.engine import SamplingParams
    from miniserve_amd.sampling import NonFiniteLogitsError, Sampler

    sampler = Sampler()
    logits = torch.tensor([[0.1, 1.0, 2.0, 3.0]], device=DEVICE)
    params = SamplingParams(temperature=1.0, seed=17)
    first = sampler.stage(logits, [("staged", params)])
    second = sampler.stage(logits, [("staged", params)])
    assert first[0].token_id == second[0].token_id and sampler.active_request_ids == ()
    stream = torch.Generator().manual_seed(17)
    draws = [Sampler.draw_uniform(stream) for _ in range(2)]
    expected = [plain_sampling.sample_row(logits[0].cpu(), 1.0, 0, 1.0, u) for u in draws]
    assert first[0].token_id == expected[0]
    sampler.commit(first)
    assert sampler.active_request_ids == ("staged",)
    assert sampler.stage(logits, [("staged", params)])[0].token_id == expected[1]
    sampler.release("staged")
    sampler.release("staged")
    assert sampler.active_request_ids == ()
    greedy = sampler.sample(logits, [("g", SamplingParams())])
    assert greedy == [3] and sampler.active_request_ids == ()                  # greedy makes no stream
    with pytest.raises(NonFiniteLogitsError, match="finite"):
        sampler.sample(torch.tensor([[0.0, float("nan")]], device=DEVICE), [("n", SamplingParams())])
    with pytest.raises(ValueError, match="vocabulary"):
        sampler.sample(logits, [("k", SamplingParams(temperature=1.0, top_k=5))])
    with pytest.raises(TypeError, match="floating-point"):
        sampler.sample(torch.tensor([[1, 2, 3]], device=DEVICE), [("i", SamplingParams())])


@pytest.mark.parametrize("m", [1, 7, 16])
@pytest.mark.parametrize("n,k", [(48, 64), (512, 96), (4096, 1024), (200, 200), (96, 2056), (64, 4104)])
def test_product_with_the_norm_as_its_prologue(ops, m, n, k):
    """RMSNorm of the 32-bit residual stream fused into the few-rows product equals the
    norm kernel followed by the product, also with the gated activation behind it."""

    residual = rand(m, k, seed=m + n, scale=2.0)
    norm_weight = (1 + 0.1 * rand(k, seed=5)).to(torch.bfloat16)
    weight = rand(n, k, seed=n + k, dtype=torch.bfloat16, scale=0.05)
    assert ops.can_fuse_norm(m, weight) and ops.can_fuse_norm(m, weight, gated=True)
    normed = ops.rmsnorm(residual, norm_weight, 1e-5)
    fused = ops.linear_normed(residual, norm_weight, 1e-5, weight)
    torch.testing.assert_close(fused.float(), ops.linear(normed, weight).float(), atol=2e-2, rtol=2e-2)
    exact = rmsnorm_reference(residual, norm_weight, 1e-5, torch.bfloat16).cpu().double() @ weight.cpu().double().T
    torch.testing.assert_close(fused.cpu().double(), exact, atol=float(exact.abs().max()) * 2**-7, rtol=2**-7)
    # gated: the error of silu(gate) * up comes from the operands, not the result.  Each of
    # gate and up carries its own rounding to bfloat16 (2^-9 of its size) and the roundings
    # of the k normalised inputs (at most 2^-9 each, independent, once here and twice in
    # `exact`: a sum whose standard deviation is 2^-9 sqrt(3/3) |x . w|_2, taken six times);
    # silu' <= 1.1.
    gated = ops.linear_normed(residual, norm_weight, 1e-5, weight, gated=True)
    normed_exact = rmsnorm_reference(residual, norm_weight, 1e-5, torch.bfloat16).cpu().double()
    spread = 6 * 2**-9 * (normed_exact.pow(2) @ weight.cpu().double().pow(2).T).sqrt()
    slack = 2**-9 * exact.abs() + spread
    gate, up = exact[:, : n // 2], exact[:, n // 2 :]
    wanted = torch.nn.functional.silu(gate) * up
    silu_slack = 1.1 * slack[:, : n // 2]
    bound = (silu_slack * up.abs() + (torch.nn.functional.silu(gate).abs() + silu_slack) * slack[:, n // 2 :]
             + 2**-8 * wanted.abs() + 1e-6)
    ratio = ((gated.cpu().double() - wanted).abs() / bound).max()
    assert float(ratio) <= 1.0, f"fused: error / bound = {float(ratio):.2f}"
    ratio = ((ops.linear_silu_mul(normed, weight).cpu().double() - wanted).abs() / bound).max()
    assert float(ratio) <= 1.0, f"unfused: error / bound = {float(ratio):.2f}"
    assert not ops.can_fuse_norm(17, weight)
    assert not ops.can_fuse_norm(m, weight.float())


@pytest.mark.parametrize("m", [1, 7, 16, 17, 40, 64])
@pytest.mark.parametrize("width,before,after", [(1024, 3072, 4096), (200, 96, 72), (4096, 1024, 6144), (5120, 64, 512),
                                                (72, 2056, 5128)])
def test_product_that_prepares_the_norm_behind_it(ops, m, width, before, after):
    """``h += x W1^T`` that leaves, for the RMSNorm of the new h, the weighted values and
    every workgroup's sum of squares; and the product of that norm made from the two.
    The first is the plain += to the bit, its by-products are what torch makes of the
    new h; the second is held against the norm and the product in float64 with nothing
    rounded (bound as in the test below), and the gated form is the activation of the
    plain one to the bit.  Widths with 13 to 512 workgroups of sums; 1 to 64 rows."""

    x = rand(m, before, seed=m + before, dtype=torch.bfloat16)
    w1 = rand(width, before, seed=width, dtype=torch.bfloat16, scale=0.05)
    w2 = rand(after, width, seed=after + 1, dtype=torch.bfloat16, scale=0.05)
    norm_weight = (1 + 0.1 * rand(width, seed=5)).to(torch.bfloat16)
    start = rand(m, width, seed=3, scale=2.0)
    with ops.forced_product("skinny"):
        assert ops.can_prepare_norm(m, w1) and ops.can_use_prepared_norm(m, w2) and ops.can_use_prepared_norm(m, w2, gated=True)
        plain = start.clone()
        ops.linear(x, w1, accumulate_into=plain)
        h = start.clone()
        weighted, squares = ops.linear_norm_ahead(x, w1, h, norm_weight)
        assert torch.equal(h, plain)
        assert torch.equal(weighted, (norm_weight.float() * h).to(torch.bfloat16))
        assert squares.shape == (ops.load().ms_gemm_skinny_groups(m, width), m)
        torch.testing.assert_close(squares.double().sum(0), h.double().pow(2).sum(-1), atol=0, rtol=1e-6)
        out = ops.linear_prepared(weighted, squares, 1e-5, w2)
        wide = h.cpu().double()
        inputs = wide / (wide.pow(2).mean(-1, keepdim=True) + 1e-5).sqrt() * norm_weight.cpu().double()
        exact = inputs @ w2.cpu().double().T
        deviation = 2**-8 / 3**0.5 * (inputs.pow(2) @ w2.cpu().double().pow(2).T).sqrt()
        bound = 6 * deviation + 2**-8 * exact.abs() + 1e-6
        ratio = ((out.cpu().double() - exact).abs() / bound).max()
        assert float(ratio) <= 1.0, f"error / bound = {float(ratio):.2f}"
        assert torch.equal(ops.linear_prepared(weighted, squares, 1e-5, w2, gated=True), ops.silu_mul(out))
        # again into the same tensors, as a recorded step does: nothing is kept between calls
        again = start.clone()
        weighted_again, squares_again = ops.linear_norm_ahead(x, w1, again, norm_weight)
        assert torch.equal(weighted_again, weighted) and torch.equal(squares_again, squares)
    from miniserve_amd.ops import KernelError

    with pytest.raises(KernelError, match="squares"):
        ops.linear_prepared(weighted, squares[:, : m - 1] if m > 1 else squares[:0], 1e-5, w2)
    with ops.forced_product("library"):
        assert not ops.can_prepare_norm(m, w1) and not ops.can_use_prepared_norm(m, w2)


@pytest.mark.parametrize("m", [1, 7, 16])
@pytest.mark.parametrize("n,k", [(5128, 64), (6144, 2048), (5120, 4104)])
def test_product_with_the_norm_as_its_prologue_against_many_rows(ops, m, n, k):
    """From 5120 rows of the matrix on a workgroup takes two blocks of rows.  Against the
    norm and the product in float64 with nothing rounded: the one rounding of a normed
    input to bfloat16 is at most 2^-8 of it (uniform, so 2^-8 / sqrt(3) in the mean), the
    roundings of the k inputs are independent, and the result is rounded once more;
    six standard deviations, and every row bit-equal to the same row alone."""

    residual = rand(m, k, seed=m + n, scale=2.0)
    norm_weight = (1 + 0.1 * rand(k, seed=5)).to(torch.bfloat16)
    weight = rand(n, k, seed=n + k, dtype=torch.bfloat16, scale=0.05)
    wide = residual.cpu().double()
    inputs = wide / (wide.pow(2).mean(-1, keepdim=True) + 1e-5).sqrt() * norm_weight.cpu().double()
    exact = inputs @ weight.cpu().double().T
    deviation = 2**-8 / 3**0.5 * (inputs.pow(2) @ weight.cpu().double().pow(2).T).sqrt()
    bound = 6 * deviation + 2**-8 * exact.abs() + 1e-6
    with ops.forced_product("skinny"):
        fused = ops.linear_normed(residual, norm_weight, 1e-5, weight)
        ratio = ((fused.cpu().double() - exact).abs() / bound).max()
        assert float(ratio) <= 1.0, f"error / bound = {float(ratio):.2f}"
        alone = ops.linear_normed(residual[m // 2 : m // 2 + 1].contiguous(), norm_weight, 1e-5, weight)
        assert torch.equal(alone[0], fused[m // 2])
        if n % 2 == 0:
            gated = ops.linear_normed(residual, norm_weight, 1e-5, weight, gated=True)
            assert torch.equal(gated, ops.silu_mul(fused))       # the same sums, rounded, then the activation
