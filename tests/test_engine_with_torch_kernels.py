"""Everything around the kernels on the CPU: the product's parts, step function, batch
builder, cache manager, scheduler and engine run with torch stand-ins in the kernels'
places (``torch_kernels.py``), in 32-bit, against the plain implementation.  What the
GPU tests show for the kernels, these show for the rest where no GPU is visible: a
position's logits do not depend on how tokens are cut into steps, on what else is in
the batch or on which pages hold them (pools start as NaN, pages are used again)."""

from __future__ import annotations

import io

import plain_qwen3 as plain
import pytest
import replay_shapes as shapes
import torch
import torch_kernels
from helpers import random_tokens, read_config, read_weights

TOLERANCE = 2e-5
LENGTHS = {"a": (45, 70, 33, 18, 64), "b": (41, 64, 57, 9), "c": (70, 37, 66, 40)}


def make_runner(folder, block_size, num_blocks, dtype="float32", **options):
    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner

    config = EngineConfig(dtype=dtype, kv_block_size=block_size, num_kv_blocks=num_blocks, max_num_seqs=8,
                          enable_chunked_prefill=True, decode_graphs=False, **options)
    runner = ModelRunner.from_folder(folder, config, device="cpu")
    for pool in (*runner.cache.key_pools, *runner.cache.value_pools):
        pool.fill_(float("nan"))
    return runner


@pytest.mark.parametrize("fused", [None, "prologue", "prepared"])
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_replay_shapes_on_the_cpu(name, fused, model_folders, monkeypatch, tmp_path):
    """``fused``: the parts hand the norms to the products around them (as the prologue of
    the product behind, or prepared by the product before) or take them plainly; the
    counts show that the way asked for is the way taken."""

    from miniserve_amd import ops
    from miniserve_amd.engine.replay import replay

    torch_kernels.install(monkeypatch, fused=fused)
    taken = {"linear_normed": 0, "linear_norm_ahead": 0, "linear_prepared": 0, "rmsnorm": 0}
    for kernel in taken:
        def counted(*args, _kernel=kernel, _function=getattr(ops, kernel), **kwargs):
            taken[_kernel] += 1
            return _function(*args, **kwargs)
        monkeypatch.setattr(ops, kernel, counted)
    folder, block_size = model_folders[name]
    config, weights = read_config(folder), read_weights(folder)
    requests = {f"r{i}": random_tokens(n, config["vocab_size"], 50 + i) for i, n in enumerate(LENGTHS[name])}
    exact = {rid: plain.forward_logits(weights, config, tokens).float() for rid, tokens in requests.items()}
    for shape, steps in (
        ("whole", shapes.whole(requests)),
        ("tail", shapes.prefill_then_decode(requests)),
        ("portions", shapes.portions(requests)),
        ("mixed", shapes.mixed(requests, seed=3)),
    ):
        pages = -(-shapes.max_live_tokens(steps) // block_size)
        runner = make_runner(folder, block_size, pages)
        out = tmp_path / shape
        assert replay(runner, shapes.to_lines(steps), out, report=io.StringIO()) == len(steps)
        got = shapes.collect(steps, out, config["vocab_size"])
        assert len(got) == sum(len(tokens) for tokens in requests.values())
        for (rid, position), row in got.items():
            error = float((row - exact[rid][position]).abs().max())
            assert error <= TOLERANCE, f"{shape}: {rid} at {position}: {error:.3e}"
        assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (pages,) * len(runner.cache.num_blocks)
        runner.cache.assert_invariants()
    layers = config["num_hidden_layers"]
    if fused is None:
        assert taken["linear_normed"] == taken["linear_norm_ahead"] == taken["linear_prepared"] == 0 and taken["rmsnorm"] > 0
    elif fused == "prologue":
        assert taken["linear_normed"] > 0 and taken["linear_prepared"] == 0
    else:
        # every norm but the first of a step (behind the embedding) and the final one is prepared
        assert taken["linear_norm_ahead"] > 0 and taken["linear_prepared"] == taken["linear_norm_ahead"]
        assert taken["linear_normed"] == 0 and taken["linear_prepared"] % (2 * layers - 1) == 0


@pytest.mark.parametrize("name", ["a", "c"])
def test_bfloat16_replay_on_the_cpu(name, model_folders, monkeypatch, tmp_path):
    """The same in bfloat16 (weights, cache and the values between kernels; the residual
    stream stays 32-bit): within three times what the reference's own rounding does to
    these logits, as the GPU tests hold the kernels."""

    from miniserve_amd.engine.replay import replay

    torch_kernels.install(monkeypatch)
    folder, block_size = model_folders[name]
    config = read_config(folder)
    weights = {key: tensor.to(torch.bfloat16).float() for key, tensor in read_weights(folder).items()}
    requests = {f"r{i}": random_tokens(n, config["vocab_size"], 50 + i) for i, n in enumerate(LENGTHS[name][:3])}
    exact = {rid: plain.forward_logits(weights, config, tokens).float() for rid, tokens in requests.items()}
    yardstick = max(float((plain.forward_logits(weights, config, tokens, rd=torch.bfloat16).float() - exact[rid]).abs().max())
                    for rid, tokens in requests.items())
    for shape, steps in (("portions", shapes.portions(requests)), ("mixed", shapes.mixed(requests, seed=3))):
        pages = -(-shapes.max_live_tokens(steps) // block_size)
        runner = make_runner(folder, block_size, pages, dtype="bfloat16")
        assert runner.cache.key_pools[0].dtype == torch.bfloat16
        out = tmp_path / shape
        replay(runner, shapes.to_lines(steps), out, report=io.StringIO())
        got = shapes.collect(steps, out, config["vocab_size"])
        worst = max(float((row - exact[rid][position]).abs().max()) for (rid, position), row in got.items())
        assert worst <= 3 * yardstick, f"{shape}: {worst:.3e} > 3 x {yardstick:.3e}"
        runner.cache.assert_invariants()


def test_the_engine_generates_the_plain_implementations_tokens_on_a_tight_pool(model_folders, monkeypatch):
    """Six requests on a pool that holds two or three of them, prompts in portions:
    requests are preempted and run again, and every request's greedy tokens are those
    the plain implementation generates from its prompt."""

    from miniserve_amd.engine import Engine, SamplingParams

    torch_kernels.install(monkeypatch)
    folder, block_size = model_folders["a"]
    config, weights = read_config(folder), read_weights(folder)
    prompts = [random_tokens(n, config["vocab_size"], 700 + n) for n in (20, 45, 12, 33, 28, 40)]
    new_tokens = 12
    runner = make_runner(folder, block_size, 9, prefill_chunk_size=16, max_num_batched_tokens=32)
    engine = Engine(runner)
    for index, prompt in enumerate(prompts):
        engine.add_request(f"r{index}", prompt, SamplingParams(max_new_tokens=new_tokens), arrival_ns=index)
    steps = 0
    while engine.has_unfinished():
        engine.step()
        runner.cache.assert_invariants()
        steps += 1
        assert steps < 1000
    results = [engine.pop_result(f"r{index}") for index in range(len(prompts))]
    assert sum(result.num_preemptions for result in results) >= 1
    assert runner.prepared_mixed_steps > 0          # steps with prompt portions were planned, and their tensors built, a step ahead
    for prompt, result in zip(prompts, results):
        tokens = list(prompt) + list(result.token_ids)
        logits = plain.forward_logits(weights, config, tokens[:-1]).float()[len(prompt) - 1 :]
        best = logits.argmax(-1).tolist()
        for place, (token, wanted) in enumerate(zip(result.token_ids, best)):
            # the engine's token is the plain implementation's, or lies within rounding of it
            assert token == wanted or float(logits[place, wanted] - logits[place, token]) <= 2 * TOLERANCE
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (9,)


def test_sampled_generation_through_the_entry_point(model_folders, monkeypatch):
    """Temperature, top-k and top-p with a seed a request, through ``LLM.generate``: every
    token is the plain sampler's for the plain implementation's logits and the request's
    own stream of uniform numbers; a pool so tight that requests are preempted and run
    again changes no token (a stream advances only with tokens that are kept)."""

    import plain_sampling

    from miniserve_amd.engine import SamplingParams
    from miniserve_amd.entrypoint import LLM
    from miniserve_amd.sampling import Sampler

    torch_kernels.install(monkeypatch)
    folder, block_size = model_folders["b"]
    config, weights = read_config(folder), read_weights(folder)
    prompts = [random_tokens(n, config["vocab_size"], 900 + n) for n in (14, 31, 22, 9)]
    params = [SamplingParams(max_new_tokens=16, temperature=0.9, top_k=(0, 12, 0, 40)[i], top_p=(1.0, 0.9, 0.7, 1.0)[i], seed=70 + i)
              for i in range(4)]
    options = dict(dtype="float32", kv_block_size=block_size, max_num_seqs=4, decode_graphs=False, device="cpu")
    roomy = LLM(str(folder), num_kv_blocks=40, **options)
    tokens = roomy.generate(prompts, params)
    for index, (prompt, generated) in enumerate(zip(prompts, tokens)):
        logits = plain.forward_logits(weights, config, list(prompt) + generated[:-1]).float()[len(prompt) - 1 :]
        stream = torch.Generator().manual_seed(70 + index)
        for place, token in enumerate(generated):
            uniform = Sampler.draw_uniform(stream)
            p = params[index]
            if plain_sampling.edge_distance(logits[place], p.temperature, p.top_k, p.top_p, uniform) > 1e-4:
                assert token == plain_sampling.sample_row(logits[place], p.temperature, p.top_k, p.top_p, uniform), (index, place)
    tight = LLM(str(folder), num_kv_blocks=-(-(31 + 16) // block_size) + 3, enable_chunked_prefill=True, **options)
    again = tight.generate(prompts, params)
    assert tight.engine.counters["preemptions"] > 0
    for index, (first, second) in enumerate(zip(tokens, again)):
        if first != second:
            # torch's products on the CPU depend on the rows beside a row in the last bit: only a draw on an edge may differ
            place = next(i for i, (a, b) in enumerate(zip(first, second)) if a != b)
            logits = plain.forward_logits(weights, config, list(prompts[index]) + first[:place]).float()[-1]
            stream = torch.Generator().manual_seed(70 + index)
            for _ in range(place + 1):
                uniform = Sampler.draw_uniform(stream)
            p = params[index]
            assert plain_sampling.edge_distance(logits, p.temperature, p.top_k, p.top_p, uniform) <= 1e-4
    assert tight.runner.cache.live_requests() == ()
    tight.runner.cache.assert_invariants()


@pytest.mark.parametrize("seed", range(10))
def test_random_mixed_traces_on_the_cpu(seed, model_folders, monkeypatch, tmp_path):
    """Ten more ways of mixing requests (who joins when, who sits a step out, portions of 2
    to 21 tokens beside single tokens, two to four live at a time), each on a pool that
    only just holds the live requests, alternating the tiny configurations and the way
    the norms are taken: every position's logits are the plain implementation's."""

    from miniserve_amd.engine.replay import replay

    name = "abc"[seed % 3]
    torch_kernels.install(monkeypatch, fused=(None, "prologue", "prepared")[(seed // 3) % 3])
    folder, block_size = model_folders[name]
    config, weights = read_config(folder), read_weights(folder)
    lengths = [torch.randint(5, 90, (), generator=torch.Generator().manual_seed(seed * 31 + i)).item() for i in range(6)]
    requests = {f"r{i}": random_tokens(n, config["vocab_size"], 200 + 10 * seed + i) for i, n in enumerate(lengths)}
    exact = {rid: plain.forward_logits(weights, config, tokens).float() for rid, tokens in requests.items()}
    steps = shapes.mixed(requests, seed=100 + seed, live_limit=2 + seed % 3, tail=3 + seed)
    pages = -(-shapes.max_live_tokens(steps, block=block_size) // block_size)
    runner = make_runner(folder, block_size, pages)
    replay(runner, shapes.to_lines(steps), tmp_path, report=io.StringIO())
    got = shapes.collect(steps, tmp_path, config["vocab_size"])
    assert len(got) == sum(lengths)
    for (rid, position), row in got.items():
        error = float((row - exact[rid][position]).abs().max())
        assert error <= TOLERANCE, f"seed {seed}: {rid} at {position}: {error:.3e}"
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (pages,)
    runner.cache.assert_invariants()
