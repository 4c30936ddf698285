"""The toy architecture of ``test_gpu_toy_parts.py`` (a mixer with state of its own, a
feed-forward with routing, another position encoding, another norm, another
arrangement of a layer, a window group with pages of its own size, a layer named twice
and one that reads another call's cache), registered, built and stepped where no GPU
is visible: with torch stand-ins in the kernels' places (``torch_kernels.py``), the
framework's own files unchanged.  The recorded-step variants stay with the GPU tests."""

from __future__ import annotations

import io

import pytest
import replay_shapes as shapes
import test_gpu_toy_parts as toy_tests
import torch
import torch_kernels
from helpers import random_tokens, read_config, read_weights
from test_gpu_toy_parts import toy  # noqa: F401  (the fixture: defines, registers and writes the toy model)


@pytest.fixture
def on_the_cpu(monkeypatch):
    torch_kernels.install(monkeypatch)


def cpu_runner(folder, **options):
    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner

    return ModelRunner.from_folder(folder, EngineConfig(dtype="float32", decode_graphs=False, **options), device="cpu")


def test_the_toy_model_is_built_from_its_folder(toy):  # noqa: F811
    toy_tests.test_the_toy_model_is_built_from_its_folder(toy)          # configuration, registry, cache layout: no kernel runs


@pytest.mark.parametrize("shape", ["whole", "portions", "mixed"])
def test_the_toy_model_steps_like_its_plain_form(toy, shape, on_the_cpu, tmp_path):  # noqa: F811
    from miniserve_amd.engine.replay import replay

    config, weights = read_config(toy), read_weights(toy)
    requests = {f"r{i}": random_tokens(n, config["vocab_size"], 60 + i) for i, n in enumerate((37, 52, 19, 44, 30, 26))}
    steps = getattr(shapes, shape)(requests, **({"seed": 2} if shape == "mixed" else {}))
    pages_full = -(-shapes.max_live_tokens(steps) // 16)
    window_pages = 4 * 2 * (toy_tests.WINDOW_PAGE // 16)
    runner = cpu_runner(toy, kv_block_size=16, num_kv_blocks=max(pages_full, window_pages), max_num_seqs=4, enable_chunked_prefill=True)
    for pool in (*runner.cache.key_pools, *runner.cache.value_pools):
        pool.fill_(float("nan"))
    replay(runner, shapes.to_lines(steps), tmp_path, report=io.StringIO())
    got = shapes.collect(steps, tmp_path, config["vocab_size"])
    assert len(got) == sum(len(t) for t in requests.values())
    for rid, tokens in requests.items():
        expected = toy_tests.toy_logits(weights, config, tokens).float()
        for position in range(len(tokens)):
            error = float((got[(rid, position)] - expected[position]).abs().max())
            assert error <= 2e-5, f"{shape}: {rid} position {position}: {error:.3e}"
    assert runner.cache.live_requests() == ()
    runner.cache.assert_invariants()


def test_a_window_group_holds_few_pages_for_a_long_request(toy, on_the_cpu):  # noqa: F811
    from miniserve_amd.engine import StepEntry

    config = read_config(toy)
    runner = cpu_runner(toy, kv_block_size=4, num_kv_blocks=40, max_num_seqs=2, enable_chunked_prefill=True)
    window_pool = 40 * 4 // toy_tests.WINDOW_PAGE
    assert runner.cache.num_blocks == (40, window_pool) and runner.cache.block_sizes == (4, toy_tests.WINDOW_PAGE)
    tokens = random_tokens(120, config["vocab_size"], 1)
    runner.admit("long")
    position = 0
    for size in (9, 3, 1, 1, 20, 1, 1, 1, 30, 2, 1, 50):
        runner.step([StepEntry("long", tuple(tokens[position : position + size]), ())])
        position += size
        free_full, free_window = runner.cache.capacity().free_blocks
        assert free_full == 40 - -(-position // 4)
        assert window_pool - free_window <= -(-toy_tests.WINDOW // toy_tests.WINDOW_PAGE) + 1
    runner.release("long")
    assert runner.cache.capacity().free_blocks == (40, window_pool)


def test_an_aborted_step_puts_the_state_back(toy, on_the_cpu):  # noqa: F811
    from miniserve_amd.engine import StepEntry

    config, weights = read_config(toy), read_weights(toy)
    tokens = random_tokens(40, config["vocab_size"], 17)
    expected = toy_tests.toy_logits(weights, config, tokens).float()
    runner = cpu_runner(toy, kv_block_size=16, num_kv_blocks=24, max_num_seqs=4, enable_chunked_prefill=True)
    runner.admit("r")
    runner.step([StepEntry("r", tuple(tokens[:12]), ())])
    states_before = [tensor.clone() for tensor in runner.cache.state_tensors]
    head_forward = runner.model.head.forward

    def failing(x):
        raise RuntimeError("the head fails")

    runner.model.head.forward = failing
    for entry in (StepEntry("r", tuple(tokens[12:20]), (7,)), StepEntry("r", (tokens[12],), (0,))):
        with pytest.raises(RuntimeError, match="the head fails"):
            runner.step([entry])
        assert runner.cache.committed_tokens("r") == 12
        for kept, tensor in zip(states_before, runner.cache.state_tensors):
            assert torch.equal(kept, tensor)
    runner.model.head.forward = head_forward
    logits = runner.step([StepEntry("r", tuple(tokens[12:20]), (0, 7))])
    assert float((logits - expected[[12, 19]]).abs().max()) <= 2e-5
    for place in range(20, 24):
        logits = runner.step([StepEntry("r", (tokens[place],), (0,))])
        assert float((logits[0] - expected[place]).abs().max()) <= 2e-5
    runner.release("r")
    runner.cache.assert_invariants()


def test_a_preempted_request_builds_its_state_again(toy, on_the_cpu):  # noqa: F811
    from miniserve_amd.engine import SamplingParams
    from miniserve_amd.entrypoint import LLM

    config, weights = read_config(toy), read_weights(toy)
    prompts = [random_tokens(n, config["vocab_size"], 500 + n) for n in (30, 41, 18, 25)]
    params = SamplingParams(max_new_tokens=24)
    options = dict(dtype="float32", kv_block_size=16, max_num_seqs=4, decode_graphs=False, device="cpu")
    roomy = LLM(str(toy), num_kv_blocks=32, **options)
    expected = roomy.generate(prompts, params)
    for prompt, tokens in zip(prompts[:2], expected[:2]):       # the roomy engine itself against the plain form
        sequence = list(prompt)
        for token in tokens[:6]:
            top = torch.topk(toy_tests.toy_logits(weights, config, sequence)[-1], 2)
            assert int(top.indices[0]) == token or float(top.values[0] - top.values[1]) < 1e-4
            sequence.append(token)
    tight = LLM(str(toy), num_kv_blocks=9, enable_chunked_prefill=True, **options)
    got = tight.generate(prompts, params)
    assert tight.engine.counters["preemptions"] > 0
    # (torch's products on the CPU depend on the rows beside a row in the last bit: a token may differ only at a near tie)
    for prompt, tokens, wanted in zip(prompts, got, expected):
        if tokens != wanted:
            place = next(i for i, (a, b) in enumerate(zip(tokens, wanted)) if a != b)
            row = toy_tests.toy_logits(weights, config, list(prompt) + wanted[:place])[-1]
            assert abs(float(row[tokens[place]] - row[wanted[place]])) < 1e-4
    tight.runner.cache.assert_invariants()


# ---- the toy of test_gpu_toy_cache.py: planes of a mixer's own, pages and a state row at once, an embedding
# ---- that reads the step's context, tables that a part asks for ------------------------------------------

import test_gpu_toy_cache as latent_tests  # noqa: E402

latent_toy = latent_tests.toy


@pytest.fixture
def gpu_names_mean_the_cpu(monkeypatch, on_the_cpu):
    """The GPU tests name their device; here the name is taken to mean the CPU."""

    from miniserve_amd.cache import CacheManager
    from miniserve_amd.engine import ModelRunner

    from_folder = ModelRunner.from_folder.__func__
    monkeypatch.setattr(ModelRunner, "from_folder", classmethod(
        lambda cls, folder, config, device="cpu": from_folder(cls, folder, config, device="cpu")))
    allocate = CacheManager.allocate_storage
    monkeypatch.setattr(CacheManager, "allocate_storage", lambda self, dtype, device: allocate(self, dtype, "cpu"))


def test_the_latent_cache_is_laid_out_as_the_mixers_say(latent_toy, gpu_names_mean_the_cpu):
    latent_tests.test_the_cache_is_laid_out_as_the_mixers_say(latent_toy)


def test_the_latent_toy_steps_like_its_plain_form(latent_toy, gpu_names_mean_the_cpu):
    latent_tests.test_the_toy_model_steps_like_its_plain_form(latent_toy, False)
