"""The runner's recorded decode steps, steps planned ahead and steps launched behind the
sampling, where no GPU is visible: the product's own runner, cache manager, engine and
sampler, with torch stand-ins for the kernels and a recording that is a note of the
forward pass, run again at every replay (``torch_kernels.py``).  What a recording
cannot show here (the stream's order, the device's own copies) stays with the GPU
tests of the same names in ``test_gpu_schedules.py``."""

from __future__ import annotations

import plain_qwen3 as plain
import pytest
import torch
import torch_kernels
from helpers import make_model_folder, random_tokens, read_config, read_weights, tiny_c

TOLERANCE = 2e-5


@pytest.fixture
def recordings(monkeypatch):
    torch_kernels.install(monkeypatch, recordings=True)


def keeping_sampler():
    from miniserve_amd.sampling import Sampler

    class KeepingSampler(Sampler):
        """The engine's sampler, keeping the logits each token was chosen from."""

        def __init__(self) -> None:
            super().__init__()
            self.kept: dict[str, list[torch.Tensor]] = {}

        def launch(self, logits, requests):
            rows = logits.clone()
            for row, (request_id, _) in enumerate(requests):
                self.kept.setdefault(request_id, []).append(rows[row])
            return super().launch(logits, requests)

    return KeepingSampler()


def test_preempted_requests_under_recorded_steps_planned_and_launched_ahead(model_folders, recordings):
    """Ten requests on a pool for three or four: preempted and run again as one prompt,
    decode steps from recordings, every next step planned while "the GPU runs", steady
    decoding launched ahead of the host's read of its tokens.  Every token of every
    request was chosen from the plain implementation's logits for the tokens before it."""

    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import Engine, ModelRunner, SamplingParams

    folder, block = model_folders["c"]
    config, weights = read_config(folder), read_weights(folder)
    lengths = (20, 95, 40, 64, 33, 120, 18, 77, 50, 101)
    prompts = [random_tokens(n, config["vocab_size"], 600 + n) for n in lengths]
    new_tokens = 24
    runner = ModelRunner.from_folder(folder, EngineConfig(
        dtype="float32", kv_block_size=block, num_kv_blocks=13, max_num_seqs=5, enable_chunked_prefill=True,
        prefill_chunk_size=48, max_num_batched_tokens=64), device="cpu")
    assert runner.engine_config.decode_graphs
    for pool in (*runner.cache.key_pools, *runner.cache.value_pools):
        pool.fill_(float("nan"))
    sampler = keeping_sampler()
    engine = Engine(runner, sampler=sampler)
    for index, prompt in enumerate(prompts):
        engine.add_request(f"r{index}", prompt, SamplingParams(max_new_tokens=new_tokens), arrival_ns=index)
    steps = 0
    while engine.has_unfinished():
        engine.step()
        runner.cache.assert_invariants()
        steps += 1
        assert steps < 3000
    results = [engine.pop_result(f"r{index}") for index in range(len(prompts))]
    preempted = sum(result.num_preemptions for result in results)
    assert preempted >= 3 and engine.counters["preemptions"] == preempted
    assert runner.graph_steps > 0 and runner.prepared_steps > 0 and runner.prepared_mixed_steps > 0 and runner.chained_steps > 0
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (13,)
    for index, (prompt, result) in enumerate(zip(prompts, results)):
        assert result.finish_reason == "length" and len(result.token_ids) == new_tokens
        kept = sampler.kept[f"r{index}"]
        assert len(kept) == new_tokens
        tokens = list(prompt) + list(result.token_ids[:-1])
        exact = plain.forward_logits(weights, config, tokens).float()[len(prompt) - 1 :]
        got = torch.stack(kept)
        assert bool(torch.isfinite(got).all())
        error = (got - exact).abs().max(dim=-1).values
        assert float(error.max()) <= TOLERANCE, f"request r{index}: token {int(error.argmax())} off by {float(error.max()):.3e}"
        assert [int(row.argmax()) for row in got] == list(result.token_ids)


def test_requests_that_end_by_length_do_not_break_the_chain(model_folders, recordings):
    """Eight requests on a roomy pool, three of which end early by length: the step behind
    one in which a request ends has fewer rows than that one sampled, and is still
    launched ahead, its tokens taken through a map of rows (eight, seven, six and five
    rows share the recording of eight).  Every token was chosen from the plain
    implementation's logits for the tokens before it."""

    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import Engine, ModelRunner, SamplingParams

    folder, block = model_folders["c"]
    config, weights = read_config(folder), read_weights(folder)
    prompts = [random_tokens(n, config["vocab_size"], 800 + n) for n in (12, 30, 21, 44, 9, 17, 26, 35)]
    lengths = (6, 20, 9, 20, 13, 20, 20, 20)
    runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", kv_block_size=block, num_kv_blocks=40, max_num_seqs=8),
                                     device="cpu")
    sampler = keeping_sampler()
    engine = Engine(runner, sampler=sampler)
    for index, prompt in enumerate(prompts):
        engine.add_request(f"r{index}", prompt, SamplingParams(max_new_tokens=lengths[index]), arrival_ns=index)
    while engine.has_unfinished():
        engine.step()
        runner.cache.assert_invariants()
    # 19 decode steps behind the prompts' step; the first makes the recording, the others are launched ahead,
    # two of them (behind the steps in which r0 and r2 end; r4 held the last row when it ended) through a map of rows
    assert sorted(runner._decode_graphs) == [(8, 256)]
    assert runner.graph_steps == 19 and runner.chained_steps == 18 and runner.mapped_chained_steps == 2
    assert runner.voided_chained_steps == 0
    for index, prompt in enumerate(prompts):
        result = engine.pop_result(f"r{index}")
        assert result.finish_reason == "length" and len(result.token_ids) == lengths[index]
        tokens = list(prompt) + list(result.token_ids[:-1])
        exact = plain.forward_logits(weights, config, tokens).float()[len(prompt) - 1 :]
        got = torch.stack(sampler.kept[f"r{index}"])
        assert float((got - exact).abs().max()) <= TOLERANCE
        assert [int(row.argmax()) for row in got] == list(result.token_ids)
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (40,)


def test_a_stop_token_throws_the_step_that_was_launched_ahead_away(model_folders, recordings):
    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import Engine, ModelRunner, SamplingParams

    folder, block = model_folders["c"]
    config = read_config(folder)
    prompts = [random_tokens(n, config["vocab_size"], 950 + n) for n in (12, 30, 21, 44)]

    def run(stops):
        runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", kv_block_size=block, num_kv_blocks=24, max_num_seqs=4),
                                         device="cpu")
        engine = Engine(runner)
        for index, prompt in enumerate(prompts):
            engine.add_request(f"r{index}", prompt, SamplingParams(max_new_tokens=40, stop_token_ids=stops[index]), arrival_ns=index)
        while engine.has_unfinished():
            engine.step()
            runner.cache.assert_invariants()
        assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (24,)
        return [engine.pop_result(f"r{index}") for index in range(len(prompts))], runner

    free, runner = run([()] * 4)
    assert runner.chained_steps > 20 and runner.voided_chained_steps == 0
    stops, cut = [()] * 4, [40] * 4
    for index, place in ((1, 8), (3, 22)):
        tokens = free[index].token_ids
        at = next(p for p in range(place, 40) if tokens[p] not in tokens[:p])
        stops[index], cut[index] = (tokens[at],), at + 1
    stopped, runner = run(stops)
    for index in range(4):
        assert stopped[index].token_ids == free[index].token_ids[: cut[index]]
        assert stopped[index].finish_reason == ("stop" if cut[index] < 40 else "length")
    assert runner.voided_chained_steps == 2 and runner.chained_steps > 20


def test_recorded_steps_under_the_models_own_context_limit(recordings, tmp_path):
    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner, StepEntry

    data = tiny_c()
    data["max_position_embeddings"] = 40960
    folder = make_model_folder(tmp_path / "long_limit", data, seed=5)
    config, weights = read_config(folder), read_weights(folder)
    runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", kv_block_size=32, num_kv_blocks=40, max_num_seqs=4), device="cpu")
    assert runner.max_model_len == 40960 and runner.engine_config.decode_graphs
    for pool in (*runner.cache.key_pools, *runner.cache.value_pools):
        pool.fill_(float("nan"))
    decoded = 45
    requests = {f"r{i}": random_tokens(n + decoded, config["vocab_size"], 30 + i) for i, n in enumerate((20, 77, 150, 240))}
    exact = {rid: plain.forward_logits(weights, config, tokens).float() for rid, tokens in requests.items()}
    position = {}
    for rid, tokens in requests.items():
        runner.admit(rid)
        head = len(tokens) - decoded
        logits = runner.step([StepEntry(rid, tuple(tokens[:head]), (head - 1,))])
        assert float((logits[0] - exact[rid][head - 1]).abs().max()) <= TOLERANCE
        position[rid] = head
    for _ in range(decoded):
        names = sorted(requests, key=lambda rid: -position[rid])
        logits = runner.step([StepEntry(rid, (requests[rid][position[rid]],), (0,)) for rid in names]).clone()
        for row, rid in enumerate(names):
            error = float((logits[row] - exact[rid][position[rid]]).abs().max())
            assert error <= TOLERANCE, f"{rid} at position {position[rid]}: {error:.3e}"
            position[rid] += 1
    assert runner.graph_steps == decoded
    assert sorted(runner._decode_graphs) == [(4, 256), (4, 512)]
    widths = {key: graph.ctx.groups[0].block_table.shape[1] for key, graph in runner._decode_graphs.items()}
    assert widths == {(4, 256): 8, (4, 512): 16}


# ---- per-request state and a mixer's own planes inside recorded steps: the toy architectures -----------------

import test_gpu_toy_cache as latent_tests  # noqa: E402
import test_gpu_toy_parts as toy_tests  # noqa: E402

toy = toy_tests.toy
latent_toy = latent_tests.toy


@pytest.fixture
def gpu_names_mean_the_cpu(monkeypatch, recordings):
    """The GPU tests name their device; here the name is taken to mean the CPU."""

    from miniserve_amd.engine import ModelRunner

    from_folder = ModelRunner.from_folder.__func__
    monkeypatch.setattr(ModelRunner, "from_folder", classmethod(
        lambda cls, folder, config, device="cpu": from_folder(cls, folder, config, device="cpu")))


def test_state_in_recorded_steps(toy, gpu_names_mean_the_cpu):  # noqa: F811
    toy_tests.test_state_in_recorded_steps(toy)


def test_an_aborted_step_puts_the_state_back_also_in_recorded_steps(toy, gpu_names_mean_the_cpu):  # noqa: F811
    toy_tests.test_an_aborted_step_puts_the_state_back(toy)


def test_a_chained_step_that_is_thrown_away_puts_the_state_back(toy, gpu_names_mean_the_cpu):  # noqa: F811
    toy_tests.test_a_chained_step_that_is_thrown_away_puts_the_state_back(toy)


def test_planes_of_a_mixers_own_and_its_tables_in_recorded_steps(latent_toy, gpu_names_mean_the_cpu):  # noqa: F811
    latent_tests.test_the_toy_model_steps_like_its_plain_form(latent_toy, True)
