"""Schedules of the whole engine against the plain implementation: requests that are
preempted and run again while decode steps are replayed from recordings and the next
step is planned ahead; recorded steps of an engine whose context limit is the model's
(tens of thousands of tokens) while the requests are short.

The engine chooses its own tokens here; what is compared is the logits it chose them
from, at every sampled position, with the plain implementation's logits for the same
tokens (the reference checks a run the same way, with given tokens:
miniserve/benchmark/compare_hf.py:306-381).
"""

from __future__ import annotations

import plain_qwen3 as plain
import pytest
import torch
from helpers import make_model_folder, random_tokens, read_config, read_weights, tiny_c

pytestmark = pytest.mark.gpu


def rounded(weights, dtype):
    if dtype == "bfloat16":
        return {name: tensor.to(torch.bfloat16).float() for name, tensor in weights.items()}
    return weights


def tolerance_for(dtype, weights, config, tokens, exact):
    """float32: a few hundred roundings; bfloat16: three times what the reference's own
    rounding does to these logits (the plain implementation with every intermediate
    rounded where the reference rounds, against itself in float64)."""

    if dtype == "float32":
        return 2e-5 * max(1.0, float(exact.abs().max()))
    reduced = plain.forward_logits(weights, config, tokens, rd=torch.bfloat16).float()
    return 3 * float((reduced - exact).abs().max())


def keeping_sampler():
    from miniserve_amd.sampling import Sampler

    class KeepingSampler(Sampler):
        """The engine's sampler, keeping the logits each token was chosen from."""

        def __init__(self) -> None:
            super().__init__()
            self.kept: dict[str, list[torch.Tensor]] = {}

        def launch(self, logits, requests):
            rows = logits.clone()          # on the device, in stream order: the step is not waited for
            for row, (request_id, _) in enumerate(requests):
                self.kept.setdefault(request_id, []).append(rows[row])
            return super().launch(logits, requests)

    return KeepingSampler()


def test_preempted_requests_under_recorded_steps_planned_ahead_match_the_plain_implementation(model_folders):
    """Ten requests on a pool that holds three or four of them: requests are preempted and
    run again as one prompt, decode steps come from recordings, every next step is
    planned while the GPU runs, in bfloat16 where the matrix-core kernels serve (heads
    of 64, pages of 32).  Every token of every request was chosen from logits that are
    the plain implementation's for the tokens before it."""

    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import Engine, ModelRunner, SamplingParams

    folder, block = model_folders["c"]
    config, weights = read_config(folder), rounded(read_weights(folder), "bfloat16")
    lengths = (20, 95, 40, 64, 33, 120, 18, 77, 50, 101)
    prompts = [random_tokens(n, config["vocab_size"], 600 + n) for n in lengths]
    new_tokens = 48
    runner = ModelRunner.from_folder(folder, EngineConfig(
        dtype="bfloat16", kv_block_size=block, num_kv_blocks=13, max_num_seqs=5, enable_chunked_prefill=True,
        prefill_chunk_size=48, max_num_batched_tokens=64))
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
    print(f"{steps} steps, {preempted} preemptions, {runner.graph_steps} recorded steps, "
          f"{runner.prepared_steps} planned ahead ({runner.prepared_mixed_steps} with prompt portions)", flush=True)
    assert preempted >= 3 and engine.counters["preemptions"] == preempted
    assert runner.graph_steps > 0 and runner.prepared_steps > 0 and runner.prepared_mixed_steps > 0
    assert runner.chained_steps > 0                 # steps launched before the host had read the tokens they ran
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (13,)
    worst = 0.0
    for index, (prompt, result) in enumerate(zip(prompts, results)):
        assert result.finish_reason == "length" and len(result.token_ids) == new_tokens
        kept = sampler.kept[f"r{index}"]
        assert len(kept) == new_tokens              # one choice a token, none made twice
        tokens = list(prompt) + list(result.token_ids[:-1])
        exact = plain.forward_logits(weights, config, tokens).float()[len(prompt) - 1 :]
        tolerance = tolerance_for("bfloat16", weights, config, tokens, plain.forward_logits(weights, config, tokens).float())
        got = torch.stack(kept).float().cpu()
        assert bool(torch.isfinite(got).all())
        error = (got - exact).abs().max(dim=-1).values
        worst = max(worst, float(error.max()))
        assert float(error.max()) <= tolerance, (
            f"request r{index} ({result.num_preemptions} preemptions): token {int((error > tolerance).nonzero()[0])} "
            f"was chosen from logits off by {float(error.max()):.3e} > {tolerance:.3e}")
        # and the token is the largest of those logits
        assert [int(row.argmax()) for row in got] == list(result.token_ids)
    print(f"worst difference from the plain implementation {worst:.2e}", flush=True)


def test_a_stop_token_throws_the_step_that_was_launched_ahead_away(model_folders):
    """Decode steps are launched before the host has read the tokens they run.  When one
    of those tokens turns out to be a request's stop token, the step that already runs is
    thrown away and the others' tokens come out as if nothing had been launched: every
    request's tokens are those of a run without stop tokens, cut behind the stop token."""

    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import Engine, ModelRunner, SamplingParams

    folder, block = model_folders["c"]
    config = read_config(folder)
    prompts = [random_tokens(n, config["vocab_size"], 950 + n) for n in (12, 30, 21, 44)]

    def run(stops):
        runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", kv_block_size=block, num_kv_blocks=24, max_num_seqs=4))
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
    # the first token that each of two requests produces for the first time at its 9th and 23rd place or later
    stops, cut = [()] * 4, [40] * 4
    for index, place in ((1, 8), (3, 22)):
        tokens = free[index].token_ids
        at = next(p for p in range(place, 40) if tokens[p] not in tokens[:p])
        stops[index], cut[index] = (tokens[at],), at + 1
    assert cut[1] < 40 and cut[3] < 40
    stopped, runner = run(stops)
    for index in range(4):
        assert stopped[index].token_ids == free[index].token_ids[: cut[index]]
        assert stopped[index].finish_reason == ("stop" if cut[index] < 40 else "length")
    assert runner.voided_chained_steps == 2 and runner.chained_steps > 20


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_steps_under_the_models_own_context_limit(dtype, tmp_path):
    """An engine that admits requests of up to 40,960 tokens serves requests of 20 to 330:
    their decode steps are recordings made for 256 and 512 tokens, not for the limit
    (whose launches would cut every row's keys into dozens of empty parts), a request
    that grows past 256 moves to the next recording, and the logits are the plain
    implementation's."""

    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner, StepEntry

    data = tiny_c()
    data["max_position_embeddings"] = 40960
    folder = make_model_folder(tmp_path / "long_limit", data, seed=5)
    config, weights = read_config(folder), rounded(read_weights(folder), dtype)
    runner = ModelRunner.from_folder(folder, EngineConfig(dtype=dtype, kv_block_size=32, num_kv_blocks=40, max_num_seqs=4))
    assert runner.max_model_len == 40960 and runner.engine_config.decode_graphs
    for pool in (*runner.cache.key_pools, *runner.cache.value_pools):
        pool.fill_(float("nan"))
    decoded = 45
    requests = {f"r{i}": random_tokens(n + decoded, config["vocab_size"], 30 + i) for i, n in enumerate((20, 77, 150, 240))}
    exact = {rid: plain.forward_logits(weights, config, tokens).float() for rid, tokens in requests.items()}
    probe = "r2"
    tolerance = tolerance_for(dtype, weights, config, requests[probe], exact[probe])
    position = {}
    for rid, tokens in requests.items():
        runner.admit(rid)
        head = len(tokens) - decoded
        logits = runner.step([StepEntry(rid, tuple(tokens[:head]), (head - 1,))]).cpu()
        assert float((logits[0] - exact[rid][head - 1]).abs().max()) <= tolerance
        position[rid] = head
    worst = 0.0
    for _ in range(decoded):
        names = sorted(requests, key=lambda rid: -position[rid])
        logits = runner.step([StepEntry(rid, (requests[rid][position[rid]],), (0,)) for rid in names]).cpu()
        for row, rid in enumerate(names):
            error = float((logits[row] - exact[rid][position[rid]]).abs().max())
            worst = max(worst, error)
            assert error <= tolerance, f"{rid} at position {position[rid]}: {error:.3e} > {tolerance:.3e}"
            position[rid] += 1
    print(f"{dtype}: worst difference {worst:.2e} (allowed {tolerance:.2e})", flush=True)
    assert runner.graph_steps == decoded
    assert sorted(runner._decode_graphs) == [(4, 256), (4, 512)]       # 240 + 45 tokens pass 256 on the way
    widths = {key: graph.ctx.groups[0].block_table.shape[1] for key, graph in runner._decode_graphs.items()}
    assert widths == {(4, 256): 8, (4, 512): 16}
