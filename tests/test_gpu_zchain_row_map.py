"""Steps launched ahead through a map of rows, on the GPU: the step behind one in which
a request ends by length takes the tokens of the requests that go on from the sampling
kernel's output by their rows there.  (Collected late on purpose: this path was added
after the other GPU tests last ran.)"""

from __future__ import annotations

import plain_qwen3 as plain
import pytest
import torch
from helpers import random_tokens, read_config, read_weights
from test_gpu_schedules import keeping_sampler, rounded, tolerance_for

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_requests_that_end_by_length_do_not_break_the_chain(dtype, model_folders):
    """Eight requests on a roomy pool, three of which end early by length (eight, seven,
    six and five rows share the recording of eight).  Every token was chosen from the
    plain implementation's logits for the tokens before it."""

    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import Engine, ModelRunner, SamplingParams

    folder, block = model_folders["c"]
    config, weights = read_config(folder), rounded(read_weights(folder), dtype)
    prompts = [random_tokens(n, config["vocab_size"], 800 + n) for n in (12, 30, 21, 44, 9, 17, 26, 35)]
    lengths = (6, 20, 9, 20, 13, 20, 20, 20)
    runner = ModelRunner.from_folder(folder, EngineConfig(dtype=dtype, kv_block_size=block, num_kv_blocks=40, max_num_seqs=8))
    for pool in (*runner.cache.key_pools, *runner.cache.value_pools):
        pool.fill_(float("nan"))
    sampler = keeping_sampler()
    engine = Engine(runner, sampler=sampler)
    for index, prompt in enumerate(prompts):
        engine.add_request(f"r{index}", prompt, SamplingParams(max_new_tokens=lengths[index]), arrival_ns=index)
    while engine.has_unfinished():
        engine.step()
        runner.cache.assert_invariants()
    assert sorted(runner._decode_graphs) == [(8, 256)]
    assert runner.graph_steps == 19 and runner.chained_steps == 18 and runner.mapped_chained_steps == 2
    assert runner.voided_chained_steps == 0
    for index, prompt in enumerate(prompts):
        result = engine.pop_result(f"r{index}")
        assert result.finish_reason == "length" and len(result.token_ids) == lengths[index]
        tokens = list(prompt) + list(result.token_ids[:-1])
        whole = plain.forward_logits(weights, config, tokens).float()
        tolerance = tolerance_for(dtype, weights, config, tokens, whole)
        got = torch.stack(sampler.kept[f"r{index}"]).float().cpu()
        error = float((got - whole[len(prompt) - 1 :]).abs().max())
        assert error <= tolerance, f"request r{index}: logits off by {error:.3e} > {tolerance:.3e}"
        assert [int(row.argmax()) for row in got] == list(result.token_ids)
    assert runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (40,)
