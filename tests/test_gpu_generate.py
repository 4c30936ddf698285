"""Generation through the entry point on the GPU: greedy against the plain
implementation, sampling with seeds, long decoding, too few pages, the command
line, and toy parts and architectures that are registered from outside."""

from __future__ import annotations

import json
import subprocess
import sys

import plain_qwen3 as plain
import plain_sampling
import pytest
import torch
from helpers import ROOT, random_tokens, read_config, read_weights

pytestmark = pytest.mark.gpu

DEVICE = "cuda:0"


def rounded(weights, dtype):
    if dtype == "bfloat16":
        return {k: v.to(torch.bfloat16).float() for k, v in weights.items()}
    return weights


def near_tie(dtype, weights, config, tokens, exact) -> float:
    """How far below the plain implementation's best logit a greedy token's logit may lie:
    twice the error that the engine's logits are allowed (the reference's near-tie rule,
    margin <= 2 * max error: miniserve/benchmark/compare_hf.py:369).  The allowed error
    is the replay tests': in float32 a few hundred roundings, in bfloat16 three times
    what the reference's own rounding does to these very logits."""

    if dtype == "float32":
        return 2 * 2e-5 * max(1.0, float(exact.abs().max()))
    reduced = plain.forward_logits(weights, config, tokens, rd=torch.bfloat16)
    return 2 * 3 * float((reduced - exact).abs().max())


def check_greedy(got, prompt, weights, config, dtype):
    """Every token the engine chose is, for the tokens before it (the engine's own, so a
    near tie cannot hide what follows it), the plain implementation's best token or
    within a near tie of it.  Returns how many leading tokens are the best ones."""

    tokens = list(prompt) + list(got[:-1])
    exact = plain.forward_logits(weights, config, tokens)
    allowed = near_tie(dtype, weights, config, tokens, exact)
    leading, exact_so_far = 0, True
    for index, token in enumerate(got):
        row = exact[len(prompt) - 1 + index]
        gap = float(row.max() - row[token])
        assert gap <= allowed, (
            f"token {index} after a prompt of {len(prompt)}: {token} lies {gap:.3e} below the best logit "
            f"(a near tie is {allowed:.3e})")
        exact_so_far = exact_so_far and gap == 0.0
        leading += int(exact_so_far)
    return leading


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_tiny_a(dtype, model_folders):
    """The first tiny configuration: prompts of 5, 17 and 33 tokens, 8 greedy tokens each."""

    from miniserve_amd.engine import SamplingParams
    from miniserve_amd.entrypoint import LLM

    folder, block = model_folders["a"]
    config, weights = read_config(folder), rounded(read_weights(folder), dtype)
    prompts = [random_tokens(n, config["vocab_size"], 200 + n) for n in (5, 17, 33)]
    llm = LLM(str(folder), dtype=dtype, kv_block_size=block, num_kv_blocks=16, max_num_seqs=4)
    got = llm.generate(prompts, SamplingParams(max_new_tokens=8))
    assert [len(tokens) for tokens in got] == [8, 8, 8]
    agreed = [check_greedy(tokens, prompt, weights, config, dtype) for tokens, prompt in zip(got, prompts)]
    if dtype == "float32":
        assert agreed == [8, 8, 8]
    cache = llm.runner.cache
    assert cache.live_requests() == () and cache.capacity().free_blocks == (16,)


def test_greedy_generation_with_wide_heads_through_recorded_steps(model_folders):
    """Tiny C has heads of 64 and pages of 32: in bfloat16 every matrix-core kernel
    serves it, and its decode steps are replayed as recorded graphs.  Prompts of
    changing length so that batches of 1 to 4 are decoded."""

    from miniserve_amd.engine import SamplingParams
    from miniserve_amd.entrypoint import LLM

    folder, block = model_folders["c"]
    config, weights = read_config(folder), rounded(read_weights(folder), "bfloat16")
    prompts = [random_tokens(n, config["vocab_size"], 400 + n) for n in (3, 40, 65, 131)]
    llm = LLM(str(folder), dtype="bfloat16", kv_block_size=block, num_kv_blocks=24, max_num_seqs=4)
    assert llm.runner.engine_config.decode_graphs
    limits = [SamplingParams(max_new_tokens=n) for n in (40, 9, 33, 20)]
    got = llm.generate(prompts, limits)
    assert [len(tokens) for tokens in got] == [40, 9, 33, 20]
    assert 0 < llm.runner.prepared_steps < llm.runner.graph_steps     # steps planned while the one before ran
    for tokens, prompt in zip(got, prompts):
        check_greedy(tokens, prompt, weights, config, "bfloat16")
    eager = LLM(str(folder), dtype="bfloat16", kv_block_size=block, num_kv_blocks=24, max_num_seqs=4, decode_graphs=False)
    for tokens, prompt in zip(eager.generate(prompts, limits), prompts):     # the same steps, launched one by one
        check_greedy(tokens, prompt, weights, config, "bfloat16")
    assert llm.runner.cache.live_requests() == ()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_chunked_prefill_mixed_with_decode_tiny_b(dtype, model_folders):
    """The second tiny configuration: prompts of 1, 9, 24 and 40 tokens, portions of
    7 mixed with decoding; greedy, then temperature 0.8 from seed 0."""

    from miniserve_amd.engine import SamplingParams
    from miniserve_amd.entrypoint import LLM
    from miniserve_amd.sampling import Sampler

    folder, block = model_folders["b"]
    config, weights = read_config(folder), rounded(read_weights(folder), dtype)
    prompts = [random_tokens(n, config["vocab_size"], 300 + n) for n in (1, 9, 24, 40)]
    llm = LLM(str(folder), dtype=dtype, kv_block_size=block, num_kv_blocks=40, max_num_seqs=4,
              enable_chunked_prefill=True, prefill_chunk_size=7, max_num_batched_tokens=16)
    got = llm.generate(prompts, SamplingParams(max_new_tokens=10))
    for tokens, prompt in zip(got, prompts):
        check_greedy(tokens, prompt, weights, config, dtype)
    assert llm.engine.counters["prefill_tokens"] == sum(len(p) for p in prompts)
    # steps of portions beside decode tokens were built while the step before ran
    assert llm.runner.prepared_mixed_steps > 0
    whole = LLM(str(folder), dtype=dtype, kv_block_size=block, num_kv_blocks=40, max_num_seqs=4)
    again = whole.generate(prompts, SamplingParams(max_new_tokens=10))
    if dtype == "float32":
        assert again == got               # the way the work is cut does not change a token

    # temperature 0.8, seed 0: every token is the plain sampler's choice for the engine's own
    # logits at that step... checked through the oracle's logits where the draw is not at an edge
    params = SamplingParams(temperature=0.8, max_new_tokens=6, seed=0)
    sampled = llm.generate(prompts, params)
    assert sampled == llm.generate(prompts, params)                               # a seed fixes the stream
    assert sampled != llm.generate(prompts, SamplingParams(temperature=0.8, max_new_tokens=6, seed=1))
    if dtype == "float32":
        for prompt, tokens in zip(prompts, sampled):
            stream = torch.Generator().manual_seed(0)
            sequence = list(prompt)
            for token in tokens:
                logits = plain.forward_logits(weights, config, sequence)[-1].float()
                uniform = Sampler.draw_uniform(stream)
                probabilities = torch.softmax(logits.double() / 0.8, dim=-1)
                edges = torch.cumsum(probabilities, dim=-1)
                if float((edges - uniform).abs().min()) < 1e-4:
                    break                                                         # a draw on an edge may fall either way
                assert token == plain_sampling.sample_row(logits, 0.8, 0, 1.0, uniform)
                sequence.append(token)


def test_long_decoding(model_folders):
    """Hundreds of decoded tokens past several page edges, compared at the end and
    on the way with the oracle's logits (teacher-forced, so a near tie cannot derail it)."""

    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner, StepEntry

    folder, block = model_folders["a"]
    config, weights = read_config(folder), read_weights(folder)
    tokens = random_tokens(400, config["vocab_size"], 77)
    runner = ModelRunner.from_folder(folder, EngineConfig(dtype="float32", kv_block_size=block, num_kv_blocks=26, decode_graphs=False))
    expected = plain.forward_logits(weights, config, tokens).float()
    runner.admit("long")
    rows = [runner.step([StepEntry("long", tuple(tokens[:3]), (2,))]).cpu()]
    for position in range(3, 400):
        rows.append(runner.step([StepEntry("long", (tokens[position],), (0,))]).cpu())
    got = torch.cat(rows)
    error = (got - expected[2:]).abs().max(dim=-1).values
    assert float(error.max()) <= 2e-5, f"first wrong position {2 + int((error > 2e-5).nonzero()[0])}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_over_hundreds_of_tokens(dtype, model_folders, tmp_path):
    """With random weights attention is nearly uniform and a lost far key would hide.
    Here the q/k norm weights are scaled so that scores are 16 times larger: weights
    concentrate on single, often far, keys."""

    from safetensors.torch import save_file

    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner, StepEntry

    folder, block = model_folders["b"]
    config, weights = read_config(folder), dict(read_weights(folder))
    for name in weights:
        if name.endswith("q_norm.weight") or name.endswith("k_norm.weight"):
            weights[name] = weights[name] * 4.0
        if name.endswith("v_proj.weight") or name.endswith("o_proj.weight"):
            weights[name] = weights[name] * 4.0
    sharp = tmp_path / "sharp"
    sharp.mkdir()
    (sharp / "config.json").write_text(json.dumps(config))
    save_file(weights, str(sharp / "model.safetensors"))
    tokens = random_tokens(700, config["vocab_size"], 5)
    oracle = rounded(weights, dtype)
    expected = plain.forward_logits(oracle, config, tokens).float()
    uniform = plain.forward_logits(rounded(read_weights(folder), dtype), config, tokens).float()
    assert float((expected - uniform).abs().max()) > 0.05                         # the scaling matters
    runner = ModelRunner.from_folder(sharp, EngineConfig(dtype=dtype, kv_block_size=block, num_kv_blocks=100,
                                                        enable_chunked_prefill=True, decode_graphs=False))
    runner.admit("s")
    rows, position = [], 0
    for size in (300, 2, 255, 100, 11) + (1,) * 32:
        part = tokens[position : position + size]
        rows.append(runner.step([StepEntry("s", tuple(part), tuple(range(len(part))))]).cpu())
        position += size
    assert position == 700
    # Scores 16 times larger carry 16 times the absolute rounding.  The yardstick is the
    # plain implementation itself in the reduced arithmetic (float32; or every intermediate
    # rounded to bfloat16 where the reference rounds) against its float64 form: the engine
    # may be off by three times that, no more.
    if dtype == "float32":
        reduced = plain.forward_logits(oracle, config, tokens, dtype=torch.float32)
    else:
        reduced = plain.forward_logits(oracle, config, tokens, rd=torch.bfloat16)
    natural = float((reduced - expected).abs().max())
    tolerance = 3 * natural
    print(f"sharp {dtype}: rounding of the plain form {natural:.2e}, tolerance {tolerance:.2e}", flush=True)
    error = (torch.cat(rows) - expected).abs().max(dim=-1).values
    assert float(error.max()) <= tolerance, f"first wrong position {int((error > tolerance).nonzero()[0])}"


def test_engine_against_itself_too_few_pages_preempt_and_give_the_same_tokens(model_folders):
    from miniserve_amd.engine import SamplingParams
    from miniserve_amd.entrypoint import LLM

    folder, block = model_folders["a"]
    config = read_config(folder)
    prompts = [random_tokens(n, config["vocab_size"], 400 + n) for n in (30, 41, 18, 25)]
    params = SamplingParams(max_new_tokens=24)
    roomy = LLM(str(folder), dtype="float32", kv_block_size=block, num_kv_blocks=32, max_num_seqs=4)
    expected = roomy.generate(prompts, params)
    tight = LLM(str(folder), dtype="float32", kv_block_size=block, num_kv_blocks=9, max_num_seqs=4,
                enable_chunked_prefill=True)
    assert tight.generate(prompts, params) == expected
    assert tight.engine.counters["preemptions"] > 0
    assert tight.runner.cache.capacity().free_blocks == (9,)
    tight.runner.cache.assert_invariants()


def test_command_line(model_folders):
    folder, block = model_folders["a"]
    config, weights = read_config(folder), read_weights(folder)
    process = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "miniserve-generate"), "--model", str(folder), "--dtype", "float32",
         "--kv-block-size", str(block), "--num-kv-blocks", "16", "--prompt-ids", "5,9,200,31", "--prompt-ids", "7",
         "--max-new-tokens", "5"],
        capture_output=True, text=True, timeout=300,
    )
    assert process.returncode == 0, process.stderr[-2000:]
    lines = [json.loads(line) for line in process.stdout.strip().splitlines()]
    assert [line["prompt_token_ids"] for line in lines] == [[5, 9, 200, 31], [7]]
    for line in lines:
        assert check_greedy(line["token_ids"], line["prompt_token_ids"], weights, config, "float32") == 5


def test_command_line_with_layer_sizes_by_name():
    """Random weights of a named size (fewer layers, so that it takes seconds): the same
    seed gives the same tokens, another seed other weights and other tokens."""

    def run(seed):
        process = subprocess.run(
            [sys.executable, str(ROOT / "bin" / "miniserve-generate"), "--random-weights", "qwen3-0.6B", "--layers", "2",
             "--seed", str(seed), "--max-model-len", "256", "--num-kv-blocks", "32", "--prompt-ids", "5,9,200,31",
             "--max-new-tokens", "6"],
            capture_output=True, text=True, timeout=300,
        )
        assert process.returncode == 0, process.stderr[-2000:]
        return json.loads(process.stdout.strip().splitlines()[-1])["token_ids"]

    first = run(3)
    assert len(first) == 6 and all(0 <= token < 151936 for token in first)
    assert run(3) == first and run(4) != first
    process = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "miniserve-generate"), "--random-weights", "qwen3-7b", "--prompt-len", "4"],
        capture_output=True, text=True, timeout=300,
    )
    assert process.returncode != 0 and "qwen3-0.6b, qwen3-32b, qwen3-8b" in process.stderr


def test_entry_point_with_layer_sizes_by_name():
    """``LLM.from_random`` with a preset's name draws what the command line draws for the
    same seed, and refuses ``layers=`` beside a configuration object."""

    from miniserve_amd.config import config_dict_from_preset_or_file, config_from_dict
    from miniserve_amd.engine import SamplingParams
    from miniserve_amd.entrypoint import LLM

    options = dict(max_model_len=256, num_kv_blocks=32, seed=3)
    by_name = LLM.from_random("qwen3-0.6b", layers=2, **options)
    tokens = by_name.generate([[5, 9, 200, 31]], SamplingParams(max_new_tokens=6))[0]
    del by_name
    data = config_dict_from_preset_or_file("qwen3-0.6b")
    data["num_hidden_layers"] = 2
    by_object = LLM.from_random(config_from_dict(data), **options)
    assert by_object.generate([[5, 9, 200, 31]], SamplingParams(max_new_tokens=6))[0] == tokens
    with pytest.raises(ValueError, match="layers="):
        LLM.from_random(config_from_dict(data), layers=1)


def test_a_seed_names_the_same_model_with_and_without_a_file(model_folders):
    """``LLM.from_random`` draws a small model as ``write_random_model`` does: its tokens are
    those of the engine over the written folder, and the plain implementation's for the
    folder's weights."""

    from miniserve_amd.config import config_from_dict
    from miniserve_amd.engine import SamplingParams
    from miniserve_amd.entrypoint import LLM

    folder, block = model_folders["a"]          # written with seed 11
    config, weights = read_config(folder), read_weights(folder)
    prompts = [random_tokens(n, config["vocab_size"], 800 + n) for n in (4, 21)]
    params = SamplingParams(max_new_tokens=7)
    options = dict(dtype="float32", kv_block_size=block, num_kv_blocks=16, max_num_seqs=2)
    drawn = LLM.from_random(config_from_dict(config), seed=11, **options).generate(prompts, params)
    assert drawn == LLM(str(folder), **options).generate(prompts, params)
    for tokens, prompt in zip(drawn, prompts):
        assert check_greedy(tokens, prompt, weights, config, "float32") == 7
    other = LLM.from_random(config_from_dict(config), seed=12, **options).runner.model.embedding.weight
    assert not torch.equal(other.cpu(), weights["model.embed_tokens.weight"])      # another seed, another model


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_engine_against_itself_recorded_steps_replay_like_eager_steps(dtype, model_folders):
    """Decode steps recorded as HIP graphs, replayed many times with eager steps
    (prompt portions, other batch sizes) and synchronisations between the
    replays: every replay gives what the eager step gives."""

    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner, StepEntry

    folder, block = model_folders["a"]
    config = read_config(folder)
    runners = [
        ModelRunner.from_folder(folder, EngineConfig(dtype=dtype, kv_block_size=block, num_kv_blocks=64, max_num_seqs=4,
                                                    enable_chunked_prefill=True, decode_graphs=graphs))
        for graphs in (True, False)
    ]
    tokens = {name: random_tokens(90, config["vocab_size"], seed) for seed, name in enumerate("abcd")}
    position = {name: 0 for name in tokens}

    def both(entries_of):
        outs = []
        for runner in runners:
            for name in entries_of:
                if not runner.cache.is_live(name):
                    runner.admit(name)
            entries = [StepEntry(n, tuple(tokens[n][position[n] : position[n] + size]), (size - 1,)) for n, size in entries_of.items()]
            outs.append(runner.step(entries).clone())
            torch.cuda.synchronize()
        for name, size in entries_of.items():
            position[name] += size
        if dtype == "float32":
            assert torch.equal(outs[0], outs[1])
        else:
            torch.testing.assert_close(outs[0], outs[1], atol=2e-2, rtol=2e-2)

    both({"a": 20, "b": 33})                       # eager: prompts
    for _ in range(6):
        both({"a": 1, "b": 1})                     # graph of batch 2, replayed
    both({"c": 17})                                # eager work in between
    for _ in range(5):
        both({"a": 1, "b": 1, "c": 1})             # graph of batch 3
    both({"a": 1, "b": 1})                         # batch 2 again, after another graph ran
    both({"d": 40, "a": 1})                        # a portion beside a decoded token: eager
    for _ in range(20):
        both({"a": 1, "b": 1, "c": 1, "d": 1})     # crosses page edges of 16
    both({"b": 1})
    assert runners[0].graph_steps == 33 and runners[1].graph_steps == 0
    assert sorted(runners[0]._decode_graphs) == [(1, 256), (2, 256), (4, 256)]    # three requests ran in the step of four


def test_engine_against_itself_steps_planned_ahead_change_no_token(model_folders):
    """The engine over the real runner, requests arriving while others run, one cancelled
    while it waits: with the next step planned while the GPU runs this one (recorded
    steps and steps with prompt portions) every request gets the tokens it gets when
    nothing is planned ahead, to the bit in 32-bit arithmetic, and nothing is left held."""

    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import Engine, ModelRunner, SamplingParams

    folder, block = model_folders["b"]
    config = read_config(folder)
    prompts = [random_tokens(n, config["vocab_size"], 900 + n) for n in (3, 41, 18, 29, 7, 55)]
    arrivals = [0, 0, 2, 5, 9, 9]
    limits = [14, 6, 11, 9, 20, 5]

    class NothingAhead:
        """The runner without the two calls that plan ahead."""

        def __init__(self, runner):
            self._runner = runner

        def __getattr__(self, name):
            if name in ("prepare_decode", "prepare_step"):
                raise AttributeError(name)
            return getattr(self._runner, name)

    def run(plan_ahead):
        runner = ModelRunner.from_folder(folder, EngineConfig(
            dtype="float32", kv_block_size=block, num_kv_blocks=40, max_num_seqs=3, enable_chunked_prefill=True,
            prefill_chunk_size=7, max_num_batched_tokens=12))
        engine = Engine(runner if plan_ahead else NothingAhead(runner))
        step, added, cancelled = 0, 0, False
        while added < len(prompts) or engine.has_unfinished():
            while added < len(prompts) and arrivals[added] <= step:
                engine.add_request(f"r{added}", prompts[added], SamplingParams(max_new_tokens=limits[added]), arrival_ns=added)
                added += 1
            engine.step()
            if not cancelled and added == len(prompts) and "r5" in engine._sequences and step >= 11:
                engine.cancel("r5")
                cancelled = True
            runner.cache.assert_invariants()
            step += 1
            assert step < 400
        assert cancelled and runner.cache.live_requests() == () and runner.cache.capacity().free_blocks == (40,)
        return [list(engine.pop_result(f"r{i}").token_ids) for i in range(5)], runner

    expected, _ = run(False)
    got, runner = run(True)
    assert got == expected
    assert [len(tokens) for tokens in got] == limits[:5]
    assert runner.prepared_mixed_steps > 0 and runner.prepared_steps > runner.prepared_mixed_steps


@pytest.mark.parametrize("live,recorded", [(11, [12]), (21, [20, 24])])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_engine_against_itself_recorded_steps_filled_up_with_spare_rows(dtype, live, recorded, model_folders):
    """Nine to eleven live requests are served by the recorded step of twelve (nineteen to
    twenty-one by those of twenty and twenty-four, where the products of more than 16
    rows take the kernel that was faster, the same in the recorded and the eager step): the rows
    that fill it up write to the spare page and the spare state slot only, and every
    request's logits are those of the eager step.  The pools are poisoned first, so
    a spare row that read or wrote a request's page would show."""

    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner, StepEntry
    from miniserve_amd.engine.runner import recorded_batch_size

    assert [recorded_batch_size(n) for n in (1, 2, 3, 4, 5, 7, 8, 9, 12, 13, 32, 33, 40, 128, 129)] == [
        1, 2, 4, 4, 8, 8, 8, 12, 12, 16, 32, 40, 40, 128, 144]
    folder, block = model_folders["b"]
    config = read_config(folder)
    runners = [
        ModelRunner.from_folder(folder, EngineConfig(dtype=dtype, kv_block_size=block, num_kv_blocks=20 * live, max_num_seqs=live,
                                                    enable_chunked_prefill=True, decode_graphs=graphs))
        for graphs in (True, False)
    ]
    for runner in runners:
        for pool in (*runner.cache.key_pools, *runner.cache.value_pools):
            pool.fill_(float("nan"))
    names = [f"r{index}" for index in range(live)]
    tokens = {name: random_tokens(80, config["vocab_size"], seed) for seed, name in enumerate(names)}
    position = {name: 0 for name in names}

    def both(entries_of):
        outs = []
        for runner in runners:
            for name in entries_of:
                if not runner.cache.is_live(name):
                    runner.admit(name)
            entries = [StepEntry(n, tuple(tokens[n][position[n] : position[n] + size]), (size - 1,)) for n, size in entries_of.items()]
            outs.append(runner.step(entries).clone())
            torch.cuda.synchronize()
        for name, size in entries_of.items():
            position[name] += size
        assert outs[0].shape == (len(entries_of), config["vocab_size"]) and torch.isfinite(outs[0]).all()
        if dtype == "float32":
            assert torch.equal(outs[0], outs[1])
        else:
            torch.testing.assert_close(outs[0], outs[1], atol=2e-2, rtol=2e-2)

    both({name: 3 + 2 * index for index, name in enumerate(names)})     # prompts of 3 tokens and more, eager
    for _ in range(3):
        both({name: 1 for name in names})                # all live: one or three spare rows
    for runner in runners:
        runner.release("r4")                             # its pages go back; the rows below move up
    for _ in range(10):
        both({name: 1 for name in names if name != "r4"})
    for runner in runners:
        runner.release("r0")
    for _ in range(10):
        both({name: 1 for name in names if name not in ("r0", "r4")})    # nine live, across page edges of 8
    assert sorted(runners[0]._decode_graphs) == [(rows, 256) for rows in recorded] and runners[0].graph_steps == 23
    cache = runners[0].cache
    assert all(cache.spare_page(0) not in cache.block_table(name) for name in cache.live_requests())


def test_a_dropped_runner_is_freed_at_once_and_recording_survives_a_collection(model_folders):
    """A runner's recorded steps hold no reference back to it: dropping the runner frees
    it, its graphs and its pinned memory without waiting for a collection of cycles -
    which, falling into a later recording, would free them there and abort the process.
    And a recording keeps the collector off while the stream records: garbage that lies
    about is still there afterwards, and goes at the next collection."""

    import gc
    import weakref

    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner, StepEntry

    folder, block = model_folders["a"]
    config = read_config(folder)

    def make():
        return ModelRunner.from_folder(folder, EngineConfig(dtype="bfloat16", kv_block_size=block, num_kv_blocks=16, max_num_seqs=2))

    def decode_once(runner):
        runner.admit("x")
        runner.step([StepEntry("x", tuple(random_tokens(5, config["vocab_size"], 1)), ())])
        return runner.step([StepEntry("x", (3,), (0,))]).clone()      # recorded, then replayed

    first = make()
    expected = decode_once(first)
    assert first.graph_steps == 1
    gone = weakref.ref(first)
    graph_gone = weakref.ref(first._decode_graphs[(1, 256)])
    del first
    assert gone() is None and graph_gone() is None

    # cyclic garbage that owns pinned and device memory, left for the collector
    class Knot:
        def __init__(self):
            self.me = self
            self.pinned = torch.zeros(1024).pin_memory()
            self.device = torch.zeros(1024, device=DEVICE)

    was_enabled = gc.isenabled()
    gc.collect()
    gc.disable()
    try:
        knot = weakref.ref(Knot())
        gc.enable()                                   # the collector may run from here on
        second = make()
        got = decode_once(second)                     # records a graph with the knot lying about
    finally:
        gc.enable() if was_enabled else gc.disable()
    assert gc.isenabled() == was_enabled
    assert torch.equal(got, expected)
    gc.collect()
    assert knot() is None
