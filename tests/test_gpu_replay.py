"""Trace replay on the GPU against the plain implementation: each request alone and
whole; most of it in one step and the last 32 tokens one by one; in portions of
changing size; mixed with other requests on so few pages that they are used
again - in 32-bit and in bfloat16, for every tiny configuration."""

from __future__ import annotations

import io
import os
import subprocess
import sys
from pathlib import Path

import plain_qwen3 as plain
import pytest
import replay_shapes as shapes
import torch
from helpers import ROOT, random_tokens, read_config, read_weights

pytestmark = pytest.mark.gpu

# Logits of these models are of size ~1.  float32 against the float64 oracle:
# rounding of a few hundred float32 operations.  bfloat16: activations carry 8
# bits, the logits themselves are rounded to bfloat16 (2^-9 relative).
TOLERANCE = {"float32": 2e-5, "bfloat16": 2.5e-2}
LENGTHS = {"a": (45, 70, 100, 33, 18, 64, 81), "b": (41, 96, 64, 57, 9, 80), "c": (150, 37, 66, 90, 129, 40)}


def reference_weights(weights, dtype):
    if dtype == "bfloat16":
        return {name: tensor.to(torch.bfloat16).float() for name, tensor in weights.items()}
    return weights


def make_runner(folder, dtype, block_size, num_blocks):
    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner

    config = EngineConfig(
        dtype=dtype, kv_block_size=block_size, num_kv_blocks=num_blocks, max_num_seqs=8,
        enable_chunked_prefill=True, decode_graphs=False,
    )
    return ModelRunner.from_folder(folder, config)


@pytest.fixture(scope="module")
def oracle(model_folders):
    """Requests and the plain implementation's logits for them, per model and dtype."""

    cache = {}

    def get(name, dtype):
        if (name, dtype) not in cache:
            folder, _ = model_folders[name]
            config = read_config(folder)
            weights = reference_weights(read_weights(folder), dtype)
            requests = {
                f"r{index}": random_tokens(length, config["vocab_size"], 50 + index)
                for index, length in enumerate(LENGTHS[name])
            }
            logits = {rid: plain.forward_logits(weights, config, tokens).float() for rid, tokens in requests.items()}
            cache[(name, dtype)] = (requests, logits, config)
        return cache[(name, dtype)]

    return get


def run_and_compare(runner, steps, requests, logits, vocab, tolerance, tmp_path):
    from miniserve_amd.engine.replay import replay

    report = io.StringIO()
    assert replay(runner, shapes.to_lines(steps), tmp_path, report=report) == len(steps)
    assert report.getvalue().split() == [w for s in steps for w in ("done", str(s["step"]))]
    got = shapes.collect(steps, tmp_path, vocab)
    assert len(got) == sum(len(tokens) for tokens in requests.values())
    worst = (0.0, None)
    for (rid, position), row in got.items():
        error = float((row - logits[rid][position]).abs().max())
        if error > worst[0]:
            worst = (error, (rid, position))
    assert worst[0] <= tolerance, f"first/worst wrong place {worst[1]}: error {worst[0]:.3e} > {tolerance}"
    assert runner.cache.live_requests() == ()
    runner.cache.assert_invariants()
    return got


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_replay_shapes(name, dtype, model_folders, oracle, tmp_path):
    folder, block_size = model_folders[name]
    requests, logits, config = oracle(name, dtype)
    vocab = config["vocab_size"]
    results = {}
    for shape, steps in (
        ("whole", shapes.whole(requests)),
        ("tail", shapes.prefill_then_decode(requests)),
        ("portions", shapes.portions(requests)),
        ("mixed", shapes.mixed(requests, seed=3)),
    ):
        pages = -(-shapes.max_live_tokens(steps) // block_size)
        runner = make_runner(folder, dtype, block_size, pages)
        print(f"replay {name} {dtype} {shape}: {len(steps)} steps, {pages} pages", flush=True)
        results[shape] = run_and_compare(
            runner, steps, requests, logits, vocab, TOLERANCE[dtype], tmp_path / shape
        )
        if shape == "mixed":
            assert any(len(s["entries"]) > 1 for s in steps)
            assert len(requests) > 4      # more requests than are live at once: later ones get used pages
    if dtype == "float32":
        # The 32-bit kernels fix the order of every sum per position, so the logits
        # at a position are the same to the bit however the work is cut.
        for shape in ("tail", "portions", "mixed"):
            for key, row in results["whole"].items():
                assert torch.equal(row, results[shape][key]), f"{shape} differs from whole at {key}"


def test_reused_pages_hold_stale_values_that_are_never_seen(model_folders, oracle, tmp_path):
    """A pool of exactly one request's pages: every request reuses the pages of the
    one before, which are first filled with a poison value."""

    folder, block_size = model_folders["a"]
    requests, logits, config = oracle("a", "float32")
    steps = shapes.portions(requests)
    pages = -(-shapes.max_live_tokens(steps) // block_size)
    runner = make_runner(folder, "float32", block_size, pages)
    for pool in (*runner.cache.key_pools, *runner.cache.value_pools):
        pool.fill_(float("nan"))
    run_and_compare(runner, steps, requests, logits, config["vocab_size"], TOLERANCE["float32"], tmp_path)


def test_first_tokens_of_a_sequence(model_folders, oracle, tmp_path):
    """Positions 0, 1, 2: a single key, no history, a portion of one token at the start."""

    folder, block_size = model_folders["b"]
    requests, logits, config = oracle("b", "float32")
    tokens = requests["r0"][:3]
    steps = [
        {"step": 0, "entries": [{"id": "r0", "tokens": tokens[:1], "want": [0]}], "end": []},
        {"step": 1, "entries": [{"id": "r0", "tokens": tokens[1:3], "want": [0, 1]}], "end": ["r0"]},
    ]
    runner = make_runner(folder, "float32", block_size, 8)
    short = {"r0": tokens}
    run_and_compare(runner, steps, short, logits, config["vocab_size"], TOLERANCE["float32"], tmp_path)


def test_steps_without_wanted_logits_and_requests_that_pause(model_folders, oracle, tmp_path):
    from miniserve_amd.engine.replay import replay

    folder, block_size = model_folders["a"]
    requests, logits, config = oracle("a", "float32")
    a, b = requests["r0"], requests["r3"]
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:20], "want": []}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:9], "want": [8]}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[20:45], "want": [24]}, {"id": "b", "tokens": b[9:11], "want": []}],
         "end": ["a"]},
        {"step": 3, "entries": [{"id": "b", "tokens": b[11:33], "want": [0, 21]}], "end": ["b"]},
    ]
    runner = make_runner(folder, "float32", block_size, 16)
    replay(runner, shapes.to_lines(steps), tmp_path, report=io.StringIO())
    assert not (tmp_path / "0.f32").exists()
    got = shapes.collect(steps, tmp_path, config["vocab_size"])
    expected = {("b", 8): logits["r3"][8], ("a", 44): logits["r0"][44], ("b", 11): logits["r3"][11], ("b", 32): logits["r3"][32]}
    assert got.keys() == expected.keys()
    for key, row in expected.items():
        assert float((got[key] - row).abs().max()) <= TOLERANCE["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(dtype, model_folders, oracle, tmp_path):
    """The program itself, as a user calls it: steps on standard input, ``done`` lines back."""

    folder, block_size = model_folders["b"]
    requests, logits, config = oracle("b", dtype)
    steps = shapes.mixed(requests, seed=5)
    out = tmp_path / "out"
    process = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", dtype, "--out", str(out),
         "--max-tokens", str(shapes.max_live_tokens(steps))],
        input="\n".join(shapes.to_lines(steps)) + "\n", capture_output=True, text=True, timeout=300,
    )
    assert process.returncode == 0, process.stderr[-2000:]
    assert process.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    got = shapes.collect(steps, out, config["vocab_size"])
    for (rid, position), row in got.items():
        assert float((row - logits[rid][position]).abs().max()) <= TOLERANCE[dtype], (rid, position)
