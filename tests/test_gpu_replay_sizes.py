"""Trace replay at the layer sizes that are served, against the plain implementation:
the widths of Qwen3-0.6B (hidden 1024, 16 query and 8 key/value heads of 128, feed-forward
3072, 151,936 tokens, tied head) with three layers, the widths of Qwen3-8B (hidden
4096, 32 and 8 heads, feed-forward 12288, untied head) and those of Qwen3-32B (hidden
5120, 64 and 8 heads: eight query heads to a key/value head, feed-forward 25600) with
one layer each and a shorter, odd vocabulary.  Requests of 90 to 700 tokens run whole, with the last 32 tokens one
by one, in portions of changing size, and mixed on so few pages that they are used
again; in 32-bit and in bfloat16, the latter with each of the two matrix products
forced in turn.  The pools are filled with NaN before every run.

The reference checks its model the same way, step by step with given tokens
(miniserve/benchmark/compare_hf.py:306-381), against a library model; here the
other side is ``tests/plain_qwen3.py`` in float64.
"""

from __future__ import annotations

import io
import shutil
import subprocess
import sys

import plain_qwen3 as plain
import pytest
import replay_shapes as shapes
import torch
from helpers import ROOT, make_model_folder, random_tokens, read_config, read_weights

pytestmark = pytest.mark.gpu


def widths_0p6b() -> dict:
    return {
        "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "hidden_size": 1024, "intermediate_size": 3072,
        "num_hidden_layers": 3, "num_attention_heads": 16, "num_key_value_heads": 8, "head_dim": 128,
        "vocab_size": 151936, "max_position_embeddings": 2048, "rms_norm_eps": 1e-6, "rope_theta": 1000000.0,
        "tie_word_embeddings": True, "hidden_act": "silu", "attention_bias": False, "attention_dropout": 0.0,
    }


def widths_8b() -> dict:
    return {
        "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "hidden_size": 4096, "intermediate_size": 12288,
        "num_hidden_layers": 1, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
        "vocab_size": 20011, "max_position_embeddings": 2048, "rms_norm_eps": 1e-6, "rope_theta": 1000000.0,
        "tie_word_embeddings": False, "hidden_act": "silu", "attention_bias": False, "attention_dropout": 0.0,
    }


def widths_32b() -> dict:
    return {
        "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "hidden_size": 5120, "intermediate_size": 25600,
        "num_hidden_layers": 1, "num_attention_heads": 64, "num_key_value_heads": 8, "head_dim": 128,
        "vocab_size": 20011, "max_position_embeddings": 2048, "rms_norm_eps": 1e-6, "rope_theta": 1000000.0,
        "tie_word_embeddings": False, "hidden_act": "silu", "attention_bias": False, "attention_dropout": 0.0,
    }


MODELS = {"0.6b": (widths_0p6b, (100, 700, 333, 257, 512)), "8b": (widths_8b, (150, 420, 90, 260, 330)),
          "32b": (widths_32b, (130, 300, 70, 200, 150))}
BLOCK = 16
# portions that end on, before and after the edges of pages (16) and of the attention kernel's tiles (64)
PORTIONS = (64, 2, 130, 17, 255, 2, 33, 1, 96, 300, 15, 49)


def wanted_positions(length: int) -> list[int]:
    """The places compared: the first three, every 16th, and the last 34 (the decoded tail and two before it)."""

    return sorted({0, 1, 2} | set(range(3, length, 16)) | set(range(max(length - 34, 0), length)))


def restrict_wants(steps: list[dict], wanted: dict[str, set[int]]) -> list[dict]:
    """The same steps asking only for the logits at the ``wanted`` positions of each request."""

    position: dict[str, int] = {}
    result = []
    for step in steps:
        entries = []
        for entry in step["entries"]:
            start = position.get(entry["id"], 0)
            entries.append({**entry, "want": [w for w in entry["want"] if start + w in wanted[entry["id"]]]})
            position[entry["id"]] = start + len(entry["tokens"])
        for name in step["end"]:
            position.pop(name, None)
        result.append({**step, "entries": entries})
    return result


@pytest.fixture(scope="module")
def sized(tmp_path_factory):
    """Per model: its folder, configuration, requests, wanted positions and the plain
    implementation's logits there (float64), made once."""

    made = {}

    def get(name: str):
        if name not in made:
            make_config, lengths = MODELS[name]
            folder = make_model_folder(tmp_path_factory.mktemp(f"sized_{name.replace('.', '_')}"), make_config(),
                                       seed=41, store_dtype="bfloat16")
            config = read_config(folder)
            weights = {key: tensor.to(torch.float64) for key, tensor in read_weights(folder).items()}
            requests = {f"r{index}": random_tokens(length, config["vocab_size"], 700 + index)
                        for index, length in enumerate(lengths)}
            wanted = {rid: wanted_positions(len(tokens)) for rid, tokens in requests.items()}
            logits = {}
            for rid, tokens in requests.items():
                print(f"plain implementation {name} {rid}: {len(tokens)} tokens", flush=True)
                rows = plain.forward_logits(weights, config, tokens, rows=wanted[rid]).float()
                logits[rid] = dict(zip(wanted[rid], rows))
            # the yardstick of bfloat16: the plain implementation with every intermediate rounded where the
            # reference rounds, against itself in float64, on the request of middle length
            probe = sorted(requests, key=lambda rid: len(requests[rid]))[len(requests) // 2]
            rounded = plain.forward_logits(weights, config, requests[probe], rows=wanted[probe], rd=torch.bfloat16).float()
            yardstick = float((rounded - torch.stack([logits[probe][p] for p in wanted[probe]])).abs().max())
            size = float(max(row.abs().max() for rows in logits.values() for row in rows.values()))
            print(f"{name}: largest logit {size:.2f}, bfloat16 yardstick {yardstick:.2e}", flush=True)
            made[name] = (folder, config, requests, wanted, logits, yardstick, size)
        return made[name]

    return get


def make_runner(folder, dtype, pages):
    from miniserve_amd.config import EngineConfig
    from miniserve_amd.engine import ModelRunner

    config = EngineConfig(dtype=dtype, kv_block_size=BLOCK, num_kv_blocks=pages, max_num_seqs=8,
                          enable_chunked_prefill=True, decode_graphs=False)
    runner = ModelRunner.from_folder(folder, config)
    for pool in (*runner.cache.key_pools, *runner.cache.value_pools):
        pool.fill_(float("nan"))
    return runner


def the_shapes(requests, wanted):
    wanted_sets = {rid: set(places) for rid, places in wanted.items()}
    return {
        "whole": restrict_wants(shapes.whole(requests), wanted_sets),
        "tail": restrict_wants(shapes.prefill_then_decode(requests), wanted_sets),
        "portions": restrict_wants(shapes.portions(requests, PORTIONS), wanted_sets),
        "mixed": restrict_wants(shapes.mixed(requests, seed=9, tail=32), wanted_sets),
    }


def run_shape(folder, dtype, steps, logits, vocab, tolerance, out_dir):
    from miniserve_amd.engine.replay import replay

    pages = -(-shapes.max_live_tokens(steps) // BLOCK)
    runner = make_runner(folder, dtype, pages)
    assert replay(runner, shapes.to_lines(steps), out_dir, report=io.StringIO()) == len(steps)
    got = shapes.collect(steps, out_dir, vocab)
    shutil.rmtree(out_dir)
    assert len(got) == sum(len(rows) for rows in logits.values())
    worst = (0.0, None)
    for (rid, position), row in sorted(got.items()):
        assert bool(torch.isfinite(row).all()), f"non-finite logits at {(rid, position)}"
        error = float((row - logits[rid][position]).abs().max())
        if error > worst[0]:
            worst = (error, (rid, position))
    assert worst[0] <= tolerance, f"worst place {worst[1]}: error {worst[0]:.3e} > {tolerance:.3e}"
    assert runner.cache.live_requests() == ()
    runner.cache.assert_invariants()
    return got, worst[0]


@pytest.mark.parametrize("name", list(MODELS))
def test_replay_at_served_widths_in_32_bit(name, sized, tmp_path):
    folder, config, requests, wanted, logits, _, size = sized(name)
    # a few hundred float32 roundings on logits of this size
    tolerance = 2e-5 * max(1.0, size)
    results = {}
    for shape, steps in the_shapes(requests, wanted).items():
        results[shape], worst = run_shape(folder, "float32", steps, logits, config["vocab_size"], tolerance, tmp_path / shape)
        print(f"{name} float32 {shape}: {len(steps)} steps, worst error {worst:.2e} (allowed {tolerance:.2e})", flush=True)
    for shape in ("tail", "portions", "mixed"):
        for key, row in results["whole"].items():
            assert torch.equal(row, results[shape][key]), f"{shape} differs from whole at {key}"


@pytest.mark.parametrize("product", ["skinny", "library"])
@pytest.mark.parametrize("name", list(MODELS))
def test_replay_at_served_widths_in_bfloat16(name, product, sized, tmp_path):
    """``product``: which of the two matrix products serves every call that both can
    serve (this library's for up to 64 rows, hipBLASLt for any number)."""

    from miniserve_amd import ops

    folder, config, requests, wanted, logits, yardstick, _ = sized(name)
    tolerance = 3 * yardstick
    with ops.forced_product(product):
        before = dict(ops.product_calls)
        for shape, steps in the_shapes(requests, wanted).items():
            _, worst = run_shape(folder, "bfloat16", steps, logits, config["vocab_size"], tolerance, tmp_path / shape)
            print(f"{name} bfloat16 {product} {shape}: {len(steps)} steps, worst error {worst:.2e} "
                  f"(allowed {tolerance:.2e})", flush=True)
        used = {kind: ops.product_calls[kind] - before[kind] for kind in before}
    assert used[product] > 0
    if product == "library":
        assert used["skinny"] == 0


def test_two_processes_give_the_same_bfloat16_logits_to_the_bit(sized, tmp_path):
    """Which kernel and which of the library's algorithms serves a product is a fixed rule
    of its shape: nothing is timed in a serving process.  The replay program, run twice in
    fresh processes on the same model and steps, writes the same bits."""

    folder, config, requests, wanted, _, _, _ = sized("0.6b")
    steps = the_shapes(requests, wanted)["mixed"]
    lines = "".join(line + "\n" for line in shapes.to_lines(steps))
    outs = []
    for run in range(2):
        out = tmp_path / f"run{run}"
        process = subprocess.run(
            [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", "bfloat16", "--out", str(out),
             "--max-tokens", str(shapes.max_live_tokens(steps))],
            input=lines, capture_output=True, text=True, timeout=600,
        )
        assert process.returncode == 0, process.stderr[-2000:]
        outs.append(out)
    files = sorted(path.name for path in outs[0].iterdir())
    assert files and files == sorted(path.name for path in outs[1].iterdir())
    for name in files:
        assert (outs[0] / name).read_bytes() == (outs[1] / name).read_bytes(), f"step file {name} differs between the runs"
