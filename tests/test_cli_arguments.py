"""The command line's options reach the entry point under the reference's names, and
what it prints is what the entry point returned: on the CPU, with a stand-in for the
entry point (no model is built)."""

from __future__ import annotations

import json
from types import SimpleNamespace

import pytest


class StandIn:
    """Records how the command line built it and what it asked it to generate."""

    last = None

    def __init__(self, model, **options):
        self.model, self.options = model, options
        self.runner = SimpleNamespace(spec=SimpleNamespace(vocab_size=50))
        StandIn.last = self
        if options.get("kv_block_size") == 3:
            raise ValueError("kv_block_size 3 is not served.")

    def generate(self, prompts, params):
        self.prompts, self.params = prompts, params
        return [[len(p), 7] for p in prompts]


@pytest.fixture
def cli(monkeypatch):
    import miniserve_amd.cli as module
    import miniserve_amd.entrypoint as entrypoint

    monkeypatch.setattr(entrypoint, "LLM", StandIn)
    return module


def test_options_carry_the_references_names_and_reach_the_entry_point(cli, capsys, tmp_path):
    folder = tmp_path / "model"
    code = cli.main([
        "--model", str(folder), "--prompt-ids", "1,2,3", "--prompt-ids", "4, 5", "--max-new-tokens", "5",
        "--temperature", "0.7", "--top-p", "0.9", "--top-k", "20", "--seed", "11", "--stop-token-ids", "2, 9",
        "--dtype", "float32", "--max-model-len", "128", "--num-kv-blocks", "40", "--max-num-seqs", "3",
        "--max-pending-requests", "9", "--max-num-batched-tokens", "64", "--kv-block-size", "32",
        "--chunked-prefill", "--prefill-chunk-size", "16", "--decode-execution", "eager",
    ])
    assert code == 0
    made = StandIn.last
    assert made.model == str(folder)
    assert made.options == dict(
        seed=11, dtype="float32", max_model_len=128, num_kv_blocks=40, max_num_seqs=3, max_pending_requests=9,
        max_num_batched_tokens=64, kv_block_size=32, enable_chunked_prefill=True, prefill_chunk_size=16, decode_graphs=False)
    assert made.prompts == [[1, 2, 3], [4, 5]]
    assert [(p.temperature, p.top_p, p.top_k, p.max_new_tokens, p.stop_token_ids) for p in made.params] == [(0.7, 0.9, 20, 5, (2, 9))] * 2
    assert [p.seed for p in made.params] == [11, 12]                     # a stream of its own for every prompt
    lines = [json.loads(line) for line in capsys.readouterr().out.splitlines()]
    assert lines == [{"prompt_token_ids": [1, 2, 3], "token_ids": [3, 7]}, {"prompt_token_ids": [4, 5], "token_ids": [2, 7]}]


def test_defaults_random_weights_and_random_prompts(cli, capsys):
    assert cli.main(["--random-weights", "qwen3-0.6b", "--layers", "2", "--prompt-len", "6", "--prompt-len", "3"]) == 0
    made = StandIn.last
    assert made.model.num_hidden_layers == 2 and made.model.hidden_size == 1024      # a configuration, not a folder
    assert made.options == dict(
        seed=0, dtype="bfloat16", max_model_len=None, num_kv_blocks=None, max_num_seqs=8, max_pending_requests=64,
        max_num_batched_tokens=None, kv_block_size=16, enable_chunked_prefill=False, prefill_chunk_size=None, decode_graphs=True)
    assert [len(p) for p in made.prompts] == [6, 3] and all(0 <= t < 50 for p in made.prompts for t in p)
    assert all(p.temperature == 0 and p.max_new_tokens == 16 and p.stop_token_ids == () for p in made.params)
    first = made.prompts
    capsys.readouterr()
    cli.main(["--random-weights", "qwen3-0.6b", "--prompt-len", "6", "--prompt-len", "3"])
    assert StandIn.last.prompts == first and StandIn.last.model.num_hidden_layers == 28    # the seed names the prompts


def test_what_the_command_line_refuses(cli, capsys):
    for argv in (
        ["--prompt-len", "4"],                                            # neither a model nor random weights
        ["--model", "m", "--random-weights", "qwen3-0.6b", "--prompt-len", "4"],
        ["--model", "m"],                                                 # no prompt
        ["--model", "m", "--prompt-len", "4", "--prompt-ids", "1"],
        ["--model", "m", "--prompt-len", "4", "--chunked-prefill", "--no-chunked-prefill"],
        ["--model", "m", "--prompt-len", "4", "--dtype", "float16"],
        ["--random-weights", "no-such-preset", "--prompt-len", "4"],
        ["--model", "m", "--prompt-len", "4", "--kv-block-size", "3"],   # the entry point's own refusal becomes a usage error
    ):
        with pytest.raises(SystemExit) as raised:
            cli.main(argv)
        assert raised.value.code == 2, argv
    assert "kv_block_size 3 is not served" in capsys.readouterr().err
