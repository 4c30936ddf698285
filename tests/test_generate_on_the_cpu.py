"""The generation tests of ``test_gpu_generate.py`` where no GPU is visible: the same test
functions, run over the torch stand-ins for the kernels and the recording that replays
a note of the forward pass (``torch_kernels.py``), with every device name taken to mean
the CPU.  They show the entry point, the engine, the runner's recorded steps,
steps planned ahead and the random-weights path; the kernels themselves, the command line
as a process, and the tests that hold a recorded step with spare rows to the bits of the
eager one (torch's products on the CPU depend on the rows beside a row in the last bit;
the library's do not) stay with the GPU tests."""

from __future__ import annotations

import inspect

import pytest
import test_gpu_generate as gpu_tests
import torch_kernels


@pytest.fixture
def on_the_cpu(monkeypatch):
    from miniserve_amd.engine import ModelRunner

    torch_kernels.install(monkeypatch, recordings=True)
    from_folder, from_random = ModelRunner.from_folder.__func__, ModelRunner.from_random.__func__
    monkeypatch.setattr(ModelRunner, "from_folder", classmethod(
        lambda cls, folder, config, device="cpu": from_folder(cls, folder, config, device="cpu")))
    monkeypatch.setattr(ModelRunner, "from_random", classmethod(
        lambda cls, config, engine_config, seed=0, device="cpu": from_random(cls, config, engine_config, seed=seed, device="cpu")))


CASES = [
    ("test_greedy_generation_tiny_a", dict(dtype="float32")),
    ("test_greedy_generation_with_wide_heads_through_recorded_steps", {}),
    ("test_chunked_prefill_mixed_with_decode_tiny_b", dict(dtype="float32")),
    ("test_long_decoding", {}),
    ("test_sharp_attention_over_hundreds_of_tokens", dict(dtype="float32")),
    ("test_engine_against_itself_too_few_pages_preempt_and_give_the_same_tokens", {}),
    ("test_a_seed_names_the_same_model_with_and_without_a_file", {}),
    ("test_engine_against_itself_recorded_steps_replay_like_eager_steps", dict(dtype="float32")),
    ("test_engine_against_itself_steps_planned_ahead_change_no_token", {}),
]


@pytest.mark.parametrize("name,extra", CASES, ids=[f"{name[5:]}{'-' + '-'.join(str(v) for v in extra.values()) if extra else ''}"
                                                   for name, extra in CASES])
def test_generation(name, extra, on_the_cpu, model_folders, tmp_path):
    function = getattr(gpu_tests, name)
    wanted = inspect.signature(function).parameters
    arguments = dict(extra)
    if "model_folders" in wanted:
        arguments["model_folders"] = model_folders
    if "tmp_path" in wanted:
        arguments["tmp_path"] = tmp_path
    function(**arguments)
