"""The replay tests of ``test_gpu_replay.py`` where no GPU is visible: the same test
functions over the torch stand-ins for the kernels (``torch_kernels.py``), with every
device name taken to mean the CPU: stale values in reused pages, the first tokens of a
sequence, steps without wanted logits and requests that pause.  (The four replay shapes
run on the CPU in ``test_engine_with_torch_kernels.py``, without the GPU tests' claim
that the ways of cutting agree to the bit, which holds for the library's kernels and not
for torch's products.  The program ``bin/trace_run`` itself stays with the GPU tests.)"""

from __future__ import annotations

import inspect

import pytest
import test_gpu_replay as gpu_tests
import torch_kernels

oracle = gpu_tests.oracle


@pytest.fixture
def on_the_cpu(monkeypatch):
    from miniserve_amd.engine import ModelRunner

    torch_kernels.install(monkeypatch)
    from_folder = ModelRunner.from_folder.__func__
    monkeypatch.setattr(ModelRunner, "from_folder", classmethod(
        lambda cls, folder, config, device="cpu": from_folder(cls, folder, config, device="cpu")))


CASES = [
    ("test_reused_pages_hold_stale_values_that_are_never_seen", {}),
    ("test_first_tokens_of_a_sequence", {}),
    ("test_steps_without_wanted_logits_and_requests_that_pause", {}),
]


@pytest.mark.parametrize("test,extra", CASES, ids=[f"{test[5:]}{'-' + '-'.join(str(v) for v in extra.values()) if extra else ''}"
                                                   for test, extra in CASES])
def test_replay(test, extra, on_the_cpu, model_folders, oracle, tmp_path):  # noqa: F811
    function = getattr(gpu_tests, test)
    wanted = inspect.signature(function).parameters
    arguments = dict(extra)
    for fixture, value in (("model_folders", model_folders), ("oracle", oracle), ("tmp_path", tmp_path)):
        if fixture in wanted:
            arguments[fixture] = value
    function(**arguments)
