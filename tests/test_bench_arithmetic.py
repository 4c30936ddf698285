"""The arithmetic behind the measurement's fractions, on the CPU: the bytes a decode step
has to read and the operations of a prefill, for the layer sizes that are measured,
against numbers worked out by hand from the configurations; the published peaks; and
that the program refuses more than one GPU with the code the contract names."""

from __future__ import annotations

import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def model_of(preset):
    from miniserve_amd.config import config_dict_from_preset_or_file, config_from_dict
    from miniserve_amd.parts import DecoderModel

    config = config_from_dict(config_dict_from_preset_or_file(preset))
    return config, DecoderModel(config.model_spec(), "bfloat16")


def by_hand(hidden, inter, layers, q_heads, kv_heads, dim, vocab, tied):
    """Elements of every matrix and norm weight a decode step reads once (``tied`` or not, one
    matrix of vocabulary x hidden: the head's, which a tied model shares with its embedding)."""

    attention = hidden * (q_heads + 2 * kv_heads) * dim + q_heads * dim * hidden + 2 * dim       # q/k/v, o, q and k norms
    layer = attention + 3 * hidden * inter + 2 * hidden                                              # + gate, up, down, two norms
    return layers * layer + hidden + vocab * hidden                                                 # + final norm + the head's matrix


@pytest.mark.parametrize("preset,sizes", [
    ("qwen3-0.6b", dict(hidden=1024, inter=3072, layers=28, q_heads=16, kv_heads=8, dim=128, vocab=151936, tied=True)),
    ("qwen3-8b", dict(hidden=4096, inter=12288, layers=36, q_heads=32, kv_heads=8, dim=128, vocab=151936, tied=False)),
    ("qwen3-32b", dict(hidden=5120, inter=25600, layers=64, q_heads=64, kv_heads=8, dim=128, vocab=151936, tied=False)),
])
def test_bytes_of_a_decode_step_and_operations_of_a_prefill(preset, sizes):
    import bench

    config, model = model_of(preset)
    # a tied head's matrix is the embedding table and counts once; an untied model's embedding table is read by
    # row and does not count, its head's matrix does
    assert bench.weight_bytes(model, 2) == 2 * by_hand(**sizes)
    h, i, layers, vocab = sizes["hidden"], sizes["inter"], sizes["layers"], sizes["vocab"]
    q, kv = sizes["q_heads"] * sizes["dim"], sizes["kv_heads"] * sizes["dim"]
    row = 2 * (h * (q + 2 * kv) + q * h + 3 * h * i)
    assert bench.per_token_flops(config) == layers * row
    tokens = 2048
    assert bench.prefill_flops(config, tokens) == layers * (row * tokens + 2 * q * tokens * tokens) + 2 * h * vocab
    # the cache of a live request, a token: keys and values of every layer
    from miniserve_amd.cache import CacheLayout

    assert CacheLayout.from_needs(model.cache_needs()).bytes_per_token(2) == layers * 2 * kv * 2


def test_the_numbers_of_the_headline_configuration():
    """0.6B sizes: 1.192 GB of weights a step; 8 rows at 2,065 tokens of context read 1.895 GB of cache; a prefill of
    2,048 tokens is 2.285 TFLOP."""

    import bench

    config, model = model_of("qwen3-0.6b")
    assert round(bench.weight_bytes(model, 2) / 1e9, 3) == 1.192
    assert 28 * 2 * 8 * 128 * 2 == 114688 and round(8 * 2065 * 114688 / 1e9, 3) == 1.895
    assert round(bench.prefill_flops(config, 2048) / 1e12, 3) == 2.285
    assert bench.HBM_GBPS == 8000.0 and bench.PEAK_TFLOPS == {"bfloat16": 2500.0, "float32": 157.3}


def test_more_than_one_gpu_is_refused_with_one_line_and_code_2():
    done = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert done.returncode == 2 and len(done.stdout.strip().splitlines()) == 1 and "--gpus 2" in done.stdout


def test_a_kernel_trace_is_accounted_step_by_step(tmp_path, capsys):
    """``--account-trace`` on a made-up trace: a step begins with the embedding kernel, decode steps are those
    of the most frequent kernel count without the first four, medians a kernel."""

    import bench

    rows, clock = ["Kernel_Name,Start_Timestamp,End_Timestamp"], 0

    def kernel(name, us):
        nonlocal clock
        rows.append(f'"{name}",{clock},{clock + int(us * 1000)}')
        clock += int(us * 1000) + 2000

    for step in range(10):                                           # ten decode steps of 1 + 2 * 3 kernels
        kernel("void (anonymous namespace)::embedding_gather_kernel<ms::bf16>(int const*)", 3)
        for _ in range(2):
            kernel("void (anonymous namespace)::gemm_skinny_kernel<1, 1, false, 8, false>(ms::bf16 const*)", 5)
            kernel("void (anonymous namespace)::attention_decode_kernel<128>(ms::bf16 const*)", 17 if step != 7 else 40)
            kernel("Cijk_Alik_Bljk_BBS_BH_MT16x16x512_MI16x16x1_SN_K1", 21)
    for _ in range(3):                                               # three prefill steps
        kernel("void (anonymous namespace)::embedding_gather_kernel<ms::bf16>(int const*)", 9)
        kernel("void (anonymous namespace)::attention_prefill_kernel<128, 2, 2>(ms::bf16 const*)", 43)
    path = tmp_path / "p_kernel_trace.csv"
    path.write_text("\n".join(rows) + "\n")
    bench.account_trace(str(path))
    out = capsys.readouterr().out
    assert "decode step: 6 steps, 7 kernels a step; kernel time 89.0 us" in out
    assert "attention_decode_kernel<128>" in out and "hipBLASLt MT16x16x512" in out and "gemm_skinny_kernel<1, 1, false, 8, false>" in out
    line = next(text for text in out.splitlines() if text.startswith("attention_decode_kernel<128>"))
    assert line.split()[-4:] == ["2", "34.0", "17.00", "6"]          # calls, us a step (median: the slow step does not move it), average, steps
    assert "prefill step: 3 steps, 2 kernels a step; kernel time 52.0 us" in out
