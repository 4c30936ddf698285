"""What the compiler makes of the kernels for gfx950, read from its own report, where no
GPU is needed: no kernel keeps registers in memory (spills), and the kernels whose speed
rests on how many waves a compute unit holds keep the registers that this takes.  A
change that breaks either shows here before it shows as a slower step on the GPU."""

from __future__ import annotations

import re
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

from miniserve_amd.ops import build

# scratch memory a lane (bytes) that is known and accepted: a local table of the nucleus search
ACCEPTED_SCRATCH = {"sample_choose_kernel": 128}


def report_of(source) -> list[dict]:
    """One entry a kernel of ``source``: name (mangled), VGPRs, AGPRs, scratch bytes a lane, waves a SIMD, LDS bytes."""

    command = [build.find_hipcc(), *build.HIPCC_FLAGS, "--cuda-device-only", "-I", str(build.CSRC_DIR), "-c", str(source),
               "-o", "/dev/null", "-Rpass-analysis=kernel-resource-usage"]
    done = subprocess.run(command, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    kernels, current = [], None
    fields = {"VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch", "Occupancy [waves/SIMD]": "waves",
              "LDS Size [bytes/block]": "lds"}
    for line in done.stderr.splitlines():
        found = re.search(r"remark: [^:]+:\d+:\d+:\s+(.*?) \[-Rpass-analysis", line) or re.search(r"remark: (.*?) \[-Rpass-analysis", line)
        text = (found.group(1) if found else line).strip()
        if text.startswith("Function Name:"):
            current = {"name": text.split(":", 1)[1].strip()}
            kernels.append(current)
        elif current is not None:
            for label, key in fields.items():
                if text.startswith(label + ":"):
                    current[key] = int(text.split(":", 1)[1])
    return kernels


@pytest.fixture(scope="module")
def kernels():
    with ThreadPoolExecutor(max_workers=8) as pool:
        reports = list(pool.map(report_of, build.sources()))
    found = [kernel for report in reports for kernel in report]
    assert len(found) > 100 and all({"vgprs", "scratch", "waves", "lds"} <= set(kernel) for kernel in found)
    return found


def test_no_kernel_spills(kernels):
    for kernel in kernels:
        allowed = next((size for name, size in ACCEPTED_SCRATCH.items() if name in kernel["name"]), 0)
        assert kernel["scratch"] <= allowed, f"{kernel['name']} keeps {kernel['scratch']} bytes a lane in memory"
        assert kernel["lds"] <= 160 * 1024, f"{kernel['name']} asks for {kernel['lds']} bytes of LDS"


def test_kernels_keep_the_waves_their_speed_rests_on(kernels):
    by_name = {kernel["name"]: kernel for kernel in kernels}

    def matching(pattern):
        found = [kernel for name, kernel in by_name.items() if re.search(pattern, name)]
        assert found, pattern
        return found

    # the few-rows product, up to two tiles a workgroup and without the norm as prologue: two workgroups of eight
    # waves on a compute unit (four waves a SIMD), so that one streams while the other sums and stores; with the
    # sums scaled by a prepared norm the widest of them may fall one short
    for kernel in matching(r"gemm_skinny_kernelILi\dELi\dELb0ELi\dELb0EE"):
        mb, rb = (int(x) for x in re.search(r"ILi(\d)ELi(\d)", kernel["name"]).groups())
        if mb * rb <= 2:
            assert kernel["waves"] >= 4, (kernel["name"], kernel["vgprs"])
    for kernel in matching(r"gemm_skinny_kernelILi1ELi[12]ELb0ELi\dELb1EE"):
        assert kernel["waves"] >= 4, (kernel["name"], kernel["vgprs"])
    # attention over the cache: two waves a SIMD for the heads that run of tokens take (up to 128; single tokens up to 176)
    for kernel in matching(r"attention_decode_kernelILi(16|32|48|64|80|96|112|128|144|160|176)EE"):
        assert kernel["waves"] >= 2, (kernel["name"], kernel["vgprs"])
    for kernel in matching(r"attention_prefill_kernelILi\d+ELi\dELi\dEE"):
        assert kernel["waves"] >= 2, (kernel["name"], kernel["vgprs"])
    # the kernels that are one launch and one trip to memory hold few registers: full occupancy
    for pattern in (r"embedding_gather_kernel", r"silu_mul", r"residual_add_kernel", r"rope_table_kernel"):
        for kernel in matching(pattern):
            assert kernel["waves"] == 8, (kernel["name"], kernel["vgprs"])
