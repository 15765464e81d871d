"""Properties of the generated gfx950 code that the kernels' speed depends on and that the compiler has broken
before without any wrong result to show for it: every `buffer_load ... lds` must take its descriptor from scalar
registers (otherwise each load becomes a loop over the distinct descriptor values), and the K loop of every GEMM
kernel must not touch scratch memory (a reload there waits for all loads in flight) nor spill scalar registers to vector lanes.  Compiles the device code of
ms_gemm.hip to assembly (no GPU needed) and reads it."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "meshslice_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


@pytest.fixture(scope="module")
def gemm_asm(tmp_path_factory):
    if not os.path.exists(HIPCC):
        pytest.skip("hipcc is not installed")
    out = tmp_path_factory.mktemp("isa") / "ms_gemm.s"
    subprocess.check_call([HIPCC, "-O3", "-std=c++17", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                           "-I" + os.path.join(ROOT, "include"), "-Wno-unused-command-line-argument", "--cuda-device-only", "-S",
                           "-o", str(out), os.path.join(CSRC, "ms_gemm.hip")], cwd=CSRC, stderr=subprocess.DEVNULL)
    text = out.read_text()
    kernels = {}
    for name in re.findall(r"^(_ZN3msk\w*gemm_(?:bf16|f32)_\w+):", text, re.M):
        start = text.index(name + ":")
        kernels[name] = text[start:text.index("s_endpgm", start)].split("\n")
    assert len(kernels) >= 80
    return kernels


def _loops(body):
    """(first line, last line) of every backward branch."""
    labels = {m.group(1): n for n, l in enumerate(body) for m in [re.match(r"^(\.LBB\d+_\d+):", l)] if m}
    for n, l in enumerate(body):
        m = re.search(r"s_cbranch_(\w+)\s+(\.LBB\d+_\d+)", l)
        if m and m.group(2) in labels and labels[m.group(2)] < n:
            yield labels[m.group(2)], n, m.group(1)


def test_no_load_is_wrapped_in_a_descriptor_loop(gemm_asm):
    offenders = []
    for name, body in gemm_asm.items():
        for a, b, cond in _loops(body):
            if cond == "execnz" and b - a < 40 and any("buffer_load" in x for x in body[a:b]):
                offenders.append(name)
                break
    assert not offenders, f"loads with vector descriptors in {offenders}"


def test_the_k_loops_do_not_touch_scratch_memory(gemm_asm):
    offenders, lane_spills = [], []
    for name, body in gemm_asm.items():
        # the K loop: the innermost loop that holds the MFMAs of at least two K steps
        inner = None
        for a, b, _ in _loops(body):
            n_mfma = sum("v_mfma" in x for x in body[a:b])
            if n_mfma >= 32 and (inner is None or b - a < inner[1] - inner[0]):
                inner = (a, b)
        assert inner is not None, f"no K loop found in {name}"
        if any("scratch_" in x for x in body[inner[0]:inner[1]]):
            offenders.append(name)
        # scalar registers spilled to vector lanes cost VALU issue slots between the MFMAs
        if any("v_readlane" in x or "v_writelane" in x for x in body[inner[0]:inner[1]]):
            lane_spills.append(name)
    assert not offenders, f"scratch traffic inside the K loop of {offenders}"
    assert not lane_spills, f"scalar registers spilled to vector lanes inside the K loop of {lane_spills}"
