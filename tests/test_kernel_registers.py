"""The 256 x 256 tile product keeps its 256 accumulators in AGPRs that only its assembly statements
name: between the loop and the reads of the accumulators the compiler must not touch them. It has no
reason to (no matrix builtins in that kernel, nothing spilled), and this test holds it to that: the kernel's
device assembly, made here with the build's own flags, uses no scratch memory, all 256 AGPRs, and has no
AGPR instruction outside the assembly statements. No GPU is needed: hipcc cross-compiles."""

from __future__ import annotations

import re
import shutil
import subprocess

import pytest

from miniserve_amd.kernels import build


@pytest.fixture(scope="module")
def gemm_assembly(tmp_path_factory):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not shutil.which(hipcc):
        pytest.skip("no hipcc")
    out = tmp_path_factory.mktemp("asm") / "gemm_bf16.s"
    flags = [f for f in build.HIP_FLAGS if f != "-fPIC"]
    subprocess.run([hipcc, *flags, "--cuda-device-only", "-S", "-o", str(out), str(build.CSRC / "gemm_bf16.hip")],
                   check=True, capture_output=True, timeout=300)
    return out.read_text()


def test_the_wide_tile_kernel_owns_its_accumulators(gemm_assembly):
    text = gemm_assembly
    name = next(m.group(1) for m in re.finditer(r"^(_Z\d+gemm_bf16_wide_kernel\w+):", text, re.M))
    figures = {k: int(v) for k, v in re.findall(rf"\.set {name}\.(\w+), (\d+)", text)}
    assert figures["private_seg_size"] == 0, "the wide tile kernel spills registers"
    assert figures["num_agpr"] == 256 and figures["num_vgpr"] == 256
    body = text[text.index(f"{name}:"):]
    body = body[: body.index("s_endpgm")]
    outside = re.sub(r";;#ASMSTART.*?;;#ASMEND", "", body, flags=re.S)
    assert "v_mfma" in body and "v_mfma" not in outside, "matrix products outside the assembly statements"
    assert "accvgpr" not in outside and not re.search(r"\ba\[?\d", outside), "the compiler uses AGPRs of its own in the wide tile kernel"
