"""The 256 x 256 tile product keeps its 256 accumulators in AGPRs that only its assembly statements
name: between the loop and the reads of the accumulators the compiler must not touch them. It has no
reason to (no matrix builtins in that kernel, nothing spilled), and this test holds it to that: the kernel's
device assembly, made here with the build's own flags, uses no scratch memory, all 256 AGPRs, and has no
AGPR instruction outside the assembly statements. The attention kernels are written to fit the registers
of two waves per SIMD (the widest merged projection holds 256 registers of weights and moves the rest through
the accumulation registers): none of them may start to spill unnoticed either. No GPU is needed: hipcc
cross-compiles."""

from __future__ import annotations

import re
import shutil
import subprocess

import pytest

from miniserve_amd.kernels import build


def device_assembly(folder, source: str) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not shutil.which(hipcc):
        pytest.skip("no hipcc")
    out = folder / (source + ".s")
    flags = [f for f in build.HIP_FLAGS if f != "-fPIC"]
    subprocess.run([hipcc, *flags, "--cuda-device-only", "-S", "-o", str(out), str(build.CSRC / (source + ".hip"))],
                   check=True, capture_output=True, timeout=300)
    return out.read_text()


def scratch_bytes(text: str) -> dict[str, int]:
    """Scratch memory per lane of every kernel in a file's device assembly, by mangled name."""
    return {name: int(v) for name, v in re.findall(r"\.set (_Z\w+)\.private_seg_size, (\d+)", text)}


@pytest.fixture(scope="module")
def gemm_assembly(tmp_path_factory):
    return device_assembly(tmp_path_factory.mktemp("asm"), "gemm_bf16")


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


def test_attention_kernels_keep_to_their_registers(tmp_path):
    decode = scratch_bytes(device_assembly(tmp_path, "attention_decode"))
    assert any("attn_decode_split_kernel" in k for k in decode) and any("attn_merge_project_kernelILi128ELi4ELi4E" in k for k in decode)
    assert not {k: v for k, v in decode.items() if v}, "a decode attention kernel spills registers"
    prefill = scratch_bytes(device_assembly(tmp_path, "attention_prefill"))
    wide = [k for k in prefill if "attn_prefill_kernelILi128ELi2ELi1E" in k or "attn_prefill_kernelILi64ELi2ELi1E" in k]
    assert len(wide) == 2 and all(prefill[k] == 0 for k in wide), "a 128-row prefill attention kernel spills registers"
    # the 64-row form at head size 128 parks four values outside its loop: no more than that
    assert max(prefill.values()) <= 16, {k: v for k, v in prefill.items() if v > 16}
