"""Compiles the GEMM kernels to gfx950 assembly (no GPU needed) and checks the hand-waited load
pipelines: no scratch memory, and no instruction touching a register whose load is still in flight."""
import os
import subprocess

import pytest

from isa_hazards import hazards, kernels, scratch_bytes

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "torch-tpu_amd", "csrc", "gemm_fp8.hip")


@pytest.fixture(scope="module")
def gemm_asm(tmp_path_factory):
    hipcc = "/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else "hipcc"
    out = tmp_path_factory.mktemp("isa") / "gemm_fp8.s"
    cmd = [hipcc, "--offload-arch=gfx950", "--cuda-device-only", "-O3", "-std=c++17", "-S",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", SRC, "-o", str(out)]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        pytest.fail("hipcc failed:\n" + r.stdout[-2000:])
    return out.read_text()


def test_checker_catches_a_planted_hazard():
    planted = """
	global_load_dwordx4 v[4:7], v2, s[0:1]
	v_mov_b32_e32 v9, v5
	s_waitcnt vmcnt(0)
	s_endpgm
"""
    assert hazards(planted)
    clean = planted.replace("v_mov_b32_e32 v9, v5\n\ts_waitcnt vmcnt(0)", "s_waitcnt vmcnt(0)\n\tv_mov_b32_e32 v9, v5")
    assert not hazards(clean)
    looped = """
.LBB0_1:
	s_waitcnt vmcnt(1)
	v_mov_b32_e32 v9, v5
	global_load_dwordx4 v[4:7], v2, s[0:1]
	global_load_dwordx4 v[12:15], v2, s[0:1]
	s_cbranch_scc1 .LBB0_1
	s_endpgm
"""
    assert hazards(looped)          # second trip reads v5 while only the older load has retired


def test_gemm_kernels_have_no_scratch_and_no_in_flight_register_use(gemm_asm):
    names = [n for n, _ in kernels(gemm_asm) if "grouped_gemm_kernel" in n]
    assert len(names) >= 10
    spills = {n: b for n, b in scratch_bytes(gemm_asm).items() if "grouped_gemm_kernel" in n and b}
    assert not spills, f"kernels spill to scratch: {spills}"
    for name, body in kernels(gemm_asm):
        if "grouped_gemm_kernel" not in name:
            continue
        assert "s_waitcnt vmcnt" in body and "global_load_lds_dwordx4" in body
        bad = hazards(body)
        assert not bad, f"{name}: {bad[:5]}"


@pytest.mark.parametrize("source", ["route.hip", "permute.hip", "quant_reduce.hip", "dense_small.hip", "decode_prep.hip",
                                    "router_front.hip", "probe.hip"])
def test_no_kernel_of_the_library_spills(source, tmp_path):
    """Every other kernel source: compiled to gfx950 assembly, no kernel may need scratch memory."""
    hipcc = "/opt/rocm/bin/hipcc" if os.path.exists("/opt/rocm/bin/hipcc") else "hipcc"
    out = tmp_path / (source + ".s")
    cmd = [hipcc, "--offload-arch=gfx950", "--cuda-device-only", "-O3", "-std=c++17", "-S", "-Wno-inline-asm",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           os.path.join(ROOT, "torch-tpu_amd", "csrc", source), "-o", str(out)]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        pytest.fail("hipcc failed:\n" + r.stdout[-2000:])
    sizes = scratch_bytes(out.read_text())
    assert sizes, "no kernel found"
    spills = {n: b for n, b in sizes.items() if b}
    assert not spills, f"kernels spill to scratch: {spills}"

