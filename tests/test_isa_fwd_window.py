"""Checks on the compiled code of attn_fwd_window_kernel (hipcc cross-compiles without a GPU).

The kernel keeps all logits of a query block in registers (16 per 32-key block and lane) and is meant to run three
wavefronts per SIMD: that needs at most 168 registers per lane and no scratch memory.  Its maxima are written so that
the compiler can see them (the wait states after an MFMA are the compiler's to insert): they must come out as
v_max3_f32, and no inline assembly may read MFMA results.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "oregon_gpt_oss_patching_amd", "csrc")


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    return None


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    hipcc = _hipcc()
    if hipcc is None:
        pytest.skip("hipcc not found")
    from oregon_gpt_oss_patching_amd import build as B
    d = tmp_path_factory.mktemp("isa_fwd_window")
    src = d / "unit.hip"
    src.write_text('#include "%s"\n' % os.path.join(CSRC, "attn_fwd_window.h") +
                   "".join("template __global__ void gptoss::attn_fwd_window_kernel<%d>(const gptoss::KArgs);\n" % wh for wh in (1, 2, 3, 4)))
    out = d / "unit.s"
    flags = [f for f in B.HIPCC_FLAGS if f not in ("-fPIC", "-shared")]
    proc = subprocess.run([hipcc, *flags, "-S", "--cuda-device-only", "-o", str(out), str(src)], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    return out.read_text()


def test_three_wavefronts_per_simd_and_no_scratch(assembly):
    vgprs = [int(x) for x in re.findall(r"\.vgpr_count:\s+(\d+)", assembly)]
    agprs = [int(x) for x in re.findall(r"\.agpr_count:\s+(\d+)", assembly)]
    assert len(vgprs) == 4
    assert all(v + a <= 168 for v, a in zip(vgprs, agprs)), (vgprs, agprs)
    assert all(int(x) == 0 for x in re.findall(r"\.private_segment_fixed_size:\s+(\d+)", assembly))
    assert all(int(x) == 0 for x in re.findall(r"\.vgpr_spill_count:\s+(\d+)", assembly))
    lds = [int(x) for x in re.findall(r"\.group_segment_fixed_size:\s+(\d+)", assembly)]
    assert max(lds) <= 160 * 1024 // 3


def test_maxima_are_compiler_made(assembly):
    assert "v_max3_f32" in assembly
    assert "#APP" not in assembly          # no inline assembly in this kernel


def test_copies_are_waited_for_in_front_of_the_first_barrier(assembly):
    for kernel in assembly.split(".end_amdhsa_kernel")[:4]:
        lines = [x.strip() for x in kernel.split("\n")]
        first_barrier = next(i for i, x in enumerate(lines) if x.startswith("s_barrier"))
        last_copy = max(i for i, x in enumerate(lines) if x.startswith("global_load_lds_dwordx4"))
        assert last_copy < first_barrier
        assert any(re.match(r"s_waitcnt vmcnt\(0\)", x) for x in lines[last_copy:first_barrier])
