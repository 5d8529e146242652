"""Checks on the compiled code of attn_fwd_pipe_kernel (hipcc cross-compiles without a GPU).

The kernel's interior-tile loop is scheduled by hand: four slots of eight micro-slots, one MFMA each, closed by
scheduling fences, with the tile copies hidden from the compiler in inline assembly.  What the source cannot
guarantee by itself is checked here on the ISA: every micro-slot of the loop got its MFMA (instruction selection
likes to move an MFMA whose result is not needed yet across the fences), the loop touches no scratch memory, and
the only wait on the vector-memory counter inside it is the kernel's own (a compiler-made `vmcnt` wait there would
also wait for the copies in flight, i.e. for the tile that was just requested).
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "oregon_gpt_oss_patching_amd", "csrc")
KERNEL = "attn_fwd_pipe_kernel"        # both instantiations are checked (with and without padded batch rows)


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    return None


@pytest.fixture(scope="module", params=[False, True], ids=["plain", "padded_rows"])
def kernel_lines(tmp_path_factory, request):
    hipcc = _hipcc()
    if hipcc is None:
        pytest.skip("hipcc not found")
    from oregon_gpt_oss_patching_amd import build as B
    d = tmp_path_factory.mktemp("isa_fwd")
    src = d / "unit.hip"
    src.write_text('#include "%s"\ntemplate __global__ void gptoss::attn_fwd_pipe_kernel<%s>(const gptoss::KArgs);\n'
                   % (os.path.join(CSRC, "attn_fwd_pipe.h"), "true" if request.param else "false"))
    out = d / "unit.s"
    flags = [f for f in B.HIPCC_FLAGS if f not in ("-fPIC", "-shared")]
    proc = subprocess.run([hipcc, *flags, "-S", "--cuda-device-only", "-o", str(out), str(src)], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    text = out.read_text()
    m = re.search(r"^(_ZN6gptoss\d+%s\w*):[^\n]*\n(.*?)\.end_amdhsa_kernel" % KERNEL, text, re.S | re.M)
    assert m, "kernel not found in the assembly"
    return m.group(2).split("\n")


def _pipelined_loop(lines):
    """The innermost loop with one tile's 32 MFMAs."""
    found = []
    for h in [i for i, line in enumerate(lines) if "Inner Loop Header" in line]:
        label = None
        for j in range(h, 0, -1):
            m = re.match(r"^(\.LBB\d+_\d+):", lines[j])
            if m:
                label = m.group(1)
                break
        back = [i for i, line in enumerate(lines) if re.search(r"s_c?branch\w*\s+%s\b" % re.escape(label), line) and i > h]
        if not back:
            continue
        body = lines[h:back[-1] + 1]
        if sum("v_mfma" in x for x in body) == 32 and sum("sched_barrier" in x for x in body) >= 32:
            found.append(body)
    assert len(found) == 1, "expected exactly one hand-scheduled loop of 32 MFMAs"
    return found[0]


def test_every_micro_slot_of_the_loop_has_its_mfma(kernel_lines):
    body = _pipelined_loop(kernel_lines)
    groups, cur = [], []
    for x in body:
        if "sched_barrier" in x:
            groups.append(cur)
            cur = []
            continue
        t = x.strip()
        if t and not t.startswith((";", ".")) and not t.endswith(":"):
            cur.append(t.split(";")[0].strip())
    groups.append(cur)
    with_mfma = [g for g in groups if any(i.startswith("v_mfma") for i in g)]
    assert len(with_mfma) == 32 and all(sum(i.startswith("v_mfma") for i in g) == 1 for g in with_mfma)
    # the softmax work is spread over them: no group carries more than a few exponentials
    assert max(sum(i.startswith("v_exp") for i in g) for g in groups) <= 4
    assert sum(i.startswith("v_exp") for g in groups for i in g) == 64


def test_loop_has_no_scratch_access_and_no_compiler_made_vmcnt_wait(kernel_lines):
    body = _pipelined_loop(kernel_lines)
    assert not [x for x in body if re.search(r"\b(scratch|buffer)_(load|store)", x)], "spill inside the pipelined loop"
    waits = [x.strip().split(";")[0].strip() for x in body if "s_waitcnt" in x and "vmcnt" in x]
    assert waits == ["s_waitcnt vmcnt(4)"], waits          # the kernel's own: one request (4 copies) may stay in flight
    assert sum("global_load_lds_dwordx4" in x for x in body) == 4
    assert sum("s_barrier" in x for x in body) == 1
