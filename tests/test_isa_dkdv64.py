"""Checks on the compiled code of attn_bwd_dkdv64_kernel (hipcc cross-compiles without a GPU).

That kernel keeps its dK / dV accumulators in AGPRs through inline-assembly MFMAs, which the compiler's
hazard handling cannot see into.  Two hazards are therefore the kernel's own business, and this test
checks the compiled code for both, following every path of the control flow:

  * read after write: no instruction other than another inline-assembly MFMA touches the registers such
    an MFMA accumulates into for the next 20 wait states (an MFMA of this shape takes 8 passes; a copy the
    compiler places where two pieces of straight-line code meet, or a spill, would read the old value);
  * vector write, then MFMA read: none of the two instructions in front of an inline-assembly MFMA writes
    one of its operands, unless the MFMA is the form that starts with s_nop 1.

And for speed: inside the pipelined loop there is no scratch access (a spill there would also wait for, and
so drain, the asynchronous copies in flight), no AGPR copy, and no branch between the scheduling fences.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "oregon_gpt_oss_patching_amd", "csrc")
KERNEL = "attn_bwd_dkdv64_kernel"        # both instantiations are checked (with and without padded batch rows)


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    return None


@pytest.fixture(scope="module", params=[False, True], ids=["plain", "padded_rows"])
def kernel_asm(tmp_path_factory, request):
    hipcc = _hipcc()
    if hipcc is None:
        pytest.skip("hipcc not found")
    from oregon_gpt_oss_patching_amd import build as B
    d = tmp_path_factory.mktemp("isa")
    src = d / "unit.hip"
    padded = "true" if request.param else "false"
    src.write_text('#include "%s"\ntemplate __global__ void gptoss::attn_bwd_dkdv64_kernel<%s>(const gptoss::KArgs);\n'
                   % (os.path.join(CSRC, "attn_bwd_dkdv64.h"), padded))
    out = d / "unit.s"
    flags = [f for f in B.HIPCC_FLAGS if f not in ("-fPIC", "-shared")]
    proc = subprocess.run([hipcc, *flags, "-S", "--cuda-device-only", "-o", str(out), str(src)], capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    text = out.read_text()
    m = re.search(r"^(_ZN6gptoss\d+%s\w*):[^\n]*\n(.*?)\.end_amdhsa_kernel" % KERNEL, text, re.S | re.M)
    assert m, "kernel not found in the assembly"
    return m.group(2).split("\n"), text


def _agprs(code):
    regs = set()
    for m in re.finditer(r"\ba\[(\d+):(\d+)\]", code):
        regs |= set(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\ba(\d+)\b", code):
        regs.add(int(m.group(1)))
    return regs


def _instructions(lines):
    """(index, in_inline_asm, text) of every instruction line."""
    in_asm = False
    for i, line in enumerate(lines):
        t = line.strip()
        if t.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if not t or t.startswith(";") or t.startswith(".") or t.endswith(":"):
            continue
        yield i, in_asm, t.split(";")[0].strip()


def test_no_spills_and_full_register_file(kernel_asm):
    _, text = kernel_asm
    meta = text[text.index("amdhsa.kernels"):]
    entries = [e for e in meta.split("\n  - ") if re.search(r"\.name:\s+\S*%s" % KERNEL, e)]
    assert len(entries) == 1
    blk = entries[0]
    # one wavefront per SIMD: beyond 256 registers the second half of the file is in use, and nothing
    # went to scratch memory
    assert int(re.search(r"\.vgpr_count:\s+(\d+)", blk).group(1)) > 256
    assert int(re.search(r"\.agpr_count:\s+(\d+)", blk).group(1)) >= 128
    assert int(re.search(r"\.vgpr_spill_count:\s+(\d+)", blk).group(1)) == 0
    lines, _ = kernel_asm
    assert not [x for x in lines if re.search(r"\b(scratch|buffer)_(load|store)", x)], "the kernel touches scratch memory"


def _regs(code, kind):
    regs = set()
    for m in re.finditer(r"\b%s\[(\d+):(\d+)\]" % kind, code):
        regs |= set((kind, r) for r in range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"\b%s(\d+)\b" % kind, code):
        regs.add((kind, int(m.group(1))))
    return regs


def _program(lines):
    """Instruction list [(code, asm_group)] with successor indices; asm_group numbers the inline-assembly
    statement an instruction belongs to (None for compiler-generated code)."""
    prog, labels, group, n_group = [], {}, None, 0
    for line in lines:
        t = line.strip()
        if t.startswith(";;#ASMSTART"):
            n_group += 1
            group = n_group
            continue
        if t.startswith(";;#ASMEND"):
            group = None
            continue
        m = re.match(r"^(\.LBB\d+_\d+):", t)
        if m:
            labels[m.group(1)] = len(prog)
            continue
        if not t or t.startswith(";") or t.startswith("."):
            continue
        prog.append((t.split(";")[0].strip(), group))
    succ = []
    for i, (code, _) in enumerate(prog):
        op = code.split()[0]
        if op == "s_endpgm":
            succ.append([])
        elif op == "s_branch":
            succ.append([labels[code.split()[1]]])
        elif op.startswith("s_cbranch"):
            succ.append([labels[code.split()[1]], i + 1])
        else:
            succ.append([i + 1] if i + 1 < len(prog) else [])
    return prog, succ


def _wait_states(code):
    m = re.match(r"s_nop\s+(\d+)", code)
    return int(m.group(1)) + 1 if m else 1


def test_accumulators_are_left_alone_until_their_mfma_has_finished(kernel_asm):
    lines, _ = kernel_asm
    prog, succ = _program(lines)
    asm_mfma = [i for i, (code, g) in enumerate(prog) if g is not None and code.startswith("v_mfma")]
    assert len(asm_mfma) >= 32 + 8 + 24
    for i in asm_mfma:
        dst = _regs(prog[i][0].split()[1].rstrip(","), "a")
        assert len(dst) == 16
        # every path from here, 20 wait states deep
        seen, todo = {}, [(j, 20) for j in succ[i]]
        while todo:
            j, left = todo.pop()
            if left <= 0 or seen.get(j, -1) >= left:
                continue
            seen[j] = left
            code, g = prog[j]
            if not (g is not None and code.startswith("v_mfma")):
                assert not (_regs(code, "a") & dst), (prog[i][0], "then, %d wait states later:" % (20 - left), code)
            left -= _wait_states(code)
            todo += [(n, left) for n in succ[j]]


def test_no_vector_write_right_in_front_of_an_inline_assembly_mfma(kernel_asm):
    lines, _ = kernel_asm
    prog, _ = _program(lines)
    for i, (code, g) in enumerate(prog):
        if g is None or not code.startswith("v_mfma"):
            continue
        if i > 0 and prog[i - 1][1] == g and prog[i - 1][0].startswith("s_nop 1"):
            continue
        ops = [x.strip() for x in code.split(None, 1)[1].split(",")]
        srcs = set()
        for o in ops[1:]:
            srcs |= _regs(o, "v") | _regs(o, "a")
        for back in (1, 2):
            if i - back < 0:
                break
            pcode, pg = prog[i - back]
            if pg is not None and pcode.startswith("v_mfma"):
                continue                                     # MFMA to MFMA is interlocked by the hardware
            if pcode.startswith(("v_", "ds_read", "global_load", "scratch_load")):
                pdst = pcode.split(None, 1)[1].split(",")[0]
                assert not ((_regs(pdst, "v") | _regs(pdst, "a")) & srcs), (pcode, "right in front of", code)


def test_pipelined_loops_have_no_scratch_access_and_no_inner_branches(kernel_asm):
    """Two innermost loops (inside the loop over the two phases of a walk): masked tiles and interior tiles.  A tile is 64 MFMAs plus up to 8 for
    the statistics steps (the compiler shares those between the two key blocks of a row block where it can,
    and drops work on blocks of the diagonal tile that it can prove invisible)."""
    lines, _ = kernel_asm
    hdr = [i for i, line in enumerate(lines) if "Inner Loop Header" in line]
    hdr = [h for h in hdr if sum("v_mfma" in x for x in lines[h:h + 400]) > 8]       # the loops that compute
    assert len(hdr) == 2, hdr
    for h in hdr:
        label = None
        for j in range(h, 0, -1):
            m = re.match(r"^(\.LBB\d+_\d+):", lines[j])
            if m:
                label = m.group(1)
                break
        back = [i for i, line in enumerate(lines) if re.search(r"s_c?branch\w*\s+%s\b" % re.escape(label), line) and i > h]
        assert back, "no back edge found"
        body = lines[h:back[-1] + 1]
        assert 56 <= sum("v_mfma" in x for x in body) <= 72, "one tile per pass of the loop"
        assert not [x for x in body if "scratch_" in x], "spill inside a pipelined loop"
        fences = [i for i, x in enumerate(body) if "sched_barrier" in x]
        inner = body[fences[0]:fences[-1]]
        assert not [x for x in inner if re.search(r"\bs_cbranch|\bs_branch", x)], "branch between the scheduling fences of the loop body"
        # The accumulators (the AGPRs the inline-assembly MFMAs write) are never copied inside a loop; the compiler
        # may park a few ordinary values in the AGPRs beyond them and fetch them back (one instruction each).
        acc = set()
        for x in lines:
            if "v_mfma" in x and re.match(r"\s*v_mfma\S*\s+a\[", x):
                acc |= _agprs(x.split()[1])
        copies = [x for x in body if re.search(r"\bv_accvgpr_(mov|read|write)", x)]
        assert len(copies) <= 8, copies
        for x in copies:
            assert "v_accvgpr_mov" not in x and not (_agprs(x) & acc), ("an accumulator is copied inside a pipelined loop", x)
