"""Static check of the compiled decoding-wave kernels: no instruction touches a register that an untracked load still owns.

The kernels in csrc/mmq_small_iq2.h, csrc/mmq_direct8.h and csrc/mmq_direct8_nn.h request packed bytes several steps ahead
with inline-asm loads the compiler does not track, and wait for them with exact `s_waitcnt vmcnt` counts.  The compiler
is free to copy such a register (a loop-carried copy at the back edge, a hoisted read) while its load is still on its
way, which copies stale data and loses the load's result: wrong numbers without any fault.  This test compiles the three
kernels to gfx950 assembly and replays every loop body twice against the in-order queue of vector-memory operations:
between an inline-asm load into a VGPR and the wait that retires it, no instruction may name that VGPR.  It also checks
that the loops hold no scratch (spill) traffic, which would drain the queue through compiler-made waits.

It also guards the compiler's own LDS waits.  A load through a pointer selected between LDS and global memory is a flat
load; the compiler never sees these kernels' inline-asm `vmcnt` waits, so it takes such a load for outstanding through
every later loop iteration and, unable to count LDS returns past it, drains ALL of a wave's LDS reads (`lgkmcnt(0)`) where
it needs the oldest of them: in front of the first MFMA of every sub-step.  The kernels must hold no flat memory
instruction, and the Q4_K main loops must wait for their LDS operands with exact counts.
"""
import pathlib
import re
import shutil
import subprocess

import pytest

CSRC = pathlib.Path(__file__).resolve().parents[1] / "transformers5-qwen3.5-recipe_amd" / "csrc"
KERNELS = {
    "mmq_small_iq2xxs_kernel": "mmq_small_iq2.h",
    "mmq_direct8_q4k_kernel": "mmq_direct8.h",
    "mmq_direct8_nn_q4k_kernel": "mmq_direct8_nn.h",
}
VMEM = re.compile(r"^(global_load|global_store|global_atomic|buffer_load|buffer_store|scratch_load|scratch_store|flat_load|flat_store)")
REG = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")


def _regs(text):
    out = set()
    for m in REG.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return out


def _instructions(body):
    """[(text, in_asm)] of a function body, comments and directives dropped."""
    out, in_asm = [], False
    for line in body.split("\n"):
        t = line.strip()
        if t.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if t.startswith(";;#ASMEND"):
            in_asm = False
            continue
        t = t.split(";")[0].strip()
        if not t or t.startswith(".") and not t.startswith(".LBB"):
            continue
        out.append((t, in_asm))
    return out


def _loops(instrs, inner_trips=1):
    """Loops that issue MFMAs: (label, [instructions from the label to its last back edge], innermost).  The body of an
    outer loop holds every loop nested in it `inner_trips` times over: the fewest iterations such a loop makes."""
    labels = {t[:-1]: i for i, (t, _) in enumerate(instrs) if t.startswith(".LBB") and t.endswith(":")}
    spans = {}
    for lab, start in labels.items():
        ends = [i for i, (t, _) in enumerate(instrs) if i > start and re.match(r"s_c?branch\w* " + re.escape(lab) + r"$", t)]
        if ends:
            spans[lab] = (start, ends[-1])

    def unrolled(start, end):  # instructions start .. end - 1, nested loops repeated
        out, i = [], start
        nested = sorted((s0, e0) for s0, e0 in spans.values() if start <= s0 and e0 < end)
        while i < end:
            hit = next(((s0, e0) for s0, e0 in nested if s0 == i), None)
            if hit:
                for _ in range(inner_trips):
                    out += unrolled(hit[0] + 1, hit[1] + 1)
                i = hit[1] + 1
            else:
                out.append(instrs[i])
                i += 1
        return out

    found = []
    for lab, (start, end) in spans.items():
        if sum(t.startswith("v_mfma") for t, _ in instrs[start + 1 : end]) >= 8:
            innermost = not any(o != lab and start < s0 and e0 < end for o, (s0, e0) in spans.items())
            found.append((lab, unrolled(start + 1, end), innermost))
    return found


def _replay(body):
    """Violations of a loop body replayed twice: instructions that name a VGPR whose inline-asm load has not been retired."""
    queue, bad = [], []  # queue: destination registers of each outstanding vector-memory operation (empty set: nothing to guard)
    for rep in range(2):
        for text, in_asm in body:
            op = text.split()[0]
            m = re.search(r"vmcnt\((\d+)\)", text)
            if op == "s_waitcnt" and m:
                keep = int(m.group(1))
                queue = queue[len(queue) - keep :] if keep < len(queue) else queue
                continue
            named = _regs(text)
            owned = set().union(*queue) if queue else set()
            if named & owned:
                bad.append((rep, text, sorted(named & owned)))
            if VMEM.match(op):
                guarded = set()
                if in_asm and op.startswith("global_load") and "_lds_" not in op:
                    guarded = _regs(text.split(",")[0])  # the destination is the first operand
                queue.append(guarded)
    return bad


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not pathlib.Path(hipcc).exists():
        pytest.skip("hipcc is not installed")
    tmp = tmp_path_factory.mktemp("isa")
    src = tmp / "decoding_wave_kernels.hip"
    src.write_text("".join(f'#include "{h}"\n' for h in sorted(set(KERNELS.values()))))
    out = tmp / "decoding_wave_kernels.s"
    cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", f"-I{CSRC}", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-S", "--cuda-device-only", str(src), "-o", str(out)]
    done = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    return out.read_text()


@pytest.mark.parametrize("kernel", sorted(KERNELS))
def test_no_instruction_names_a_register_a_load_still_owns(assembly, kernel):
    m = re.search(r"^(_ZN3ggq\d+" + kernel + r"\w*):", assembly, re.M)
    assert m, f"{kernel} is not in the assembly"
    body = assembly[m.end() : assembly.index(".Lfunc_end", m.end())]
    # the grad-input kernel's step loop takes two steps per iteration, and the host launches it for four steps or more
    loops = _loops(_instructions(body), inner_trips=2 if kernel == "mmq_direct8_nn_q4k_kernel" else 1)
    assert loops, f"{kernel}: no MFMA loop found"
    assert any(inner for _, _, inner in loops)
    for label, loop, innermost in loops:
        if innermost:
            assert not any(t.startswith("scratch_") for t, _ in loop), f"{kernel} {label}: spill traffic inside the loop"
        bad = _replay(loop)
        assert not bad, f"{kernel} {label}: {bad[:5]}"


def test_the_replay_flags_a_copy_of_a_register_in_flight():
    loop = [("global_load_dwordx2 v[10:11], v1, s[2:3]", True), ("v_mov_b32_e32 v20, v10", False), ("s_waitcnt vmcnt(0)", True), ("v_add_u32_e32 v3, v10, v11", False)]
    bad = _replay(loop)
    assert [b[1] for b in bad] == ["v_mov_b32_e32 v20, v10", "v_mov_b32_e32 v20, v10"]
    ok = [("global_load_dwordx2 v[10:11], v1, s[2:3]", True), ("global_load_lds_dwordx4 v1, s[2:3]", True), ("s_waitcnt vmcnt(1)", True), ("v_mov_b32_e32 v20, v10", False)]
    assert not _replay(ok)


@pytest.mark.parametrize("kernel", sorted(KERNELS))
def test_no_flat_memory_instruction(assembly, kernel):
    m = re.search(r"^(_ZN3ggq\d+" + kernel + r"\w*):", assembly, re.M)
    body = assembly[m.end() : assembly.index(".Lfunc_end", m.end())]
    flat = [t for t, _ in _instructions(body) if re.match(r"flat_(load|store|atomic)", t)]
    assert not flat, f"{kernel}: {flat[:3]}"


@pytest.mark.parametrize("kernel", ["mmq_direct8_q4k_kernel", "mmq_direct8_nn_q4k_kernel"])
def test_main_loops_wait_for_lds_operands_with_exact_counts(assembly, kernel):
    """In the inner loops of the tile variants with two or more row blocks, a compiler-made `lgkmcnt(0)` stands only in
    front of the step barrier (the kernels' own wait), never in front of an MFMA."""
    m = re.search(r"^(_ZN3ggq\d+" + kernel + r"\w*):", assembly, re.M)
    body = assembly[m.end() : assembly.index(".Lfunc_end", m.end())]
    checked = 0
    for label, loop, innermost in _loops(_instructions(body)):
        texts = [t for t, _ in loop]
        mfmas = sum(t.startswith("v_mfma") for t in texts)
        if not innermost or mfmas < 32:  # one-block tiles read each operand one sub-step ahead: nothing newer is in flight behind it
            continue
        drains = [b for a, b in zip(texts, texts[1:]) if a.startswith("s_waitcnt") and "lgkmcnt(0)" in a and b.startswith("v_mfma")]
        assert not drains, f"{kernel} {label}: {len(drains)} of {mfmas} MFMAs wait for every LDS read"
        checked += 1
    assert checked >= 3
