"""Static checks of the device assembly of the kernels that issue vector-memory loads by hand.

The streaming GEMV kernels put activation loads in flight with inline assembly and wait for them later, so
that weight loads can be queued behind them.  The compiler treats such a statement as complete where it
stands, and its hazard recogniser does not look inside it.  Two things then depend on register assignment,
not on the source, and a change of either turns a correct kernel into one that reads a wild address:

  * a vector-memory instruction must not read a scalar register within five wait states of a vector
    instruction writing it (v_readlane restoring a spilled scalar, v_readfirstlane, v_cmp into a scalar
    pair): a build of q4k_gemv_rows_kernel under scalar-register pressure had `v_readlane_b32 s37, ..`
    directly in front of a hand-written `global_load_dwordx4 .., s[36:37]` and faulted the GPU;
  * between a hand-written load and the `s_waitcnt vmcnt` that retires it nothing may read or write the
    load's destination registers (a copy or a reuse would race with the data landing).

Both are checked here on the assembly hipcc emits for gfx950 (device pass only, a few seconds).  The first
check runs in program order and starts over at every label, so it can miss a hazard across a branch but
never reports a false one; the second is a data-flow analysis over the kernels' control-flow graphs.
"""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "doppler_amd", "csrc")
SOURCES = ["q4k_gemv_rows.hip", "q4k_gemv_i8.hip", "q4k_gemv_chain.hip"]
VMEM_PREFIXES = ("global_", "buffer_", "flat_", "scratch_")
SREG = re.compile(r"\bs(\d+)\b|\bs\[(\d+):(\d+)\]")
VREG = re.compile(r"\bv(\d+)\b|\bv\[(\d+):(\d+)\]")


def _regs(rx, text):
    out = set()
    for m in rx.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            out.update(range(int(m.group(2)), int(m.group(3)) + 1))
    return out


def _instructions(path):
    """(line number, text, inside inline asm, kernel) of every instruction; labels come as text ending in ':'."""
    kernel, in_asm = None, False
    for ln, line in enumerate(open(path), 1):
        if "#ASMSTART" in line:
            in_asm = True
            continue
        if "#ASMEND" in line:
            in_asm = False
            continue
        s = line.split(";")[0].strip()
        if not s or s.startswith("."):
            if s.endswith(":"):
                yield ln, s, in_asm, kernel          # a local label
            continue
        if s.endswith(":"):
            kernel = s[:-1]
        yield ln, s, in_asm, kernel


def scalar_operand_hazards(path):
    hits, hist = [], []
    for ln, s, in_asm, kernel in _instructions(path):
        if s.endswith(":"):
            hist = []
            continue
        op, _, args = s.partition(" ")
        if in_asm and op.startswith(VMEM_PREFIXES):
            used, states = _regs(SREG, args), 0
            for pln, ps, pop, pdst in reversed(hist):
                if states >= 5:
                    break
                if pdst & used:
                    hits.append("%s line %d: `%s` reads a scalar register written %d wait states earlier by `%s` (line %d)"
                                % (kernel, ln, s, states, ps, pln))
                states += int(ps.split()[1], 0) + 1 if pop == "s_nop" else 1
        dst = _regs(SREG, args.split(",")[0]) if op.startswith("v_") and args else set()
        hist = (hist + [(ln, s, op, dst)])[-8:]
    return hits


def _vmcnt(ins):
    m = re.search(r"vmcnt\((\d+)\)", ins)
    if m:
        return int(m.group(1))
    m = re.match(r"s_waitcnt\s+(0x[0-9a-f]+|\d+)$", ins)
    if m:
        v = int(m.group(1), 0)
        return (v & 0xF) | (((v >> 14) & 3) << 4)
    return None


def in_flight_destination_hazards(path):
    """Forward data-flow over the control-flow graph of every kernel.  State: the hand-written loads that are
    in flight on EVERY path to this point, i.e. issued with no wait on the vector-memory counter since (a
    join keeps what both sides hold).  The kernels choose the count of their waits at run time, a switch
    that compiles into a tree of branches around single s_waitcnt instructions; an analysis that follows
    every path of that tree sees one that skips all of them, hence the intersection: it can miss a hazard
    that exists on one side of a branch only, and never reports a false one.  That a wait's count is right
    shows in the results (a short wait yields wrong numbers, which the parity tests see); what cannot show
    there reliably is the window from a load to its wait, which is straight-line code and fully covered."""
    ins = list(_instructions(path))
    label_at = {s[:-1]: i for i, (_, s, _, _) in enumerate(ins) if s.endswith(":")}
    hits, hand_loads = {}, 0

    def successors(i):
        s = ins[i][1]
        op, _, args = s.partition(" ")
        if op == "s_endpgm":
            return []
        nxt = [i + 1] if i + 1 < len(ins) else []
        if op == "s_branch":
            return [label_at[args.strip()]]
        if op.startswith("s_cbranch"):
            return nxt + [label_at[args.strip()]]
        return nxt

    starts = [i for i, (_, s, _, _) in enumerate(ins) if s.endswith(":") and not s.startswith(".L")]
    state_in = {i: frozenset() for i in starts}
    work = list(starts)
    while work:
        i = work.pop()
        st = set(state_in[i])
        ln, s, in_asm, kernel = ins[i]
        if not s.endswith(":"):
            op, _, args = s.partition(" ")
            if op == "s_waitcnt":
                n = _vmcnt(s)
                if n is not None and n < 63:
                    st = set()
            elif in_asm and op.startswith(VMEM_PREFIXES) and "_load_" in op and "lds" not in op:
                st.add((ln, s, tuple(sorted(_regs(VREG, args.split(",")[0])))))
        st = frozenset(st)
        for j in successors(i):
            old = state_in.get(j)
            new = st if old is None else old & st
            if new != old:
                state_in[j] = new
                work.append(j)
    # the states have settled: now look at what every instruction touches
    for i, (ln, s, in_asm, kernel) in enumerate(ins):
        if s.endswith(":") or i not in state_in:
            continue
        op, _, args = s.partition(" ")
        if in_asm and op.startswith(VMEM_PREFIXES) and "_load_" in op and "lds" not in op:
            hand_loads += 1
        if op == "s_waitcnt":
            continue
        touched = _regs(VREG, args)
        for pln, ps, dst in state_in[i]:
            if touched & set(dst):
                hits[(ln, pln)] = ("%s line %d: `%s` touches v%s while `%s` (line %d) is in flight"
                                   % (kernel, ln, s, sorted(touched & set(dst)), ps, pln))
    return [hits[k] for k in sorted(hits)], hand_loads


@pytest.fixture(scope="module")
def assembly():
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not available")
    d = tempfile.mkdtemp(prefix="doppler_amd_asm_")
    procs = []
    for src in SOURCES:
        out = os.path.join(d, src.replace(".hip", ".s"))
        cmd = [hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-I" + CSRC, "-I" + os.path.join(ROOT, "include"),
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-S",
               os.path.join(CSRC, src), "-o", out]
        procs.append((src, out, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)))
    paths = {}
    for src, out, p in procs:
        _, err = p.communicate(timeout=600)
        assert p.returncode == 0, err[-2000:]
        paths[src] = out
    yield paths
    shutil.rmtree(d, ignore_errors=True)


@pytest.mark.parametrize("src", SOURCES)
def test_no_scalar_register_hazard_in_front_of_hand_written_loads(assembly, src):
    assert scalar_operand_hazards(assembly[src]) == []


@pytest.mark.parametrize("src", SOURCES)
def test_destinations_of_hand_written_loads_are_left_alone_until_their_wait(assembly, src):
    hits, hand_loads = in_flight_destination_hazards(assembly[src])
    assert hand_loads > 0, "the scan found no hand-written load in %s: the parser no longer matches the assembly" % src
    assert hits == []


@pytest.mark.parametrize("src", SOURCES)
def test_no_scratch_memory_in_the_streaming_kernels(assembly, src):
    """Scratch loads and stores are vector-memory operations: the compiler waits for them with vmcnt(0), i.e.
    for the weight load in flight too, once per use (an array indexed by a loop counter did that at every
    tile end of the two-row int8 kernel).  Only the scalar-load fallback of the few-row kernel (rows that
    cannot be loaded four elements at a time) may spill."""
    used = {}
    for _, s, _, kernel in _instructions(assembly[src]):
        if s.startswith("scratch_"):
            used[kernel] = used.get(kernel, 0) + 1
    allowed = ("q4k_gemv_rows_kernelILb0ELb0E", "q4k_gemv_rows_kernelILb1ELb0E")
    assert {k: v for k, v in used.items() if not any(a in k for a in allowed)} == {}


def test_the_scans_see_what_they_look_for(tmp_path):
    """The assembly of the build that faulted, reduced to the lines that matter, and a register reuse."""
    bad = tmp_path / "bad.s"
    bad.write_text("\n".join([
        "kernel_a:", "\tv_readlane_b32 s36, v127, 0", "\tv_mfma_f32_16x16x32_f16 v[48:51], v[16:19], v[48:51], 0",
        "\tv_min_i32_e32 v16, s17, v76", "\tv_add_lshl_u32 v77, v16, v66, 2", "\tv_readlane_b32 s37, v127, 1",
        "\t;;#ASMSTART", "\tglobal_load_dwordx4 v[16:19], v77, s[36:37]", "\t;;#ASMEND",
        "\tv_mov_b32_e32 v17, 0", "\ts_waitcnt vmcnt(0)", "\tv_mov_b32_e32 v18, 0", "\ts_endpgm", ""]))
    hits = scalar_operand_hazards(str(bad))
    assert len(hits) == 2 and "written 0 wait states earlier by `v_readlane_b32 s37" in hits[0], hits
    hits, n = in_flight_destination_hazards(str(bad))
    assert n == 1 and len(hits) == 1 and "v_mov_b32_e32 v17" in hits[0], hits
    good = tmp_path / "good.s"
    good.write_text(bad.read_text().replace("\tglobal_load_dwordx4", "\ts_nop 4\n\tglobal_load_dwordx4").replace(
        "\tv_mov_b32_e32 v17, 0\n", ""))
    assert scalar_operand_hazards(str(good)) == []
    assert in_flight_destination_hazards(str(good))[0] == []
