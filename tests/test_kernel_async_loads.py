"""The attention kernel loads the mask word and the Q rows with inline-assembly loads whose results arrive
asynchronously, and retires them with explicit `s_waitcnt vmcnt(n)` that count the loads still allowed in flight.  The
compiler knows nothing of that protocol: were it to copy or read one of those registers between the load and its wait
(it did once, when the wait was written into two branches), it would read stale data without any error.  This test
compiles the kernel to assembly and checks, for every instantiation, that no instruction touches an asynchronously
loaded register before a wait that is strict enough to have retired the load.  Host-side: needs hipcc, no GPU."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "int8-flash-attention-fmha-quantization_amd", "csrc", "fmha_i8_api.hip")

LOAD = re.compile(r"\s+global_load_(dword|dwordx4|lds_dwordx4)\s+(v\[(\d+):(\d+)\]|v(\d+)),")
WAIT = re.compile(r"\s+s_waitcnt\b.*vmcnt\((\d+)\)")


def _regs(line):
    used = set(int(x) for x in re.findall(r"\bv(\d+)\b", line))
    for a, b in re.findall(r"v\[(\d+):(\d+)\]", line):
        used |= set(range(int(a), int(b) + 1))
    return used


def _assembly(path, *extra):
    subprocess.run(["hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
                    "-packed-fp32-ops", "-S", "--cuda-device-only", *extra, "-o", path, SRC], check=True,
                   capture_output=True)
    text = open(path).read()
    funcs = re.split(r"\n(?=_ZN14fmha_i8_gfx95018fmha_i8_fwd_kernel[^\n]*:\s)", text)[1:]
    assert len(funcs) == 64
    return funcs


@pytest.fixture(scope="module")
def kernels(tmp_path_factory):
    return _assembly(str(tmp_path_factory.mktemp("asm") / "kernel.s"))


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_the_compiler_fuses_no_multiply_add_on_its_own(kernels, tmp_path):
    """The source pins floating-point contraction off and writes out every fma it wants, so the result bits do not
    depend on which products an optimiser fuses (hipcc's default is to fuse where it sees fit: two builds of the same
    arithmetic once differed in one output LSB of a few elements per thousand).  Compiled with contraction switched
    off on the command line, every kernel must come out the same instruction for instruction."""
    def stream(f):
        ops = []
        for line in f.split("\n")[1:]:
            t = line.split(";")[0].strip()
            if t.startswith("s_endpgm"):
                break
            if t and not t.startswith(".") and not t.endswith(":"):
                ops.append(re.sub(r"\.LBB\d+_\d+", "L", re.sub(r"_ZZN\w+", "SYM", t)))
        return ops
    pinned = _assembly(str(tmp_path / "kernel_off.s"), "-ffp-contract=off")
    for a, b in zip(kernels, pinned):
        assert a.split(":")[0] == b.split(":")[0]
        assert stream(a) == stream(b), a.split(":")[0]


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_no_read_of_an_asynchronously_loaded_register_before_its_wait(kernels):
    funcs = kernels
    checked = 0
    for f in funcs:
        name = f.split(":")[0]
        # template arguments <D, BK, BIAS, FASTACC, RAGGED, FULLP>; a RAGGED prologue has alternative load paths: weaker check
        ragged = re.search(r"ELb1ELb[01]EEEvNS_10KernelArgsE$", name) is not None
        lines = f.split("\n")
        issued = 0          # loads issued so far, in program order (they return in that order)
        pending = {}        # register -> (line of its load, ordinal of the load)
        waits = []          # (line, loads issued before it, count allowed in flight)
        for i, line in enumerate(lines):
            if "s_barrier" in line:
                break       # the mask word and Q are loaded, and first used, in front of the first barrier
            m = LOAD.match(line)
            if m:
                if m.group(1) != "lds_dwordx4":  # a load that returns into registers
                    regs = range(int(m.group(3)), int(m.group(4)) + 1) if m.group(3) else [int(m.group(5))]
                    for r in regs:
                        pending[r] = (i, issued)
                issued += 1
                continue
            w = WAIT.match(line)
            if w:
                waits.append((i, issued, int(w.group(1))))
                continue
            if re.match(r"\s+(v_|ds_|global_|buffer_|flat_)", line):
                for r in _regs(line) & set(pending):
                    at, ordinal = pending.pop(r)
                    ok = any(at < j < i and (ragged or before - allowed >= ordinal + 1) for j, before, allowed in waits)
                    assert ok, "%s: line %d `%s` touches v%d before its load has been waited for" % (
                        name, i, line.strip(), r)
                    checked += 1
    assert checked >= 32  # at least the mask word of every kernel (Q is first used behind the barrier: any touch of
    # it in front of the barrier, such as a copy, is what this test is looking for)
