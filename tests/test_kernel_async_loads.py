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


def _blocks(func_text):
    """Basic blocks of one function of the assembly: name -> (instructions, successors).  A block ends at a label or
    after a branch; `s_branch` has no fall-through, `s_endpgm` has no successor."""
    blocks, order, cur = {}, [], "entry"
    blocks[cur] = []
    order.append(cur)
    for line in func_text.split("\n")[1:]:
        t = line.split(";")[0].rstrip()
        m = re.match(r"^(\.LBB\d+_\d+):", t)
        if m:
            cur = m.group(1)
            blocks[cur] = []
            order.append(cur)
            continue
        t = t.strip()
        if not t or t.startswith(".") or t.endswith(":"):
            continue
        blocks[cur].append(t)
        if t.startswith("s_endpgm"):
            break
        if re.match(r"s_c?branch", t):  # a branch ends the block: what follows is an anonymous fall-through block
            nxt = "%s+%d" % (cur, len(blocks[cur]))
            blocks[nxt] = []
            order.append(nxt)
            cur = nxt
    succ = {}
    for i, name in enumerate(order):
        ins = blocks[name]
        out = []
        last = ins[-1] if ins else ""
        m = re.match(r"(s_c?branch\w*)\s+(\.LBB\d+_\d+)", last)
        if m:
            out.append(m.group(2))
        if not last.startswith("s_branch") and not last.startswith("s_endpgm") and i + 1 < len(order):
            out.append(order[i + 1])
        succ[name] = out
    return blocks, succ, order


VMEM = re.compile(r"(global|buffer|flat)_(load|store|atomic)\w*")
REG_LOAD = re.compile(r"global_load_(dword|dwordx2|dwordx3|dwordx4|ubyte|sbyte|ushort|sshort)\s+(v\[(\d+):(\d+)\]|v(\d+)),")


def _check_function(name, text):
    """For every load that returns into registers: on EVERY path from the load, its registers are not mentioned by any
    instruction until an `s_waitcnt vmcnt(n)` has been passed with n <= the number of vector memory instructions issued
    on that path since the load (memory reads return in issue order).  A forward data-flow over the basic blocks with
    the state "fewest memory instructions issued since the load on any path to here"; a wait that is strict enough
    ends the path."""
    blocks, succ, order = _blocks(text)
    checked = 0
    for bname in order:
        for idx, ins in enumerate(blocks[bname]):
            m = REG_LOAD.match(ins)
            if not m:
                continue
            regs = set(range(int(m.group(3)), int(m.group(4)) + 1)) if m.group(3) else {int(m.group(5))}
            # the compiler's own loads are followed by its own waits; the hand-written ones are those it knows nothing
            # about - both kinds must satisfy the property, so both are checked
            best = {}  # block -> fewest instructions issued since the load at block entry
            work = []

            def run(block, start, k):
                for j in range(start, len(blocks[block])):
                    t = blocks[block][j]
                    w = WAIT.match("\t" + t)
                    if w and int(w.group(1)) <= k:
                        return None  # retired on this path
                    if re.match(r"(v_|ds_|global_|buffer_|flat_|s_)", t) and (_regs(t) & regs) and not t.startswith("s_waitcnt"):
                        raise AssertionError("%s: `%s` touches v%s before the load `%s` has been waited for" % (
                            name, t, sorted(_regs(t) & regs), ins))
                    if VMEM.match(t):
                        k += 1
                return min(k, 64)

            k = run(bname, idx + 1, 0)
            if k is not None:
                work = [(s_, k) for s_ in succ[bname]]
            while work:
                b, k = work.pop()
                if b in best and best[b] <= k:
                    continue
                best[b] = k
                out = run(b, 0, k)
                if out is not None:
                    work.extend((s_, out) for s_ in succ[b])
            checked += 1
    return checked


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_no_read_of_an_asynchronously_loaded_register_before_its_wait(kernels):
    checked = 0
    for f in kernels:
        checked += _check_function(f.split(":")[0], f)
    # at least the mask bytes and the Q rows (two or four loads) of every kernel
    assert checked >= 3 * len(kernels)


def test_the_checker_itself_finds_a_missing_wait():
    """A path on which the wait is too weak, and one on which a branch skips it."""
    ok = "f:\n\tglobal_load_dwordx4 v[2:5], v1, s[0:1]\n\tglobal_load_lds_dwordx4 v1, s[2:3]\n\ts_waitcnt vmcnt(1)\n\tv_mov_b32 v9, v2\n\ts_endpgm\n"
    assert _check_function("ok", ok) == 1
    weak = ok.replace("vmcnt(1)", "vmcnt(2)")
    with pytest.raises(AssertionError):
        _check_function("weak", weak)
    skipped = ("f:\n\tglobal_load_dwordx4 v[2:5], v1, s[0:1]\n\ts_cbranch_vccnz .LBB0_2\n\ts_waitcnt vmcnt(0)\n.LBB0_2:\n"
               "\tv_mov_b32 v9, v2\n\ts_endpgm\n")
    with pytest.raises(AssertionError):
        _check_function("skipped", skipped)
