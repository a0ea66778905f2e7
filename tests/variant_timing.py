#!/usr/bin/env python3
"""Times one build of the library on one benchmark configuration (a measurement tool, not a test).

    make -C tests variants
    python tests/variant_timing.py --lib tests/bin/libfmha_i8_ko_softmax.so --workload C3
    rocprofv3 --pmc SQ_INSTS_VALU SQ_INSTS_SALU SQ_INSTS_LDS SQ_WAIT_ANY ... -- python3 tests/variant_timing.py --lib ... --calls 50

The test builds (tests/Makefile, target `variants`) each remove or change one thing in the attention kernel - no softmax,
no MFMA phase, no LDS operand reads, no tile loads, no LDS swizzle - so that what every piece costs can be re-measured;
their results are garbage on purpose, and only the build called `few` (the shipped kernel with fewer instantiations) and
`no_swizzle` are checked against the shipped library here.  With a `trace_ticks` build the per-wavefront time stamps
of the barriers are read back and summarised: how long a wavefront works between two barriers and how long it waits.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--lib", default=None, help="library to time (default: the shipped libfmha_i8.so)")
    ap.add_argument("--workload", default="C3", choices=["C1", "C2", "C3", "C4", "C5"])
    ap.add_argument("--calls", type=int, default=1000)
    ap.add_argument("--preheat-ms", type=float, default=100.0)
    ap.add_argument("--compare", action="store_true", help="compare the output bytes with the shipped library's")
    args = ap.parse_args()

    import numpy as np
    import torch
    import __graft_entry__ as g
    import fmha_cases as fc

    pkg = g.load_package()
    shipped = pkg.load_library()
    path = os.path.abspath(args.lib) if args.lib else None
    lib = C.CDLL(path) if path else shipped
    lib.FMHAInferI8Status.argtypes = [C.c_void_p, pkg.FMHAParamI8, pkg.AttnDataDescriptor] + [C.c_void_p] * 5 + [C.c_bool]
    lib.FMHAInferI8Status.restype = C.c_int
    dev = torch.device("cuda:0")
    c = fc.make_config(args.workload)
    B, H, S, d = c["q"].shape
    q, k, v, m = (torch.from_numpy(c[n]).to(dev) for n in ("q", "k", "v", "mask"))
    o = torch.zeros_like(q)
    P = pkg.FMHAParamI8(c["q_amax"], c["k_amax"], c["v_amax"], c["o_amax"], 1.0)
    A = pkg.AttnDataDescriptor(B, S, H, d)
    stream = torch.cuda.current_stream(dev)
    call = (stream.cuda_stream, P, A, q.data_ptr(), k.data_ptr(), v.data_ptr(), m.data_ptr(), o.data_ptr(), True)

    def step():
        st = lib.FMHAInferI8Status(*call)
        if st != 0:
            raise RuntimeError("status %d" % st)

    t0 = time.perf_counter()
    heat = 0
    while (time.perf_counter() - t0) * 1e3 < args.preheat_ms:
        for _ in range(200):
            step()
        torch.cuda.synchronize()
        heat += 200
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(args.calls):
        step()
    e1.record(stream)
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / args.calls
    out = {"lib": os.path.relpath(path, ROOT) if path else "shipped", "workload": args.workload, "calls": args.calls,
           "preheat_calls": heat, "us_per_call": round(us, 3),
           "pct_of_int8_peak": round(4.0 * B * H * S * S * d / (us * 1e-6) / 5033.2e12 * 100, 2)}
    if args.compare:
        got = o.cpu().numpy()
        ref = torch.zeros_like(q)
        rc = list(call)
        rc[7] = ref.data_ptr()
        assert shipped.FMHAInferI8Status(*rc) == 0
        torch.cuda.synchronize()
        out["bytes_differing_from_shipped"] = int((got != ref.cpu().numpy()).sum())
    if hasattr(lib, "FMHAInferI8DebugReadTrace"):
        nwg = min(4096, B * H * ((S + 255) // 256))
        buf = (C.c_uint * (nwg * 8 * 64))()
        lib.FMHAInferI8DebugReadTrace.argtypes = [C.c_void_p, C.c_int]
        assert lib.FMHAInferI8DebugReadTrace(buf, nwg * 8 * 64) == 0
        t = np.frombuffer(buf, dtype=np.uint32).reshape(nwg, 8, 64).astype(np.int64)
        work, wait = [[], []], [[], []]
        cycles = ticks = 0
        for wg in range(nwg):
            for w in range(8):
                x = t[wg, w, :62]
                n = int(np.argmax(x == 0)) if (x == 0).any() else 62
                if n >= 2 and n < 62:  # (a full stamp register has lost its last stamp)
                    cycles += int((x[n - 1] - x[0]) & 0xffffffff)
                    ticks += int((t[wg, w, 63] - t[wg, w, 62]) & 0xffffffff)
                dx = np.diff(x[:n]) & 0xffffffff  # start | (arrive, leave)* | end
                if len(dx) > 12:
                    wait[w // 4].append(dx[1::2][3:-3])
                    work[w // 4].append(dx[2::2][3:-3])
        for grp, name in ((0, "wavefronts 0-3"), (1, "wavefronts 4-7")):
            if not work[grp]:  # too few key blocks for a steady state
                continue
            wk, wt = np.concatenate(work[grp]), np.concatenate(wait[grp])
            out["ticks_" + name.replace(" ", "_")] = {
                "work_between_barriers_mean": round(float(wk.mean()), 1), "wait_at_barrier_mean": round(float(wt.mean()), 1),
                "work_even_ticks_mean": round(float(np.concatenate([a[0::2] for a in work[grp]]).mean()), 1),
                "work_odd_ticks_mean": round(float(np.concatenate([a[1::2] for a in work[grp]]).mean()), 1)}
        out["tick_unit"] = "s_memtime counts, steady-state ticks only (first and last three dropped)"
        if ticks:
            out["shader_mhz_inside_the_kernel"] = round(100.0 * cycles / ticks, 1)  # s_memtime counts per 10 ns
            out["wavefront_lifetime_cycles_mean"] = round(cycles / (nwg * 8.0), 1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
