"""The "before" builds that the measurements compare the shipped kernel with (tests/Makefile, target `variants`) must
compute the same bytes as the shipped library: a layout or schedule variant that differs in its results would be
measuring a different computation.  The knock-out builds compute garbage on purpose and are not checked here."""
import ctypes as C
import os

import numpy as np
import pytest

import fmha_cases as fc

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
# same results by construction: LDS layouts, tile path and barrier count only
SAME_BYTES = ["few", "no_swizzle", "old_k_swizzle", "staged_loads", "two_barriers"]
# (B, H, S, d, distribution): whole blocks of 128 keys only - the test builds carry no other instantiation; both
# arithmetic variants (accumulators read as floats / converted), no masked key and a masked tail
SHAPES = [
    (2, 4, 1024, 128, "normal", "none"),
    (1, 2, 1536, 128, "normal", "tail256"),
    (2, 4, 1024, 64, "normal", "none"),
    (2, 2, 2048, 64, "student_t", "none"),
    (4, 3, 512, 64, "student_t", "bert"),
]


def run(lib, pkg, dev, c):
    import torch
    lib.FMHAInferI8Status.argtypes = [C.c_void_p, pkg.FMHAParamI8, pkg.AttnDataDescriptor] + [C.c_void_p] * 5 + [C.c_bool]
    lib.FMHAInferI8Status.restype = C.c_int
    B, H, S, d = c["q"].shape
    q, k, v, m = (torch.from_numpy(np.ascontiguousarray(c[n])).to(dev) for n in ("q", "k", "v", "mask"))
    o = torch.full_like(q, 77)
    st = lib.FMHAInferI8Status(torch.cuda.current_stream(dev).cuda_stream,
                               pkg.FMHAParamI8(c["q_amax"], c["k_amax"], c["v_amax"], c["o_amax"], 1.0),
                               pkg.AttnDataDescriptor(B, S, H, d), q.data_ptr(), k.data_ptr(), v.data_ptr(), m.data_ptr(),
                               o.data_ptr(), True)
    torch.cuda.synchronize()
    assert st == 0, "status %d" % st
    return o.cpu().numpy()


@pytest.mark.parametrize("variant", SAME_BYTES)
def test_variant_build_writes_the_shipped_bytes(pkg, dev, variant):
    path = os.path.join(HERE, "bin", "libfmha_i8_%s.so" % variant)
    assert os.path.exists(path), "%s is missing: build it with `make -C tests variants`" % path
    lib = C.CDLL(path)
    shipped = pkg.load_library()
    for B, H, S, d, dist, pad in SHAPES:
        c = fc.make_inputs(B, H, S, d, dist=dist, sigma=0.5 if dist == "student_t" else 1.0, pad=pad, seed=424242)
        print(variant, (B, H, S, d, dist, pad), flush=True)
        want = run(shipped, pkg, dev, c)
        got = run(lib, pkg, dev, c)
        assert np.array_equal(got, want), (variant, (B, H, S, d, dist, pad), int((got != want).sum()))
