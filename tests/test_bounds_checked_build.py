"""The attention kernel compiled with FMHA_CHECK_BOUNDS (tests/bin/libfmha_i8_checked.so, built by the tests' Makefile):
every global access is checked against the tensor - for K and V the head - it belongs to, and an access that would
leave it is counted and redirected instead of performed.  An out-of-bounds READ changes no result and, inside the pool
of a caching allocator, raises no fault either, so no other test can see one; this one does, without ever faulting.
(A key sequence shorter than one block was once fetched whole at the later issue points of the key loop: 0 results
changed, the GPU faulted only when the tensors happened to lie at the end of mapped memory.)"""
import ctypes as C
import os

import numpy as np
import pytest

import fmha_cases as fc

HERE = os.path.dirname(os.path.abspath(__file__))
CHECKED = os.path.join(HERE, "bin", "libfmha_i8_checked.so")


def test_the_shipped_library_has_no_debug_entry_point(pkg):
    lib = pkg.load_library()
    assert not hasattr(lib, "FMHAInferI8DebugOutOfBounds")


@pytest.fixture(scope="module")
def checked(pkg):
    if not os.path.exists(CHECKED):
        pytest.fail("%s is not built; run `make -C tests`" % CHECKED)
    lib = pkg.load_library(CHECKED)
    lib.FMHAInferI8DebugOutOfBounds.argtypes = []
    lib.FMHAInferI8DebugOutOfBounds.restype = C.c_int
    return lib


def _run(pkg, lib, dev, q, k, v, mask, scales, full_range_p=False):
    import torch
    t = [torch.from_numpy(np.ascontiguousarray(a)).to(dev) for a in (q, k, v, mask)]
    o = torch.empty_like(t[0])
    B, H, Sq, d = q.shape
    entry = lib.FMHAInferI8CrossFullRangeP if full_range_p else lib.FMHAInferI8Cross
    st = entry(None, pkg.FMHAParamI8(*scales, 1.0), pkg.FMHACrossAttnDescriptor(B, Sq, k.shape[2], H, d),
               *(x.data_ptr() for x in t), o.data_ptr())
    assert st == pkg.FMHA_I8_OK
    return o


@pytest.mark.gpu
def test_checked_build_counts_nothing_on_any_shape(pkg, orc, checked, dev):
    assert checked.FMHAInferI8DebugOutOfBounds() == 0  # (also clears the counter)
    rng = np.random.default_rng(77)
    shapes = [(3, 3, 319, 3, 64), (1, 1, 1, 1, 128), (2, 2, 70, 70, 128), (2, 1, 300, 129, 64), (1, 2, 64, 64, 64),
              (1, 2, 1024, 1024, 128), (2, 2, 2048, 2048, 64), (1, 1, 100, 4095, 128), (1, 1, 4097, 65, 64),
              (2, 1, 40, 15, 64), (2, 1, 40, 16, 128), (2, 1, 40, 17, 64), (2, 1, 40, 31, 128), (1, 1, 40, 4100, 64)]
    for _ in range(40):
        S = int(rng.choice([rng.integers(1, 130), rng.integers(1, 700), rng.integers(500, 2600), 64 * rng.integers(1, 40)]))
        Sq = S if rng.random() < 0.4 else int(rng.choice([rng.integers(1, 70), rng.integers(1, 600), rng.integers(200, 1500)]))
        shapes.append((int(rng.integers(1, 4)), int(rng.integers(1, 4)), Sq, S, int(rng.choice([64, 128]))))
    for n, (B, H, Sq, S, d) in enumerate(shapes):
        c = fc.make_inputs(B, H, (S + 63) // 64 * 64, d, pad=str(rng.choice(["none", "scatter"])), seed=300 + n)
        mask = c["mask"][:, :S].copy()
        if n % 3 == 0:
            mask[:, S // 2 + 1:] = 1  # trailing padding: fewer blocks than the length has
        mask[:, 0] = 0
        k, v = (np.ascontiguousarray(c[x][:, :, :S]) for x in ("k", "v"))
        q = fc.make_inputs(B, H, Sq, d, seed=700 + n)["q"]
        scales = (c["q_amax"], c["k_amax"], c["v_amax"], 1.0)
        print("shape", B, H, Sq, S, d, flush=True)
        for full in (False, True):  # the reference's P on 128 steps, and P on 255 steps
            o = _run(pkg, checked, dev, q, k, v, mask, scales, full)
            assert checked.FMHAInferI8DebugOutOfBounds() == 0, (B, H, Sq, S, d, full)
            st = fc.parity_stats(o.cpu().numpy(), orc.fmha_i8_blockwise_cross(q, k, v, mask, *scales, full_range_p=full))
            assert st["within1"] >= 0.999 and st["max"] <= 2, ((B, H, Sq, S, d, full), st)
