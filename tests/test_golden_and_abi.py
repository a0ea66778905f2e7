"""CPU tests: the committed known-answer fixtures still come out of the checker bit for bit, and the C-ABI library
loads and exports every symbol that include/fmha_i8.h and include/fmha_quant.h declare (no compute call is made here)."""
import ctypes
import glob
import os
import re

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))


def test_fixtures_exist():
    assert len(FIXTURES) >= 4


@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p) for p in FIXTURES])
def test_checker_reproduces_fixture(orc, path):
    f = np.load(path)  # allow_pickle stays False
    qa, ka, va, oa = (float(x) for x in f["amax"])
    got = orc.fmha_i8_blockwise(f["q"], f["k"], f["v"], f["mask"], qa, ka, va, oa)
    assert np.array_equal(got, f["o"])
    full = orc.fmha_i8_blockwise_cross(f["q"], f["k"], f["v"], f["mask"], qa, ka, va, oa, full_range_p=True)
    assert np.array_equal(full, f["o_full_range_p"]) and not np.array_equal(full, f["o"])


def _declared_symbols():
    names = set()
    for header in ("fmha_i8.h", "fmha_quant.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        body = text.split('extern "C" {', 1)[1].split('} /* extern "C" */', 1)[0]
        names |= set(re.findall(r"\b(FMHA[A-Z]\w*)\s*\(", body))
    return sorted(names)


def test_library_exports_every_declared_symbol(pkg):
    names = _declared_symbols()
    assert set(names) == set(pkg.EXPORTED_SYMBOLS), names
    lib = ctypes.CDLL(pkg.LIB_PATH)
    for n in names:
        assert getattr(lib, n) is not None
    assert pkg.version().startswith("fmha_i8 gfx950")


def test_struct_layout_matches_the_reference(pkg):
    # inc/fmha_param_i8.h:3-17: 4 x int, 5 x float, same order and defaults
    assert ctypes.sizeof(pkg.AttnDataDescriptor) == 16 and ctypes.sizeof(pkg.FMHAParamI8) == 20
    assert [n for n, _ in pkg.AttnDataDescriptor._fields_] == ["batch_num", "seq_len", "head_num", "head_dim"]
    assert [n for n, _ in pkg.FMHAParamI8._fields_] == ["q_amax", "k_amax", "v_amax", "o_amax", "s_max"]
    a, p = pkg.AttnDataDescriptor(), pkg.FMHAParamI8()
    assert (a.batch_num, a.seq_len, a.head_num, a.head_dim) == (1, 64, 4, 64)
    assert (p.q_amax, p.k_amax, p.v_amax, p.o_amax, p.s_max) == (0.0, 0.0, 0.0, 1.0, 1.0)


def test_argument_checks_need_no_gpu(pkg):
    P = pkg.FMHAParamI8(1.0, 1.0, 1.0, 1.0)
    ok = pkg.AttnDataDescriptor(2, 256, 3, 128)
    a16 = 0x1000
    assert pkg.FMHAInferI8CheckArgs(P, ok, a16, a16, a16, a16 + 1, a16) == pkg.FMHA_I8_OK  # mask may be unaligned
    assert pkg.FMHAInferI8CheckArgs(P, ok, None, a16, a16, a16, a16) == pkg.FMHA_I8_ERR_NULL_POINTER
    assert pkg.FMHAInferI8CheckArgs(P, ok, a16, a16, a16, None, a16) == pkg.FMHA_I8_ERR_NULL_POINTER
    assert pkg.FMHAInferI8CheckArgs(P, ok, a16, a16 + 8, a16, a16, a16) == pkg.FMHA_I8_ERR_ALIGNMENT
    for d in (0, 32, 96, 256):
        assert pkg.FMHAInferI8CheckArgs(P, pkg.AttnDataDescriptor(1, 128, 1, d), a16, a16, a16, a16, a16) == \
            pkg.FMHA_I8_ERR_HEAD_DIM
    for s in (0, -128, 65537, 65600):
        assert pkg.FMHAInferI8CheckArgs(P, pkg.AttnDataDescriptor(1, s, 1, 64), a16, a16, a16, a16, a16) == \
            pkg.FMHA_I8_ERR_SEQ_LEN
    # every length of the reference's ladder (src/fmha_i8.cu:39-154), and lengths it does not have
    for s in (64, 128, 192, 320, 448, 512, 4096, 65536, 1, 32, 100, 1000):
        assert pkg.FMHAInferI8CheckArgs(P, pkg.AttnDataDescriptor(1, s, 1, 64), a16, a16, a16, a16, a16) == pkg.FMHA_I8_OK
    assert pkg.FMHAInferI8CheckArgs(P, pkg.AttnDataDescriptor(0, 128, 1, 64), a16, a16, a16, a16, a16) == \
        pkg.FMHA_I8_ERR_BATCH_HEAD
    assert pkg.FMHAInferI8CheckArgs(pkg.FMHAParamI8(1, 1, 1, 0.0), ok, a16, a16, a16, a16, a16) == pkg.FMHA_I8_ERR_SCALE
    assert pkg.FMHAInferI8CheckArgs(pkg.FMHAParamI8(float("nan"), 1, 1, 1), ok, a16, a16, a16, a16, a16) == \
        pkg.FMHA_I8_ERR_SCALE
    # finite amax values whose product or quotient overflows: the derived scales would be inf / NaN
    for bad in (pkg.FMHAParamI8(1e20, 1e20, 1, 1), pkg.FMHAParamI8(1, 1, 3e38, 1e-3), pkg.FMHAParamI8(3e38, 3e38, 1, 1)):
        assert pkg.FMHAInferI8CheckArgs(bad, ok, a16, a16, a16, a16, a16) == pkg.FMHA_I8_ERR_SCALE
        # the launching entry point refuses it before any HIP call (no GPU needed to see that)
        assert pkg.FMHAInferI8Status(None, bad, ok, a16, a16, a16, a16, a16, True) == pkg.FMHA_I8_ERR_SCALE
    assert pkg.FMHAInferI8CheckArgs(pkg.FMHAParamI8(1e18, 1e18, 1e30, 1e-5), ok, a16, a16, a16, a16, a16) == pkg.FMHA_I8_OK
    for code in range(0, 7):
        assert pkg.status_string(code)


def test_missing_library_is_an_error_not_a_fallback(pkg, tmp_path):
    with pytest.raises((FileNotFoundError, OSError)):
        pkg.load_library(str(tmp_path / "libfmha_i8.so"))
