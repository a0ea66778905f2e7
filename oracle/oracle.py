"""TEST INFRASTRUCTURE ONLY: ctypes binding of the CPU checker (oracle/liboracle.so, oracle/_ref/libfmha_ref_cpu.so).

Only the test-suite, the smoke test and the CPU-baseline leg of the benchmark import this module.  The GPU product
path never does.  Each function names the reference lines its C++ counterpart restates (see fmha_oracle.hpp).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "liboracle.so")
_REF = os.path.join(_HERE, "_ref", "libfmha_ref_cpu.so")

_i8p = np.ctypeslib.ndpointer(np.int8, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")


def build(force=False):
    """Compile liboracle.so (and _ref when the reference tree is present) with the Makefile beside this file."""
    if force or not os.path.exists(_LIB):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "all"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB)
        L.oracle_cpu_gemm_f32.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_long, C.c_long, C.c_long,
                                          C.c_int, C.c_float, C.c_float, C.c_int, C.c_int, C.c_int]
        L.oracle_cpu_gemm_i8.argtypes = [_i8p, _i8p, _i32p, C.c_int, C.c_int, C.c_int, C.c_long, C.c_long, C.c_long,
                                         C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
        L.oracle_cpu_attention_masked_softmax_f32.argtypes = [_f32p, _f32p, _i32p, C.c_int, C.c_int, C.c_int, C.c_int,
                                                              C.c_int]
        L.oracle_quantize_i8.argtypes = [_f32p, _i8p, C.c_long, C.c_float]
        L.oracle_abs_max.argtypes = [_f32p, C.c_long]
        L.oracle_abs_max.restype = C.c_float
        L.oracle_mean_rel_deviation_pct.argtypes = [_i8p, _f32p, C.c_long, C.c_float]
        L.oracle_mean_rel_deviation_pct.restype = C.c_float
        L.oracle_reference_row_scale.argtypes = [C.c_int]
        L.oracle_reference_row_scale.restype = C.c_float
        L.oracle_fmha_i8_blockwise.argtypes = [_i8p, _i8p, _i8p, _i8p, _i8p, C.c_int, C.c_int, C.c_int, C.c_int,
                                               C.c_float, C.c_float, C.c_float, C.c_float, C.c_int, C.c_int, C.c_long,
                                               C.c_long]
        L.oracle_fmha_i8_blockwise_cross.argtypes = [_i8p, _i8p, _i8p, _i8p, _i8p, C.c_int, C.c_int, C.c_int, C.c_int,
                                                     C.c_int, C.c_float, C.c_float, C.c_float, C.c_float, C.c_int,
                                                     C.c_int, C.c_long, C.c_long]
        L.oracle_fmha_i8_blockwise_cross.restype = None
        L.oracle_fmha_i8_blockwise_cross_full_range_p.argtypes = L.oracle_fmha_i8_blockwise_cross.argtypes
        L.oracle_fmha_i8_blockwise_cross_full_range_p.restype = None
        L.oracle_fmha_fp32.argtypes = [_f32p, _f32p, _f32p, _i8p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                       C.c_long, C.c_long]
        L.oracle_hardware_threads.restype = C.c_int
        _lib = L
    return _lib


def have_ref():
    return os.path.exists(_REF)


def ref():
    """The reference's own cpuGEMM.hpp / cpuSoftmax.hpp, compiled from the reference tree (None if never built)."""
    global _ref
    if _ref is None and have_ref():
        R = C.CDLL(_REF)
        R.ref_cpu_gemm_f32.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                       C.c_int, C.c_float, C.c_float, C.c_int, C.c_int, C.c_int]
        R.ref_cpu_gemm_i8.argtypes = [_i8p, _i8p, _i32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int,
                                      C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
        R.ref_cpu_attention_masked_softmax_f32.argtypes = [_f32p, _f32p, _i32p, C.c_int, C.c_int, C.c_int, C.c_int,
                                                           C.c_int]
        R.ref_fmha_fp32_heads.argtypes = [_f32p, _f32p, _f32p, _i32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int,
                                          C.c_long, C.c_long]
        _ref = R
    return _ref


def hardware_threads():
    return int(lib().oracle_hardware_threads())


# ---- inc/cpuGEMM.hpp:8-31 --------------------------------------------------------------------------------------
def cpu_gemm_f32(a, b, c, M, N, K, sa, sb, sc, batch, alpha, beta, trans_a, trans_b, col_major_c):
    lib().oracle_cpu_gemm_f32(a, b, c, M, N, K, sa, sb, sc, batch, alpha, beta, int(trans_a), int(trans_b),
                              int(col_major_c))
    return c


def cpu_gemm_i8(a, b, c, M, N, K, sa, sb, sc, batch, alpha, beta, trans_a, trans_b, col_major_c):
    lib().oracle_cpu_gemm_i8(a, b, c, M, N, K, sa, sb, sc, batch, alpha, beta, int(trans_a), int(trans_b),
                             int(col_major_c))
    return c


# ---- inc/cpuSoftmax.hpp:11-51 ----------------------------------------------------------------------------------
def cpu_attention_masked_softmax_f32(s, mask_i32, batch, seq_q, seq_k, head_num, head_dim):
    p = np.zeros_like(s)
    lib().oracle_cpu_attention_masked_softmax_f32(s, p, mask_i32, batch, seq_q, seq_k, head_num, head_dim)
    return p


# ---- inc/utils.hpp:23-39,59-89 ---------------------------------------------------------------------------------
def quantize_i8(x, amax):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.int8)
    lib().oracle_quantize_i8(x.reshape(-1), out.reshape(-1), x.size, float(amax))
    return out


def abs_max(x):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    return float(lib().oracle_abs_max(x, x.size))


def mean_rel_deviation_pct(res_i8, ref_f32, o_amax):
    res = np.ascontiguousarray(res_i8, dtype=np.int8).reshape(-1)
    rf = np.ascontiguousarray(ref_f32, dtype=np.float32).reshape(-1)
    return float(lib().oracle_mean_rel_deviation_pct(res, rf, res.size, float(o_amax)))


def reference_row_scale(head_dim):
    return float(lib().oracle_reference_row_scale(int(head_dim)))


# ---- inc/fmha_i8.cuh int8 pipeline -----------------------------------------------------------------------------
def fmha_i8_blockwise(q, k, v, mask, q_amax, k_amax, v_amax, o_amax, block=128, threads=None, heads=None):
    """q, k, v: int8 [B,H,S,d]; mask: int8 [B,S], nonzero = masked out.  Returns int8 O [B,H,S,d].
    heads=(begin, end) restricts the work to that range of the flattened batch*head index (others stay 0)."""
    B, H, S, d = q.shape
    q, k, v = (np.ascontiguousarray(t, dtype=np.int8) for t in (q, k, v))
    mask = np.ascontiguousarray(mask, dtype=np.int8)
    assert k.shape == q.shape and v.shape == q.shape and mask.shape == (B, S)
    o = np.zeros_like(q)
    hb, he = (0, B * H) if heads is None else heads
    lib().oracle_fmha_i8_blockwise(q.reshape(-1), k.reshape(-1), v.reshape(-1), mask.reshape(-1), o.reshape(-1), B, H,
                                   S, d, q_amax, k_amax, v_amax, o_amax, block,
                                   threads or hardware_threads(), hb, he)
    return o


def fmha_i8_blockwise_cross(q, k, v, mask, q_amax, k_amax, v_amax, o_amax, block=None, threads=None,
                            full_range_p=False):
    """q: int8 [B,H,Sq,d]; k, v: int8 [B,H,S,d]; mask: int8 [B,S], nonzero = masked out.  Returns int8 O [B,H,Sq,d].
    block defaults to what the reference's ladder would give S: 128 keys for multiples of 128, else 64.  A key count
    that is no multiple of 64 means the next multiple of 64 with the missing keys masked out.
    full_range_p: P = rne(255 p) in [0, 255] instead of rne(-128 p) in [-128, 0] (README.md:15,186, planned there)."""
    B, H, Sq, d = q.shape
    S = k.shape[2]
    assert k.shape == (B, H, S, d) and v.shape == k.shape and mask.shape == (B, S)
    q, k, v = (np.ascontiguousarray(t, dtype=np.int8) for t in (q, k, v))
    mask = np.ascontiguousarray(mask, dtype=np.int8)
    o = np.zeros_like(q)
    fn = lib().oracle_fmha_i8_blockwise_cross_full_range_p if full_range_p else lib().oracle_fmha_i8_blockwise_cross
    fn(q.reshape(-1), k.reshape(-1), v.reshape(-1), mask.reshape(-1), o.reshape(-1), B, H, Sq, S, d, q_amax, k_amax,
       v_amax, o_amax, block or (128 if (S + 63) // 64 * 64 % 128 == 0 else 64), threads or hardware_threads(), 0, B * H)
    return o


# ---- test_fmha_i8.cpp:141-162 float path -----------------------------------------------------------------------
def fmha_fp32(q, k, v, mask, threads=None, heads=None):
    B, H, S, d = q.shape
    q, k, v = (np.ascontiguousarray(t, dtype=np.float32) for t in (q, k, v))
    mask = np.ascontiguousarray(mask, dtype=np.int8)
    o = np.zeros_like(q)
    hb, he = (0, B * H) if heads is None else heads
    lib().oracle_fmha_fp32(q.reshape(-1), k.reshape(-1), v.reshape(-1), mask.reshape(-1), o.reshape(-1), B, H, S, d,
                           threads or hardware_threads(), hb, he)
    return o


def ref_fmha_fp32(q, k, v, mask, heads=None):
    """Same path through the reference's own headers (single thread, as in the reference)."""
    B, H, S, d = q.shape
    q, k, v = (np.ascontiguousarray(t, dtype=np.float32) for t in (q, k, v))
    m = np.ascontiguousarray((np.asarray(mask) != 0).astype(np.int32))
    o = np.zeros_like(q)
    hb, he = (0, B * H) if heads is None else heads
    ref().ref_fmha_fp32_heads(q.reshape(-1), k.reshape(-1), v.reshape(-1), m.reshape(-1), o.reshape(-1), B, H, S, d,
                              hb, he)
    return o
