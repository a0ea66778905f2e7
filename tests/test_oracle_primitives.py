"""CPU tests that pin the primitives of the checker: the GEMM and masked-softmax restatements against the reference's
own headers compiled from the reference tree (oracle/_ref, when present) and against closed forms; the quantiser and
the acceptance metric against known answers."""
import numpy as np
import pytest

import fmha_cases as fc


def _need_ref(orc):
    if not orc.have_ref():
        pytest.skip("oracle/_ref not built (reference tree absent on this machine)")
    return orc.ref()


# ---------------------------------------------------------------- cpu_gemm (inc/cpuGEMM.hpp:8-31)
@pytest.mark.parametrize("trans_a,trans_b,col_c", [(1, 0, 0), (1, 1, 0), (0, 0, 0), (0, 1, 1), (1, 0, 1)])
def test_gemm_f32_matches_reference_header(orc, trans_a, trans_b, col_c):
    R = _need_ref(orc)
    rng = np.random.default_rng(1)
    M, N, K, batch = 7, 5, 11, 3
    a = rng.standard_normal(batch * M * K).astype(np.float32)
    b = rng.standard_normal(batch * N * K).astype(np.float32)
    c0 = rng.standard_normal(batch * M * N).astype(np.float32)
    mine, theirs = c0.copy(), c0.copy()
    orc.cpu_gemm_f32(a, b, mine, M, N, K, M * K, N * K, M * N, batch, 1.5, 0.25, trans_a, trans_b, col_c)
    R.ref_cpu_gemm_f32(a, b, theirs, M, N, K, M * K, N * K, M * N, batch, 1.5, 0.25, trans_a, trans_b, col_c)
    assert np.array_equal(mine, theirs)  # same loop order, same float operations: bit-identical


@pytest.mark.parametrize("trans_a,trans_b", [(1, 0), (1, 1)])
def test_gemm_i8_matches_reference_header_and_numpy(orc, trans_a, trans_b):
    rng = np.random.default_rng(2)
    M, N, K, batch = 9, 6, 64, 2
    a = rng.integers(-128, 128, (batch, M, K), dtype=np.int8)
    b = rng.integers(-128, 128, (batch, N, K) if not trans_b else (batch, K, N), dtype=np.int8)
    mine = np.zeros((batch, M, N), np.int32)
    orc.cpu_gemm_i8(a.reshape(-1), b.reshape(-1), mine.reshape(-1), M, N, K, M * K, N * K, M * N, batch, 1, 0, trans_a,
                    trans_b, 0)
    bm = b.astype(np.int64) if trans_b else b.astype(np.int64).transpose(0, 2, 1)
    want = a.astype(np.int64) @ bm
    assert np.array_equal(mine, want)
    if orc.have_ref():
        theirs = np.zeros((batch, M, N), np.int32)
        orc.ref().ref_cpu_gemm_i8(a.reshape(-1), b.reshape(-1), theirs.reshape(-1), M, N, K, M * K, N * K, M * N, batch,
                                  1, 0, trans_a, trans_b, 0)
        assert np.array_equal(mine, theirs)


def test_gemm_identity_and_layouts(orc):
    # A (stored [M][K]) times identity: C row-major reproduces A; column-major C is its transpose in memory.
    M = K = N = 4
    a = np.arange(16, dtype=np.float32)
    eye = np.eye(4, dtype=np.float32).reshape(-1)
    c = np.zeros(16, np.float32)
    orc.cpu_gemm_f32(a, eye, c, M, N, K, 0, 0, 0, 1, 1.0, 0.0, 1, 0, 0)
    assert np.array_equal(c, a)
    c = np.zeros(16, np.float32)
    orc.cpu_gemm_f32(a, eye, c, M, N, K, 0, 0, 0, 1, 1.0, 0.0, 1, 0, 1)
    assert np.array_equal(c.reshape(4, 4), a.reshape(4, 4).T)
    # transA == false means A is stored [K][M]
    c = np.zeros(16, np.float32)
    orc.cpu_gemm_f32(a, eye, c, M, N, K, 0, 0, 0, 1, 1.0, 0.0, 0, 0, 0)
    assert np.array_equal(c.reshape(4, 4), a.reshape(4, 4).T)
    # beta path reads C
    c = np.ones(16, np.float32)
    orc.cpu_gemm_f32(a, eye, c, M, N, K, 0, 0, 0, 1, 2.0, 3.0, 1, 0, 0)
    assert np.array_equal(c, 2 * a + 3)


# ---------------------------------------------------------------- masked softmax (inc/cpuSoftmax.hpp:11-51)
def test_softmax_matches_reference_header(orc):
    R = _need_ref(orc)
    rng = np.random.default_rng(3)
    B, H, Sq, Sk, d = 2, 3, 5, 16, 64
    s = (rng.standard_normal((B, H, Sq, Sk)) * 20).astype(np.float32)
    mask = (rng.random((B, Sk)) < 0.3).astype(np.int32)
    mask[1, :] = 1  # a fully masked batch entry
    mine = orc.cpu_attention_masked_softmax_f32(s.reshape(-1), mask.reshape(-1), B, Sq, Sk, H, d).reshape(s.shape)
    theirs = np.zeros_like(s)
    R.ref_cpu_attention_masked_softmax_f32(s.reshape(-1).copy(), theirs.reshape(-1), mask.reshape(-1), B, Sq, Sk, H, d)
    assert np.array_equal(mine, theirs)
    assert np.all(mine[1] == 0) and not np.isnan(mine).any()


def test_softmax_closed_forms(orc):
    # two keys, scores [1, 2], d = 4: softmax([0.5, 1.0]) = [1/(1+e^.5), e^.5/(1+e^.5)]
    s = np.array([1.0, 2.0], np.float32)
    p = orc.cpu_attention_masked_softmax_f32(s, np.zeros(2, np.int32), 1, 1, 2, 1, 4)
    e = np.exp(0.5)
    assert np.allclose(p, [1 / (1 + e), e / (1 + e)], rtol=1e-6)
    # masking a key renormalises over the rest; mask value 2 is NOT a mask for this function (== 1 test)
    s = np.array([3.0, 100.0, 3.0, 3.0], np.float32)
    p = orc.cpu_attention_masked_softmax_f32(s, np.array([0, 1, 0, 0], np.int32), 1, 1, 4, 1, 16)
    assert np.allclose(p, [1 / 3, 0, 1 / 3, 1 / 3], rtol=1e-6)
    p = orc.cpu_attention_masked_softmax_f32(s, np.array([0, 2, 0, 0], np.int32), 1, 1, 4, 1, 16)
    assert p[1] > 0.99
    # rows pick the mask of their own batch entry: row r -> batch r // (seq_q * head_num)
    B, H, Sq, Sk = 2, 2, 3, 4
    s = np.zeros((B, H, Sq, Sk), np.float32)
    mask = np.array([[0, 0, 1, 1], [1, 0, 0, 0]], np.int32)
    p = orc.cpu_attention_masked_softmax_f32(s.reshape(-1), mask.reshape(-1), B, Sq, Sk, H, 64).reshape(s.shape)
    assert np.allclose(p[0], np.broadcast_to([.5, .5, 0, 0], (H, Sq, Sk)))
    assert np.allclose(p[1], np.broadcast_to([0, 1 / 3, 1 / 3, 1 / 3], (H, Sq, Sk)))


# ---------------------------------------------------------------- quantiser, amax, metric (inc/utils.hpp:23-39,59-89)
def test_quantizer_known_answers(orc):
    amax = 2.0
    step = amax / 127.0
    xs = np.array([0.0, amax, -amax, 0.5 * step, -0.5 * step, 1.5 * step, -1.5 * step, 0.49 * step, 3 * amax, -3 * amax,
                   126.4 * step, 126.6 * step], np.float32)
    # half-up: +0.5 -> 1, -0.5 -> 0, +1.5 -> 2, -1.5 -> -1; clamp at +-127
    want = np.array([0, 127, -127, 1, 0, 2, -1, 0, 127, -127, 126, 127], np.int8)
    got = orc.quantize_i8(xs, amax)
    assert np.array_equal(got, want)
    assert np.array_equal(fc.quantize_i8_np(xs, amax), want)
    # floorf takes a float: with amax = 127 the scale is exactly 1, and the float just below 0.5 rounds up to 1.0f in the
    # sum and quantises to 1; its neighbour one ulp further down does not
    edge = np.array([0x3EFFFFFF, 0x3EFFFFFE, 0x3F000000, 0xBF000000, 0xBF000001], np.uint32).view(np.float32)
    assert np.array_equal(orc.quantize_i8(edge, 127.0), np.array([1, 0, 1, 0, -1], np.int8))
    assert np.array_equal(fc.quantize_i8_np(edge, 127.0), np.array([1, 0, 1, 0, -1], np.int8))
    rng = np.random.default_rng(5)
    x = rng.standard_normal(10000).astype(np.float32) * 3
    a = orc.abs_max(x)
    assert a == np.abs(x).max()
    assert np.array_equal(orc.quantize_i8(x, a), fc.quantize_i8_np(x, a))
    assert orc.abs_max(np.zeros(0, np.float32)) == 0.0


def test_deviation_metric_closed_form(orc):
    # res = 127 everywhere, o_amax = 2 -> dequantised 2.0; ref = 1.0 -> |2-1|/(1+0.01)*100
    n = 128
    res = np.full(n, 127, np.int8)
    ref = np.ones(n, np.float32)
    assert orc.mean_rel_deviation_pct(res, ref, 2.0) == pytest.approx(100 / 1.01, rel=1e-5)
    # exact representation -> 0
    res = np.array([0, 127, -127, 64] * 16, np.int8)
    ref = res.astype(np.float32) / 127 * 3.0
    assert orc.mean_rel_deviation_pct(res, ref, 3.0) == pytest.approx(0.0, abs=1e-4)
    # the reference sums rows of 64 only: a tail of len % 64 is ignored in the sum but counted in the divisor
    res = np.full(96, 127, np.int8)
    ref = np.ones(96, np.float32)
    assert orc.mean_rel_deviation_pct(res, ref, 2.0) == pytest.approx(100 / 1.01 * 64 / 96, rel=1e-5)


def test_row_scale_is_the_kernels_constexpr_sqrt(orc):
    # inc/fmha_i8.cuh:13-34,71: Newton iteration to a fixed point; 1/8 exactly for d=64, and within 1 ulp of
    # 1/sqrt(128) for d=128
    assert orc.reference_row_scale(64) == 0.125
    r = np.float32(orc.reference_row_scale(128))
    exact = 1.0 / np.sqrt(128.0)
    assert abs(float(r) - exact) <= np.spacing(np.float32(exact))
