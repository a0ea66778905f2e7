"""GPU tests of the quantisation front end / back end (include/fmha_quant.h), called through the C ABI, against the CPU
checker's restatement of inc/utils.hpp:23-39,53.  Integer and byte work: the bar is bit-exact."""
import numpy as np
import pytest

import fmha_cases as fc

pytestmark = pytest.mark.gpu


def _dev(dev, a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _quantize(pkg, dev, x, amax=None, amax_dev=None):
    import torch
    xd = _dev(dev, x)
    out = torch.full((x.size + 16,), 99, dtype=torch.int8, device=dev)  # canary bytes behind the end
    st = pkg.FMHAQuantizeI8(None, xd, x.size, 0.0 if amax is None else amax, amax_dev, out)
    assert st == pkg.FMHA_I8_OK, st
    torch.cuda.synchronize()
    o = out.cpu().numpy()
    assert (o[x.size:] == 99).all()
    return o[:x.size]


@pytest.mark.parametrize("n", [0, 1, 3, 4, 5, 15, 16, 17, 1023, 4096, 1000003])
def test_quantize_matches_the_checker_bit_for_bit(pkg, orc, dev, n):
    rng = np.random.default_rng(n + 1)
    x = (3.0 * rng.standard_normal(n)).astype(np.float32)
    amax = float(np.abs(x).max()) if n else 1.0
    got = _quantize(pkg, dev, x, amax=amax)
    assert np.array_equal(got, orc.quantize_i8(x, amax) if n else np.zeros(0, np.int8))


def test_quantize_edge_values(pkg, orc, dev):
    # amax = 127 makes the scale exactly 1: ties go half-up, the float just below 0.5 rounds up inside the float add
    # (inc/utils.hpp:26: floorf takes a float), values beyond amax clamp to +-127, infinities clamp, NaN gives 0
    bits = np.array([0x3EFFFFFF, 0x3EFFFFFE, 0x3F000000, 0xBF000000, 0xBF000001, 0x00000000, 0x80000000], np.uint32)
    x = np.concatenate([bits.view(np.float32),
                        np.array([1.5, -1.5, 2.5, -2.5, 126.5, 126.49, 127.0, 128.0, -127.0, -1000.0, 2e9, -2e9],
                                 np.float32)])
    want = orc.quantize_i8(x, 127.0)
    assert list(want[:5]) == [1, 0, 1, 0, -1] and want[-1] == -127 and want[-2] == 127
    assert np.array_equal(_quantize(pkg, dev, x, amax=127.0), want)
    # beyond the int32 range the reference's float -> int conversion is undefined; here it saturates
    huge = np.array([1e30, -1e30, np.inf, -np.inf], np.float32)
    assert list(_quantize(pkg, dev, huge, amax=127.0)) == [127, -127, 127, -127]
    with_nan = np.array([np.nan, 1.0, -np.nan, 2.0], np.float32)
    assert list(_quantize(pkg, dev, with_nan, amax=127.0)) == [0, 1, 0, 2]
    # amax = 0: 127/0 = inf, 0 * inf = NaN -> 0, anything else saturates
    assert list(_quantize(pkg, dev, np.array([0.0, 1.0, -1.0, 0.0], np.float32), amax=0.0)) == [0, 127, -127, 0]


@pytest.mark.parametrize("n", [0, 1, 5, 4096, 777777])
def test_abs_max_matches_the_checker(pkg, orc, dev, n):
    import torch
    rng = np.random.default_rng(100 + n)
    x = rng.standard_normal(n).astype(np.float32)
    if n > 4:
        x[n // 2] = -7.5  # the maximum is a negative number
        x[1] = np.nan     # skipped, as `abs_val > max_val` skips it (inc/utils.hpp:36)
    out = torch.full((1,), -1.0, dtype=torch.float32, device=dev)
    assert pkg.FMHAAbsMaxF32(None, _dev(dev, x), n, out) == pkg.FMHA_I8_OK
    torch.cuda.synchronize()
    want = np.float32(np.nanmax(np.abs(x))) if n else np.float32(0)
    assert out.item() == want
    if n:
        assert out.item() == orc.abs_max(np.nan_to_num(x, nan=0.0))


def test_quantize_with_the_maximum_left_on_the_device(pkg, orc, dev):
    import torch
    x = (0.5 * np.random.default_rng(9).standard_t(3, 300001)).astype(np.float32)
    xd = _dev(dev, x)
    q, a = pkg.quantize_tensor(xd)  # abs-max and quantise back to back on one stream, no host round trip between them
    torch.cuda.synchronize()
    amax = float(np.abs(x).max())
    assert a.item() == np.float32(amax)
    assert np.array_equal(q.cpu().numpy(), orc.quantize_i8(x, amax))


@pytest.mark.parametrize("n", [0, 1, 7, 4096, 300001])
def test_dequantize_is_exact(pkg, dev, n):
    import torch
    v = np.random.default_rng(n).integers(-128, 128, n).astype(np.int8)
    amax = 3.25
    out = torch.full((n + 4,), 5.0, dtype=torch.float32, device=dev)
    assert pkg.FMHADequantizeI8(None, _dev(dev, v), n, amax, out) == pkg.FMHA_I8_OK
    torch.cuda.synchronize()
    o = out.cpu().numpy()
    want = v.astype(np.float32) / np.float32(127.0) * np.float32(amax)  # inc/utils.hpp:53, same order
    assert np.array_equal(o[:n], want) and (o[n:] == 5.0).all()


def test_argument_checks(pkg, dev):
    import torch
    x = torch.zeros(64, dtype=torch.float32, device=dev)
    o = torch.zeros(64, dtype=torch.int8, device=dev)
    assert pkg.FMHAQuantizeI8(None, x.data_ptr() + 4, 8, 1.0, None, o) == pkg.FMHA_I8_ERR_ALIGNMENT
    assert pkg.FMHAQuantizeI8(None, x, 8, 1.0, None, o.data_ptr() + 1) == pkg.FMHA_I8_ERR_ALIGNMENT
    assert pkg.FMHAQuantizeI8(None, None, 8, 1.0, None, o) == pkg.FMHA_I8_ERR_NULL_POINTER
    assert pkg.FMHAQuantizeI8(None, x, 8, float("nan"), None, o) == pkg.FMHA_I8_ERR_SCALE
    assert pkg.FMHAAbsMaxF32(None, x, 8, None) == pkg.FMHA_I8_ERR_NULL_POINTER
    assert pkg.FMHADequantizeI8(None, o, -1, 1.0, x) == pkg.FMHA_I8_ERR_NULL_POINTER


def test_float_tensors_through_the_whole_path(pkg, orc, dev):
    """fp32 Q, K, V -> abs-max + quantise on the GPU -> FMHAInferI8 -> de-quantise on the GPU, against the same steps of
    the reference's driver done by the CPU checker (test_fmha_i8.cpp:91-110,141-162,180-222)."""
    import torch
    c = fc.make_inputs(2, 3, 256, 64, dist="normal", pad="scatter", seed=123)
    dq, dk, dv = (_dev(dev, c[n]) for n in ("qf", "kf", "vf"))
    (q8, qa), (k8, ka), (v8, va) = (pkg.quantize_tensor(t) for t in (dq, dk, dv))
    amax = [t.item() for t in (qa, ka, va)]
    assert amax == [np.float32(c[n]) for n in ("q_amax", "k_amax", "v_amax")]
    for got, name in ((q8, "q"), (k8, "k"), (v8, "v")):
        assert np.array_equal(got.cpu().numpy(), c[name])
    o8 = pkg.fmha_infer_i8(q8, k8, v8, _dev(dev, c["mask"]), amax[0], amax[1], amax[2], 1.0)
    of = pkg.dequantize_tensor(o8, 1.0)
    torch.cuda.synchronize()
    want8 = orc.fmha_i8_blockwise(c["q"], c["k"], c["v"], c["mask"], c["q_amax"], c["k_amax"], c["v_amax"], 1.0)
    st = fc.parity_stats(o8.cpu().numpy(), want8)
    assert st["within1"] >= 0.999 and st["max"] <= 2, st
    assert np.array_equal(of.cpu().numpy(), o8.cpu().numpy().astype(np.float32) / np.float32(127.0) * np.float32(1.0))


# ---- bfloat16 tensors --------------------------------------------------------------------------------------------
def _to_bf16_bits(x):
    """float32 -> bfloat16 bit patterns, round to nearest even (finite inputs)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def _widen(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


@pytest.mark.parametrize("n", [0, 1, 7, 8, 9, 31, 4096, 1000003])
def test_bf16_abs_max_and_quantize_match_the_checker_on_the_widened_values(pkg, orc, dev, n):
    import torch
    rng = np.random.default_rng(300 + n)
    bits = _to_bf16_bits(3.0 * rng.standard_normal(n))
    wide = _widen(bits)
    xd = torch.from_numpy(bits.view(np.int16)).to(dev).view(torch.bfloat16)
    q, a = pkg.quantize_tensor(xd)
    torch.cuda.synchronize()
    amax = float(np.abs(wide).max()) if n else 0.0
    assert a.item() == np.float32(amax)
    if n:
        assert np.array_equal(q.cpu().numpy(), orc.quantize_i8(wide, amax))
        # and with the scale passed by value, ties and clamps included
        bits2 = _to_bf16_bits(np.array([0.5, -0.5, 1.5, 2.5, -2.5, 126.5, 127.0, 200.0, -200.0, 0.49609375], np.float32))
        x2 = torch.from_numpy(bits2.view(np.int16)).to(dev).view(torch.bfloat16)
        q2, _ = pkg.quantize_tensor(x2, amax=127.0)
        assert np.array_equal(q2.cpu().numpy(), orc.quantize_i8(_widen(bits2), 127.0))


@pytest.mark.parametrize("n", [0, 1, 9, 4096, 300001])
def test_bf16_dequantize_rounds_the_float_result_once(pkg, dev, n):
    import torch
    v = np.random.default_rng(400 + n).integers(-128, 128, n).astype(np.int8)
    amax = 3.3
    out = pkg.dequantize_tensor(_dev(dev, v), amax, dtype=torch.bfloat16)
    torch.cuda.synchronize()
    want = _to_bf16_bits(v.astype(np.float32) / np.float32(127.0) * np.float32(amax))
    assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), want)


def test_bf16_nan_is_skipped_and_quantises_to_zero(pkg, dev):
    import torch
    bits = np.array([0x7FC0, 0x3F80, 0xFFC1, 0xC000, 0x0000, 0x8000, 0x3F00, 0x4000, 0x7F80], np.uint16)  # NaN 1 NaN -2 0 -0 .5 2 inf
    xd = torch.from_numpy(bits.view(np.int16)).to(dev).view(torch.bfloat16)
    a = torch.zeros(1, dtype=torch.float32, device=dev)
    assert pkg.FMHAAbsMaxBF16(None, xd, bits.size, a) == pkg.FMHA_I8_OK
    q, _ = pkg.quantize_tensor(xd, amax=127.0)
    torch.cuda.synchronize()
    assert a.item() == float("inf")
    assert list(q.cpu().numpy()) == [0, 1, 0, -2, 0, 0, 1, 2, 127]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_float_in_float_out_flow_matches_the_host_flow(pkg, orc, dev, dtype_name):
    """fmha_infer_from_float does on the GPU what the reference's driver does around its kernel (quantise by abs-max,
    launch, de-quantise: test_fmha_i8.cpp:91-110,204-222, inc/utils.hpp:53).  Against the same flow on the host with
    the checker: the int8 tensors it feeds the kernel are bit-identical, the int8 O passes the usual gate, and the float
    O is that int8 O times o_amax / 127 exactly."""
    import torch
    dtype = getattr(torch, dtype_name)
    c = fc.make_inputs(2, 3, 320, 64, pad="scatter", seed=55)
    c["mask"][:, 0] = 0
    floats = [torch.from_numpy(c[n]).to(dev).to(dtype).contiguous() for n in ("qf", "kf", "vf")]
    host = [t.float().cpu().numpy() for t in floats]  # what the GPU really sees (bfloat16 rounds the inputs)
    amax = [orc.abs_max(x) for x in host]
    qi, ki, vi = (orc.quantize_i8(x, a) for x, a in zip(host, amax))
    o_amax = 0.75
    for full in (False, True):
        o_f, o_i8, got_amax = pkg.fmha_infer_from_float(*floats, torch.from_numpy(c["mask"]).to(dev), o_amax, full_range_p=full)
        torch.cuda.synchronize()
        assert list(got_amax) == [float(a) for a in amax]
        want = orc.fmha_i8_blockwise_cross(qi, ki, vi, c["mask"], *amax, o_amax, full_range_p=full)
        st = fc.parity_stats(o_i8.cpu().numpy(), want)
        assert st["within1"] >= 0.999 and st["max"] <= 2, (dtype_name, full, st)
        assert o_f.dtype == dtype
        expect = (o_i8.float().cpu() / 127.0 * o_amax).to(dtype)  # inc/utils.hpp:53, rounded once to the output type
        assert torch.equal(o_f.cpu(), expect)
