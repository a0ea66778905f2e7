"""GPU parity tests proper: the HIP kernel, called through the C ABI of libfmha_i8.so, against the CPU checker on the
same seeded inputs.  Gate (int8 O): within +-1 LSB on >= 99.9 % of elements and max |delta| <= 2."""
import glob
import os

import numpy as np
import pytest

import fmha_cases as fc

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
WITHIN1_MIN = 0.999  # tolerance of the gate, in fractions of elements within +-1 LSB
MAX_ABS_LSB = 2


def to_dev(dev, *arrays):
    import torch
    return [torch.from_numpy(np.ascontiguousarray(a)).to(dev) for a in arrays]


def gpu_run(pkg, dev, c, **scales):
    import torch
    s = dict(q_amax=c["q_amax"], k_amax=c["k_amax"], v_amax=c["v_amax"], o_amax=c["o_amax"])
    s.update(scales)
    q, k, v, m = to_dev(dev, c["q"], c["k"], c["v"], c["mask"])
    o = pkg.fmha_infer_i8(q, k, v, m, s["q_amax"], s["k_amax"], s["v_amax"], s["o_amax"])
    torch.cuda.synchronize()
    return o.cpu().numpy()


def cpu_run(orc, c, heads=None, **scales):
    s = dict(q_amax=c["q_amax"], k_amax=c["k_amax"], v_amax=c["v_amax"], o_amax=c["o_amax"])
    s.update(scales)
    # softmax blocks of 128 keys, or of 64 for the lengths that are not multiples of 128 (src/fmha_i8.cu:41-60)
    block = 128 if c["q"].shape[2] % 128 == 0 else 64
    return orc.fmha_i8_blockwise(c["q"], c["k"], c["v"], c["mask"], s["q_amax"], s["k_amax"], s["v_amax"], s["o_amax"],
                                 block=block, heads=heads)


def check(got, want, what):
    st = fc.parity_stats(got, want)
    print(what, st, flush=True)
    assert st["within1"] >= WITHIN1_MIN and st["max"] <= MAX_ABS_LSB, (what, st)
    return st


# ---- committed known-answer fixtures -----------------------------------------------------------------------------
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))


@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p) for p in FIXTURES])
def test_golden_fixture(pkg, dev, path):
    f = np.load(path)
    qa, ka, va, oa = (float(x) for x in f["amax"])
    c = dict(q=f["q"], k=f["k"], v=f["v"], mask=f["mask"], q_amax=qa, k_amax=ka, v_amax=va, o_amax=oa)
    check(gpu_run(pkg, dev, c), f["o"], os.path.basename(path))


# ---- the reference's own sweep (test_fmha_i8.cpp:295-309: B=H=1, d in {64,128}) on the 128-multiples, reference-style
# data (uniform +-0.5, V = |u|, scattered 20 % mask, o_amax measured from the float path), both criteria ---------------
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("S", [128, 256, 384, 512, 1024])
def test_reference_sweep(pkg, orc, dev, S, d):
    c = fc.make_inputs(1, 1, S, d, dist="reference", pad="scatter", seed=31)
    o_ref = orc.fmha_fp32(c["qf"], c["kf"], c["vf"], c["mask"])
    c["o_amax"] = orc.abs_max(o_ref)  # test_fmha_i8.cpp:161
    got = gpu_run(pkg, dev, c)
    check(got, cpu_run(orc, c), "sweep S=%d d=%d" % (S, d))
    dev_pct = orc.mean_rel_deviation_pct(got, o_ref, c["o_amax"])
    assert dev_pct < 20.0, dev_pct  # inc/utils.hpp:88


# ---- the reference's other lengths (src/fmha_i8.cu:41-60: 64, 192, 320, 448 run with 64-key softmax blocks), plus a
# longer odd multiple of 64; unmasked, scattered mask and a padded tail that leaves whole blocks masked -------------------
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("S", [64, 192, 320, 448, 1088])
@pytest.mark.parametrize("pad", ["none", "scatter", "tail"])
def test_sixty_four_key_blocks(pkg, orc, dev, S, d, pad):
    B, H = 2, 3
    if pad == "tail":
        c = fc.make_inputs(B, H, S, d, dist="normal", seed=77, valid_lengths=[S - 32, max(S - 160, 16)])
    else:
        c = fc.make_inputs(B, H, S, d, dist="normal", pad=pad, seed=77)
    check(gpu_run(pkg, dev, c), cpu_run(orc, c), "S=%d d=%d %s" % (S, d, pad))


def test_sixty_four_key_blocks_reference_sweep(pkg, orc, dev):
    # the reference driver's own sweep over its 64-multiples (test_fmha_i8.cpp:295-309), reference-style data
    for d in (64, 128):
        for S in (64, 192, 320, 448):
            c = fc.make_inputs(1, 1, S, d, dist="reference", pad="scatter", seed=31)
            o_ref = orc.fmha_fp32(c["qf"], c["kf"], c["vf"], c["mask"])
            c["o_amax"] = orc.abs_max(o_ref)
            got = gpu_run(pkg, dev, c)
            check(got, cpu_run(orc, c), "sweep64 S=%d d=%d" % (S, d))
            assert orc.mean_rel_deviation_pct(got, o_ref, c["o_amax"]) < 20.0


# ---- the five benchmark configurations -----------------------------------------------------------------------------
def test_config_c1_all_heads(pkg, orc, dev):
    c = fc.make_config("C1")
    check(gpu_run(pkg, dev, c), cpu_run(orc, c), "C1")


def test_config_c2_all_heads(pkg, orc, dev):
    c = fc.make_config("C2")
    assert c["mask"].any()
    check(gpu_run(pkg, dev, c), cpu_run(orc, c), "C2")


@pytest.mark.parametrize("name", ["C3", "C4", "C5"])
def test_large_configs_every_head(pkg, orc, dev, name):
    # full-size run on the GPU against the checker on EVERY (batch, head) pair; the checker spreads the heads over the
    # host's threads (C4 and C5 are 1.4e11 multiply-adds each: tens of seconds on 16 cores)
    c = fc.make_config(name)
    got = gpu_run(pkg, dev, c)
    want = cpu_run(orc, c)
    st = check(got, want, name + " all %d heads" % (c["q"].shape[0] * c["q"].shape[1]))
    assert st["n"] == got.size


# ---- size-independent properties at full benchmark size (no CPU pass needed) ----------------------------------------
def test_full_size_properties_c3(pkg, dev):
    import torch
    c = fc.make_config("C3")
    base = gpu_run(pkg, dev, c)
    # determinism: same call, same bits
    assert np.array_equal(gpu_run(pkg, dev, c), base)
    # head/batch independence: a [1,1] call on one head equals that head of the full call, bit for bit
    for b, h in ((0, 0), (3, 15), (2, 7)):
        one = dict(c, q=c["q"][b:b + 1, h:h + 1], k=c["k"][b:b + 1, h:h + 1], v=c["v"][b:b + 1, h:h + 1],
                   mask=c["mask"][b:b + 1])
        assert np.array_equal(gpu_run(pkg, dev, one)[0, 0], base[b, h])
    # only q_amax*k_amax and v_amax/o_amax matter
    alt = gpu_run(pkg, dev, c, q_amax=c["q_amax"] * 2, k_amax=c["k_amax"] / 2, v_amax=c["v_amax"] * 4, o_amax=4.0)
    assert np.array_equal(alt, base)
    # permuting the key blocks (K and V together) changes only float merge order
    S = c["q"].shape[2]
    order = np.random.default_rng(5).permutation(S // 128)
    idx = np.concatenate([np.arange(128) + 128 * b for b in order])
    perm = dict(c, k=np.ascontiguousarray(c["k"][:, :, idx]), v=np.ascontiguousarray(c["v"][:, :, idx]))
    st = fc.parity_stats(gpu_run(pkg, dev, perm), base)
    assert st["within1"] >= 0.9999 and st["max"] <= 1, st
    # Q == 0: uniform attention, closed form rne(clamp(v_amax/o_amax * mean V))
    z = dict(c, q=np.zeros_like(c["q"]))
    got = gpu_run(pkg, dev, z, v_amax=2.0, o_amax=1.0).astype(np.int64)
    y = 2.0 * c["v"].astype(np.float64).mean(axis=2, keepdims=True)
    want = np.broadcast_to(np.clip(np.rint(y), -127, 127), got.shape)
    assert np.abs(got - want).max() <= 1 and (got == want).mean() > 0.99
    del torch


@pytest.mark.parametrize("S,d", [(65536, 64), (65472, 64), (16384, 128)])
def test_longest_sequences_by_closed_forms(pkg, dev, S, d):
    """The longest sequences the library takes (512 key blocks of 128, or 1023 of 64): no CPU pass of that size finishes
    in seconds, so the checks are closed forms.  Q == 0 makes attention uniform over the unmasked keys, so that
    O = rne(clamp(v_amax/o_amax * mean V)); a one-key "needle" (one K row far closer to every Q row than the rest)
    makes O the V row of that key; determinism; and a masked tail must equal the sequence cut at the same place."""
    rng = np.random.default_rng(S + d)
    valid = S - 3 * 64 - 17  # the masked tail covers whole key blocks and a ragged part of one
    v = rng.integers(-127, 128, (1, 1, S, d), dtype=np.int8)
    k = rng.integers(-20, 21, (1, 1, S, d), dtype=np.int8)
    mask = np.zeros((1, S), np.int8)
    mask[0, valid:] = 1
    base = dict(k=k, v=v, mask=mask, q_amax=1.0, k_amax=1.0, v_amax=2.0, o_amax=1.0)
    # uniform attention over the valid keys
    got = gpu_run(pkg, dev, dict(base, q=np.zeros((1, 1, S, d), np.int8))).astype(np.int64)
    y = 2.0 * v[0, 0, :valid].astype(np.float64).mean(axis=0)
    want = np.broadcast_to(np.clip(np.rint(y), -127, 127), got.shape)
    assert np.abs(got - want).max() <= 1 and (got == want).mean() > 0.99
    assert np.array_equal(gpu_run(pkg, dev, dict(base, q=np.zeros((1, 1, S, d), np.int8))).astype(np.int64), got)
    # a needle: key j0 is the only one that matters (score 127*127*d against at most 127*20*d, scaled up by the amax
    # product), in a block in the middle of the sequence
    j0 = (valid // 2) | 1
    kn = k.copy()
    kn[0, 0, j0] = 127
    q = np.full((1, 1, S, d), 127, np.int8)
    got = gpu_run(pkg, dev, dict(base, q=q, k=kn, q_amax=30.0, k_amax=30.0, v_amax=1.0)).astype(np.int64)
    assert np.array_equal(got[0, 0], np.broadcast_to(v[0, 0, j0].astype(np.int64), (S, d)))
    # the same needle behind the mask is invisible: the result is then far from that V row
    kn2 = k.copy()
    kn2[0, 0, valid + 5] = 127
    got2 = gpu_run(pkg, dev, dict(base, q=q, k=kn2, q_amax=30.0, k_amax=30.0, v_amax=1.0)).astype(np.int64)
    assert not np.array_equal(got2[0, 0, 0], v[0, 0, valid + 5].astype(np.int64))


def test_full_size_mask_properties_c4(pkg, dev):
    c = fc.make_config("C4")
    base = gpu_run(pkg, dev, c)
    # keys behind the mask cannot change a bit
    rng = np.random.default_rng(6)
    c2 = dict(c, k=c["k"].copy(), v=c["v"].copy())
    c2["k"][:, :, 3840:] = rng.integers(-127, 128, c2["k"][:, :, 3840:].shape, dtype=np.int8)
    c2["v"][:, :, 3840:] = 127
    assert np.array_equal(gpu_run(pkg, dev, c2), base)
    # 3840 = 30 whole blocks: the first 3840 query rows equal the 3840-long unmasked problem
    short = dict(c, q=c["q"][:, :, :3840], k=c["k"][:, :, :3840], v=c["v"][:, :, :3840],
                 mask=np.zeros((1, 3840), np.int8))
    assert np.array_equal(gpu_run(pkg, dev, short), base[:, :, :3840])


# ---- edge cases ------------------------------------------------------------------------------------------------------
def test_all_masked_rows_give_zero_and_literal_all_ones_mask(pkg, orc, dev):
    c = fc.make_inputs(2, 2, 256, 64, seed=41, valid_lengths=[0, 256])
    got = gpu_run(pkg, dev, c)
    assert not got[0].any()
    check(got, cpu_run(orc, c), "batch 0 fully masked")
    ones = dict(c, mask=np.ones((2, 256), np.int8))  # "all ones" under the reference polarity masks everything
    assert not gpu_run(pkg, dev, ones).any()


@pytest.mark.parametrize("d", [64, 128])
def test_ragged_and_scattered_masks(pkg, orc, dev, d):
    # valid lengths that cut blocks at every kind of boundary, one key only, a hole in the middle, non-{0,1} bytes
    lens = [1, 127, 128, 129, 255, 300, 511, 512]
    c = fc.make_inputs(len(lens), 2, 512, d, seed=42, valid_lengths=lens)
    check(gpu_run(pkg, dev, c), cpu_run(orc, c), "ragged d=%d" % d)
    c = fc.make_inputs(3, 2, 512, d, seed=43, pad="scatter")
    c["mask"][1, 128:384] = 1          # two whole interior blocks masked
    c["mask"][2, :128] = 1             # the FIRST block fully masked (the reference kernel yields NaN here)
    c["mask"] = (c["mask"] * np.int8(-7)).astype(np.int8)  # any nonzero byte masks (inc/fmha_i8.cuh:191)
    check(gpu_run(pkg, dev, c), cpu_run(orc, c), "scattered d=%d" % d)


def test_unaligned_mask_pointer(pkg, orc, dev):
    import torch
    c = fc.make_inputs(1, 2, 256, 64, seed=44, valid_lengths=[200])
    q, k, v = to_dev(dev, c["q"], c["k"], c["v"])
    buf = torch.zeros(256 + 3, dtype=torch.int8, device=dev)
    buf[3:] = torch.from_numpy(c["mask"][0]).to(dev)
    o = torch.empty_like(q)
    st = pkg.FMHAInferI8Status(None, pkg.FMHAParamI8(c["q_amax"], c["k_amax"], c["v_amax"], 1.0),
                               pkg.AttnDataDescriptor(1, 256, 2, 64), q, k, v, buf.data_ptr() + 3, o, True)
    torch.cuda.synchronize()
    assert st == 0
    check(o.cpu().numpy(), cpu_run(orc, c), "mask at odd address")


def test_saturation_and_clamp(pkg, orc, dev):
    # heavy tails and v_amax > o_amax: a visible share of O sits at +-127 on both sides
    c = fc.make_inputs(2, 2, 384, 128, dist="student_t", sigma=0.5, seed=45)
    want = cpu_run(orc, c, v_amax=4 * c["v_amax"])
    assert (np.abs(want) == 127).mean() > 0.02
    check(gpu_run(pkg, dev, c, v_amax=4 * c["v_amax"]), want, "saturating")


@pytest.mark.parametrize("S,d", [(512, 128), (512, 64), (320, 128), (320, 64), (500, 128), (500, 64), (300, 128), (300, 64)])
@pytest.mark.parametrize("qk_scale,vo_ratio", [(1.0, 1.0), (1.0, 60.0), (40.0, 1.0), (40.0, 60.0)])
def test_every_kernel_variant(pkg, orc, dev, S, d, qk_scale, vo_ratio):
    """The library picks one of four arithmetic variants of the kernel from the scales (accumulators read as floats or
    converted; accumulator offset folded into the running O or not) for each head_dim, softmax block size (128 or 64
    keys) and for lengths with and without a partly filled last block.  A large q_amax*k_amax forces the converting
    variant, a large v_amax/o_amax the unfolded one: all thirty-two instantiations must meet the same gate."""
    c = fc.make_inputs(2, 2, S, d, dist="normal", pad="scatter", seed=91)
    kw = dict(q_amax=c["q_amax"] * qk_scale, v_amax=vo_ratio, o_amax=1.0 if vo_ratio == 1.0 else 2.0)
    s = dict(q_amax=c["q_amax"], k_amax=c["k_amax"], v_amax=c["v_amax"], o_amax=c["o_amax"])
    s.update(kw)
    want = orc.fmha_i8_blockwise_cross(c["q"], c["k"], c["v"], c["mask"], s["q_amax"], s["k_amax"], s["v_amax"], s["o_amax"])
    check(gpu_run(pkg, dev, c, **kw), want, "variant S=%d d=%d qk=%g vo=%g" % (S, d, qk_scale, vo_ratio))


@pytest.mark.parametrize("d", [64, 128])
def test_extreme_scores_stay_inside_the_float_window(pkg, orc, dev, d):
    """On the variant that reads the GEMM 1 accumulators as floats, the accumulators start inside a float binade and
    the largest possible |S| = 127*127*d must not leave it (at head_dim 64 the start value sits closer to the lower
    edge than at 128).  Rows of +-127 reach both extremes; a tiny score scale selects that variant and keeps the
    softmax non-trivial (x = S*c differs by a few units across keys)."""
    S = 256
    rng = np.random.default_rng(d)
    q = np.full((1, 2, S, d), 127, np.int8)
    q[0, 1, ::2] = -127
    k = np.where(rng.random((1, 2, S, 1)) < 0.5, 127, -127).astype(np.int8) * np.ones((1, 1, 1, d), np.int8)
    k[0, :, 5, :] = rng.integers(-127, 128, (2, d))  # one ordinary key per head
    v = rng.integers(-127, 128, (1, 2, S, d)).astype(np.int8)
    mask = np.zeros((1, S), np.int8)
    mask[0, 200:230] = 1
    c = dict(q=q, k=k, v=v, mask=mask, q_amax=0.02, k_amax=0.02, v_amax=1.0, o_amax=1.0)
    want = cpu_run(orc, c)
    check(gpu_run(pkg, dev, c), want, "extreme scores d=%d" % d)


# Key blocks come in three kinds - no masked key (P), some (M), all (F) - and the kernel serves them with three loops
# (a steady-state loop for runs of P, a second one from the first M on, a general loop for F blocks and the last
# block); masked keys of an M block are handled where GEMM 1 starts its accumulators.  Every transition between the
# loops, at both head sizes and both block sizes, full-range P included; a masked key also carries the largest score
# of its row (K = Q there), so that a mask that is ignored cannot go unnoticed.
BLOCK_PATTERNS = ["PMPF", "MPPM", "FPMP", "PPFM", "MMMM", "FFPF", "PFFM", "MFMP", "PPPM", "MPPP", "PMMPPFMP", "F", "M", "FM", "MF"]


@pytest.mark.parametrize("d,block", [(128, 128), (64, 128), (128, 64), (64, 64)])
@pytest.mark.parametrize("full_range_p", [False, True])
def test_every_sequence_of_block_kinds(pkg, orc, dev, d, block, full_range_p):
    import torch
    rng = np.random.default_rng([d, block, int(full_range_p)])
    for pattern in BLOCK_PATTERNS:
        n = len(pattern)
        S = n * block
        pattern_here = pattern
        if block == 64 and S % 128 == 0:  # (a multiple of 128 runs blocks of 128 keys: one more block of 64)
            pattern_here, S = pattern + "P", S + 64
        if block == 128 and S % 128 != 0:
            continue
        B, H = 2, 2
        c = fc.make_inputs(B, H, S, d, dist="normal", sigma=1.0, pad="none", seed=int(rng.integers(1 << 30)))
        mask = np.zeros((B, S), np.int8)
        for b in range(B):
            for i, kind in enumerate(pattern_here if b == 0 else pattern_here[::-1]):
                lo = i * block
                if kind == "F":
                    mask[b, lo:lo + block] = 1
                elif kind == "M":
                    mask[b, lo:lo + block] = (rng.random(block) < 0.3).astype(np.int8)
                    mask[b, lo + int(rng.integers(block))] = 0   # at least one key stays
                    mask[b, lo + int(rng.integers(block))] = 3   # ... and one goes, with a byte other than 1
        c["mask"] = mask
        # masked keys that would win every maximum: K row = Q row of the same position, scaled up
        kq = np.clip(c["q"].astype(np.int32) * 2, -127, 127).astype(np.int8)
        for b in range(B):
            gone = np.nonzero(mask[b])[0][::7]
            c["k"][b][:, gone, :] = kq[b][:, gone, :]
        q, k, v, m = to_dev(dev, c["q"], c["k"], c["v"], c["mask"])
        o = pkg.fmha_infer_i8(q, k, v, m, c["q_amax"], c["k_amax"], c["v_amax"], c["o_amax"], full_range_p=full_range_p)
        torch.cuda.synchronize()
        blk = 128 if S % 128 == 0 else 64
        if full_range_p:
            want = orc.fmha_i8_blockwise_cross(c["q"], c["k"], c["v"], c["mask"], c["q_amax"], c["k_amax"], c["v_amax"],
                                               c["o_amax"], block=blk, full_range_p=True)
        else:
            want = orc.fmha_i8_blockwise(c["q"], c["k"], c["v"], c["mask"], c["q_amax"], c["k_amax"], c["v_amax"],
                                         c["o_amax"], block=blk)
        check(o.cpu().numpy(), np.asarray(want).reshape(o.shape), "blocks %s d=%d block=%d full=%s" % (pattern_here, d, blk, full_range_p))


@pytest.mark.parametrize("S,d", [(256, 128), (192, 64)])
def test_zero_scale_with_masked_keys(pkg, orc, dev, S, d):
    """q_amax = 0 (an all-zero Q tensor quantised by abs-max): every score scales to 0, the softmax is uniform over the
    unmasked keys, and a masked key must still weigh exactly nothing."""
    c = fc.make_inputs(1, 2, S, d, pad="scatter", seed=46)
    got = gpu_run(pkg, dev, c, q_amax=0.0, v_amax=2.0, o_amax=1.0).astype(np.int64)
    keep = c["mask"][0] == 0
    y = 2.0 * c["v"][:, :, keep, :].astype(np.float64).mean(axis=2, keepdims=True)
    assert np.abs(got - np.clip(np.rint(y), -127, 127)).max() <= 1
    check(got, cpu_run(orc, c, q_amax=0.0, v_amax=2.0, o_amax=1.0), "zero scale S=%d d=%d" % (S, d))


def test_negative_score_scale_is_refused(pkg, dev):
    import torch
    c = fc.make_inputs(1, 1, 128, 64, seed=47)
    q, k, v, m = to_dev(dev, c["q"], c["k"], c["v"], c["mask"])
    o = torch.full_like(q, 55)
    P = pkg.FMHAParamI8(-1.0, 1.0, 1.0, 1.0, 1.0)
    assert pkg.FMHAInferI8Status(None, P, pkg.AttnDataDescriptor(1, 128, 1, 64), q, k, v, m, o) == pkg.FMHA_I8_ERR_SCALE
    P = pkg.FMHAParamI8(-1.0, -1.0, 1.0, 1.0, 1.0)  # the product is what scales the scores
    assert pkg.FMHAInferI8CheckArgs(P, pkg.AttnDataDescriptor(1, 128, 1, 64), q, k, v, m, o) == pkg.FMHA_I8_OK
    torch.cuda.synchronize()
    assert (o == 55).all().item()


def test_exponent_offsets_of_the_order_of_a_hundred_thousand(pkg, orc, dev):
    """Heavy-tailed Q, K and a forty-fold score scale: block maxima of 10^5 in base-2 units, where one unit in the last
    place of the offset is a percent of p.  The largest p of a row must still quantise to at most 128 in magnitude (it
    once reached 129, whose low byte is +127: two rows of this very problem came out with the wrong sign)."""
    import torch
    c = fc.make_inputs(2, 3, 1152, 64, dist="student_t", sigma=1.0, seed=1128)
    q = fc.make_inputs(2, 3, 470, 64, seed=5128)["q"]
    scales = (c["q_amax"] * 40.0, c["k_amax"], c["v_amax"], 1.0)
    want = orc.fmha_i8_blockwise_cross(q, c["k"], c["v"], c["mask"], *scales)
    t = to_dev(dev, q, c["k"], c["v"], c["mask"])
    got = pkg.fmha_infer_i8(*t, *scales)
    torch.cuda.synchronize()
    check(got.cpu().numpy(), want, "large offsets")


def test_masked_sentinel_corner(pkg, orc, dev):
    # every unmasked score of a partially masked block lies below the -1,000,000 substituted for masked keys
    S, d = 128, 128
    rng = np.random.default_rng(46)
    q = np.full((1, 1, S, d), 127, np.int8)
    k = np.full((1, 1, S, d), -127, np.int8)
    k[0, 0, ::2, :64] = -100
    v = rng.integers(-127, 128, (1, 1, S, d), dtype=np.int8)
    mask = np.zeros((1, S), np.int8)
    mask[0, 100:] = 1
    a = float(np.sqrt(0.18))
    c = dict(q=q, k=k, v=v, mask=mask, q_amax=a, k_amax=a, v_amax=1.0, o_amax=1.0)
    check(gpu_run(pkg, dev, c), cpu_run(orc, c), "sentinel")


def test_one_hot_attention_closed_form_on_gpu(pkg, dev):
    S = d = 128
    rng = np.random.default_rng(47)
    perm = rng.permutation(d)
    k = np.zeros((1, 1, S, d), np.int8)
    q = np.zeros((1, 1, S, d), np.int8)
    k[0, 0, np.arange(S), np.arange(S)] = 127
    q[0, 0, np.arange(S), perm] = 127
    v = rng.integers(-127, 128, (1, 1, S, d), dtype=np.int8)
    c = dict(q=q, k=k, v=v, mask=np.zeros((1, S), np.int8), q_amax=30.0, k_amax=30.0, v_amax=2.0, o_amax=1.0)
    want = np.clip(2 * v[0, 0, perm].astype(np.int64), -127, 127)
    assert np.array_equal(gpu_run(pkg, dev, c)[0, 0], want)


# ---- API behaviour -----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("B,H,S,d,pad", [(4, 16, 1024, 128, "none"), (2, 4, 2048, 128, "tail256"), (1, 3, 1337, 128, "scatter"),
                                         (2, 2, 2048, 64, "none"), (1, 2, 704, 64, "scatter")])
def test_back_to_back_launches_write_the_same_bytes(pkg, dev, B, H, S, d, pad):
    # The K/V tiles live in a ring of LDS stages that is refilled while other wavefronts still compute: a stage
    # refilled too early, or read before it is published, would show as launches of one problem that differ.  200
    # launches back to back into alternating output buffers, every one compared with the first on the GPU.
    import torch
    Sp = (S + 63) // 64 * 64
    c = fc.make_inputs(B, H, Sp, d, pad="scatter" if pad == "scatter" else pad, seed=77)
    q, k, v = (np.ascontiguousarray(c[n][:, :, :S]) for n in ("q", "k", "v"))
    m = np.ascontiguousarray(c["mask"][:, :S])
    m[:, 0] = 0
    tq, tk, tv, tm = to_dev(dev, q, k, v, m)
    outs = [torch.empty_like(tq), torch.empty_like(tq), torch.empty_like(tq)]
    args = (c["q_amax"], c["k_amax"], c["v_amax"], c["o_amax"])
    pkg.fmha_infer_i8(tq, tk, tv, tm, *args, out=outs[0])
    differing = torch.zeros((), dtype=torch.int64, device=dev)
    for it in range(200):
        o = outs[1 + it % 2]
        pkg.fmha_infer_i8(tq, tk, tv, tm, *args, out=o)
        differing += (o != outs[0]).sum()
    torch.cuda.synchronize()
    assert int(differing.item()) == 0


def test_void_entry_point_streams_and_use_tcu_flag(pkg, orc, dev):
    import torch
    c = fc.make_inputs(2, 2, 256, 128, seed=48, valid_lengths=[256, 100])
    q, k, v, m = to_dev(dev, c["q"], c["k"], c["v"], c["mask"])
    want = cpu_run(orc, c)
    P = pkg.FMHAParamI8(c["q_amax"], c["k_amax"], c["v_amax"], c["o_amax"], 123.0)  # s_max is ignored
    A = pkg.AttnDataDescriptor(2, 256, 2, 128)
    side = torch.cuda.Stream(device=dev)
    for use_tcu, stream in ((True, None), (False, side)):
        o = torch.zeros_like(q)
        if stream is not None:
            stream.wait_stream(torch.cuda.current_stream(dev))
        pkg.FMHAInferI8(stream, P, A, q, k, v, m, o, use_tcu)  # the reference's signature: returns nothing
        torch.cuda.synchronize()
        check(o.cpu().numpy(), want, "void entry use_tcu=%s" % use_tcu)


def test_concurrent_host_threads_on_their_own_streams(pkg, dev):
    """The library keeps no state between calls (the reference's launch function has none either, src/fmha_i8.cu:157-173),
    so any host thread may call it: four threads, each with its own stream, problem and buffers, two hundred calls each
    of both entry points, all at once; every thread must end with exactly the bytes a single-threaded call gives."""
    import threading
    import torch
    problems = []
    for t in range(4):
        c = fc.make_inputs(2, 2 + t, 256 + 64 * t, 64 if t % 2 else 128, pad="scatter", seed=90 + t)
        c["mask"][:, 0] = 0
        bufs = to_dev(dev, c["q"], c["k"], c["v"], c["mask"])
        scales = (c["q_amax"], c["k_amax"], c["v_amax"], c["o_amax"])
        want = [pkg.fmha_infer_i8(*bufs, *scales, full_range_p=full).cpu().numpy() for full in (False, True)]
        problems.append((bufs, scales, want))
    torch.cuda.synchronize()
    errors = []

    def worker(t):
        try:
            bufs, scales, want = problems[t]
            stream = torch.cuda.Stream(device=dev)
            outs = [torch.empty_like(bufs[0]), torch.empty_like(bufs[0])]
            for _ in range(200):
                for full in (False, True):
                    pkg.fmha_infer_i8(*bufs, *scales, out=outs[full], stream=stream, full_range_p=full)
            stream.synchronize()
            for full in (False, True):
                if not np.array_equal(outs[full].cpu().numpy(), want[full]):
                    errors.append("thread %d, full_range_p=%s: output differs" % (t, full))
        except Exception as e:  # noqa: BLE001 - reported by the main thread
            errors.append("thread %d: %r" % (t, e))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=120)
    assert not any(th.is_alive() for th in threads), "a worker did not finish"
    assert not errors, errors


def test_graph_capture_and_replay(pkg, orc, dev):
    """The call allocates nothing and never synchronises, so it can be recorded into a HIP graph: capture one launch,
    replay it several times with eager work and synchronisations in between and with new inputs written into the same
    buffers, and check every replay against the eager result."""
    import torch
    c = fc.make_inputs(2, 2, 384, 128, dist="normal", pad="scatter", seed=61)
    q, k, v, m = to_dev(dev, c["q"], c["k"], c["v"], c["mask"])
    o = torch.zeros_like(q)
    P = pkg.FMHAParamI8(c["q_amax"], c["k_amax"], c["v_amax"], c["o_amax"])
    A = pkg.AttnDataDescriptor(2, 384, 2, 128)
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    with torch.cuda.stream(side):
        assert pkg.FMHAInferI8Status(side, P, A, q, k, v, m, o, True) == 0  # warm-up outside the capture
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        assert pkg.FMHAInferI8Status(torch.cuda.current_stream(dev), P, A, q, k, v, m, o, True) == 0
    want = cpu_run(orc, c)
    for rep in range(4):
        if rep == 2:  # new inputs in the same buffers: the graph holds pointers, not data
            c = fc.make_inputs(2, 2, 384, 128, dist="normal", pad="scatter", seed=62)
            for dst, name in ((q, "q"), (k, "k"), (v, "v"), (m, "mask")):
                dst.copy_(torch.from_numpy(c[name]))
            want = cpu_run(orc, dict(c, q_amax=P.q_amax, k_amax=P.k_amax, v_amax=P.v_amax, o_amax=P.o_amax))
        o.fill_(77)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        eager = pkg.fmha_infer_i8(q, k, v, m, P.q_amax, P.k_amax, P.v_amax, P.o_amax)
        torch.cuda.synchronize()
        assert torch.equal(o, eager), rep
        check(o.cpu().numpy(), want, "graph replay %d" % rep)


def test_stale_error_of_an_unrelated_call_is_neither_reported_nor_cleared(pkg, orc, dev):
    """The status is that of this call's own launch.  An earlier failure of an unrelated HIP call (here hipSetDevice on
    a device that does not exist: host-side, no GPU work) must not come back as this call's status, the call must still
    do its work, and the stale error must still be there for the caller afterwards."""
    import ctypes
    import torch
    hip = ctypes.CDLL(os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so"))
    hip.hipGetLastError.restype = ctypes.c_int
    hip.hipSetDevice.restype = ctypes.c_int
    c = fc.make_inputs(1, 2, 256, 64, seed=77)
    q, k, v, m = to_dev(dev, c["q"], c["k"], c["v"], c["mask"])
    o = torch.zeros_like(q)
    torch.cuda.synchronize()
    P = pkg.FMHAParamI8(c["q_amax"], c["k_amax"], c["v_amax"], c["o_amax"], 1.0)
    A = pkg.AttnDataDescriptor(1, 256, 2, 64)
    stream = torch.cuda.current_stream(dev)
    hip.hipGetLastError()  # start clean
    stale = hip.hipSetDevice(9999)
    assert stale != 0
    try:
        status = pkg.FMHAInferI8Status(stream, P, A, q, k, v, m, o, True)
        left = hip.hipGetLastError()  # reads and clears what the caller would have seen
    finally:
        hip.hipGetLastError()
    assert status == pkg.FMHA_I8_OK, pkg.status_string(status)
    assert left == stale, "the caller's pending error was swallowed"
    torch.cuda.synchronize()
    check(o.cpu().numpy(), cpu_run(orc, c), "after a stale error")
    # the quantisation entry points follow the same rule
    x = torch.randn(4096, device=dev)
    amax = torch.zeros(1, device=dev)
    torch.cuda.synchronize()
    assert hip.hipSetDevice(9999) != 0
    try:
        status = pkg.FMHAAbsMaxF32(stream, x, x.numel(), amax)
    finally:
        hip.hipGetLastError()
    assert status == pkg.FMHA_I8_OK
    torch.cuda.synchronize()
    assert float(amax) == float(x.abs().max())


def test_unsupported_shapes_leave_output_untouched(pkg, dev):
    import torch
    q = torch.zeros(1, 1, 160, 64, dtype=torch.int8, device=dev)
    m = torch.zeros(1, 160, dtype=torch.int8, device=dev)
    o = torch.full_like(q, 55)
    P = pkg.FMHAParamI8(1, 1, 1, 1)
    assert pkg.FMHAInferI8Status(None, P, pkg.AttnDataDescriptor(1, 65537, 1, 64), q, q, q, m, o) == \
        pkg.FMHA_I8_ERR_SEQ_LEN
    pkg.FMHAInferI8(None, P, pkg.AttnDataDescriptor(1, 128, 1, 96), q, q, q, m, o, True)  # prints, launches nothing
    torch.cuda.synchronize()
    assert bool((o == 55).all())
    with pytest.raises(pkg.FMHAError):
        pkg.fmha_infer_i8(q, q, q, m, 1.0, 1.0, 1.0, o_amax=0.0)


# ---- the C++ harness (host C++ calling the C ABI the way the reference's driver calls its launch function) -------------
def test_cpp_harness_config1_and_reference_sweep(tmp_path):
    import json
    import subprocess
    exe = os.path.join(HERE, "bin", "test_fmha_i8")
    assert os.path.exists(exe), "tests/bin/test_fmha_i8 is not built (python -c 'import __graft_entry__ as g; g.build()')"
    js = str(tmp_path / "harness.json")
    r = subprocess.run([exe, "--config", "1", "--sweep", "--iters", "20", "--warmup", "20", "--cpu-heads", "0", "--json", js],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    print(r.stdout[-3000:])
    assert r.returncode == 0
    recs = [json.loads(l) for l in open(js)]
    assert len(recs) == 23 and all(x["pass"] for x in recs)
    assert all(x["mean_rel_dev_pct"] < 20.0 for x in recs if x["case"] == "sweep")
