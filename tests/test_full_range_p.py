"""P on all 255 steps of a byte - the "uint8 x int8" variant that the reference lists as planned (README.md:15,186)
and has no code for.  Nothing in the reference computes it, so its checker mode (P = rne(255 p), every 128 of the
pipeline of inc/fmha_i8.cuh:241,298,318 replaced by 255) is pinned by what the mathematics fixes: the closed forms of
uniform and one-hot attention, mask invariance, an independent numpy restatement, and the property that gives the
variant its point - its output lies closer to unquantised attention than the 128-step output does.  The GPU tests
hold FMHAInferI8CrossFullRangeP to that checker with the usual gate."""
import numpy as np
import pytest

import fmha_cases as fc
import np_model

WITHIN1_MIN = 0.999
MAX_ABS_LSB = 2


def _scales(c):
    return c["q_amax"], c["k_amax"], c["v_amax"], c["o_amax"]


def _full(orc, c, **kw):
    s = dict(q_amax=c["q_amax"], k_amax=c["k_amax"], v_amax=c["v_amax"], o_amax=c["o_amax"])
    s.update(kw)
    return orc.fmha_i8_blockwise_cross(c["q"], c["k"], c["v"], c["mask"], s["q_amax"], s["k_amax"], s["v_amax"],
                                       s["o_amax"], full_range_p=True)


def _gate(got, want, what):
    st = fc.parity_stats(got, want)
    assert st["within1"] >= WITHIN1_MIN and st["max"] <= MAX_ABS_LSB, (what, st)
    return st


# ---- the checker mode ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("S,d,valid", [(128, 64, 128), (256, 128, 129), (384, 64, 200), (100, 128, 77)])
def test_checker_uniform_attention_closed_form(orc, S, d, valid):
    # Q == 0: p = 1 and P = 255 on every unmasked key, so O = rne(v_amax/o_amax * mean of the unmasked V rows)
    c = fc.make_inputs(1, 2, (S + 63) // 64 * 64, d, seed=71)
    c = dict(c, q=np.zeros_like(c["q"][:, :, :S]), k=c["k"][:, :, :S], v=c["v"][:, :, :S])
    c["mask"] = np.zeros((1, S), np.int8)
    c["mask"][:, valid:] = 1
    got = _full(orc, c, v_amax=3.0, o_amax=1.5).astype(np.int64)
    y = 2.0 * c["v"][:, :, :valid].astype(np.float64).mean(axis=2, keepdims=True)
    want = np.broadcast_to(np.clip(np.rint(y), -127, 127), got.shape)
    near_tie = np.broadcast_to(np.abs(np.abs(y - np.floor(y)) - 0.5) < 1e-3, got.shape)
    assert np.array_equal(got[~near_tie], want[~near_tie]) and np.abs(got - want).max() <= 1


def test_checker_one_hot_attention_closed_form(orc):
    # every query selects one key per block with p = 1 (P = 255), all others underflow to 0:
    # O = rne(clamp(2 * mean of the selected V rows)), exactly, ties and clamp included
    S, d = 256, 128
    rng = np.random.default_rng(72)
    perm = rng.permutation(d)
    k = np.zeros((1, 1, S, d), np.int8)
    q = np.zeros((1, 1, S, d), np.int8)
    for j in range(S):
        k[0, 0, j, j % d] = 127
        q[0, 0, j, perm[j % d]] = 127
    v = rng.integers(-127, 128, (1, 1, S, d), dtype=np.int8)
    got = orc.fmha_i8_blockwise_cross(q, k, v, np.zeros((1, S), np.int8), 30.0, 30.0, 2.0, 1.0,
                                      full_range_p=True).astype(np.int64)
    sel = np.stack([v[0, 0, perm[np.arange(S) % d] + blk * d, :].astype(np.float64) for blk in range(S // d)])
    want = np.clip(np.rint(2.0 * sel.mean(axis=0)), -127, 127)
    assert np.array_equal(got[0, 0], want) and (np.abs(want) == 127).any()


def test_checker_masked_keys_do_not_matter(orc):
    c = fc.make_inputs(2, 2, 384, 64, pad="scatter", seed=73)
    ref = _full(orc, c)
    rng = np.random.default_rng(74)
    other = dict(c, k=c["k"].copy(), v=c["v"].copy())
    gone = c["mask"] != 0
    for b in range(2):
        other["k"][b][:, gone[b]] = rng.integers(-127, 128, other["k"][b][:, gone[b]].shape)
        other["v"][b][:, gone[b]] = rng.integers(-127, 128, other["v"][b][:, gone[b]].shape)
    assert np.array_equal(_full(orc, other), ref)
    c["mask"][:] = 1
    assert not _full(orc, c).any()  # no key left: zeros


@pytest.mark.parametrize("S,d,pad,dist", [(128, 64, "none", "normal"), (256, 128, "scatter", "normal"),
                                         (384, 64, "bert", "student_t"), (512, 128, "tail256", "normal")])
def test_checker_against_independent_numpy_model(orc, S, d, pad, dist):
    c = fc.make_inputs(2, 2, S, d, dist=dist, pad=pad, seed=75)
    want = np_model.fmha_i8(c["q"], c["k"], c["v"], c["mask"], *_scales(c), full_range_p=True)
    st = fc.parity_stats(orc.fmha_i8_blockwise_cross(c["q"], c["k"], c["v"], c["mask"], *_scales(c), block=128,
                                                     full_range_p=True), want)
    assert st["exact"] >= 0.999 and st["max"] <= 1, st


def test_checker_full_range_is_a_different_and_finer_quantisation(orc):
    # against float64 attention on the de-quantised inputs, with an output scale fine enough to see P's resolution:
    # the 255-step output is the closer one, and the two outputs are not the same bytes
    c = fc.make_inputs(2, 4, 1024, 64, seed=76)
    deq = [c[n].astype(np.float64) * c[n + "_amax"] / 127.0 for n in ("q", "k", "v")]
    o64 = np_model.attention_fp64(deq[0], deq[1], deq[2], c["mask"])
    o_amax = float(np.abs(o64).max())
    want = o64 * 127.0 / o_amax
    narrow = orc.fmha_i8_blockwise_cross(c["q"], c["k"], c["v"], c["mask"], c["q_amax"], c["k_amax"], c["v_amax"], o_amax)
    full = _full(orc, c, o_amax=o_amax)
    err_narrow = np.abs(narrow - want).mean()
    err_full = np.abs(full - want).mean()
    assert not np.array_equal(narrow, full)
    assert err_full < err_narrow and err_full < 0.5, (err_full, err_narrow)


# ---- the HIP kernel ------------------------------------------------------------------------------------------------
def _gpu(pkg, dev, c, scales=None):
    import torch
    t = [torch.from_numpy(np.ascontiguousarray(c[n])).to(dev) for n in ("q", "k", "v", "mask")]
    o = pkg.fmha_infer_i8(*t, *(scales or _scales(c)), full_range_p=True)
    torch.cuda.synchronize()
    return o.cpu().numpy()


@pytest.mark.gpu
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("S,pad", [(128, "none"), (64, "none"), (192, "scatter"), (512, "bert"), (1024, "none"),
                                   (1152, "scatter"), (2048, "tail256")])
def test_full_range_p_against_the_checker(pkg, orc, dev, S, d, pad):
    c = fc.make_inputs(2, 3, S, d, pad=pad, seed=77)
    _gate(_gpu(pkg, dev, c), _full(orc, c), "S=%d d=%d %s" % (S, d, pad))


@pytest.mark.gpu
def test_full_range_p_closed_forms_on_the_gpu(pkg, dev):
    # uniform attention: exactly rne(v_amax/o_amax * mean(V)) - every P is 255, the column sums carry the whole result
    c = fc.make_inputs(2, 2, 640, 128, seed=78, valid_lengths=[640, 333])
    c["q"][:] = 0
    got = _gpu(pkg, dev, c, (1.0, 1.0, 3.0, 1.5)).astype(np.int64)
    for b, valid in enumerate((640, 333)):
        y = 2.0 * c["v"][b, :, :valid].astype(np.float64).mean(axis=1, keepdims=True)
        want = np.broadcast_to(np.clip(np.rint(y), -127, 127), got[b].shape)
        near_tie = np.broadcast_to(np.abs(np.abs(y - np.floor(y)) - 0.5) < 1e-3, got[b].shape)
        assert np.array_equal(got[b][~near_tie], want[~near_tie]) and np.abs(got[b] - want).max() <= 1


@pytest.mark.gpu
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("S", [1, 5, 63, 100, 129, 255, 1000, 2049])
def test_full_range_p_any_key_and_query_count(pkg, orc, dev, S, d):
    B, H = 2, 2
    c = fc.make_inputs(B, H, (S + 63) // 64 * 64, d, pad="scatter" if S > 8 else "none", seed=79)
    c["mask"][:, 0] = 0
    for Sq in sorted({S, 77, 300}):
        cc = dict(c, q=fc.make_inputs(B, H, Sq, d, seed=80)["q"], k=np.ascontiguousarray(c["k"][:, :, :S]),
                  v=np.ascontiguousarray(c["v"][:, :, :S]), mask=np.ascontiguousarray(c["mask"][:, :S]))
        _gate(_gpu(pkg, dev, cc), _full(orc, cc), "S=%d Sq=%d d=%d" % (S, Sq, d))


@pytest.mark.gpu
def test_full_range_p_every_kernel_variant(pkg, orc, dev):
    """Score scales on both sides of the switch between the two ways the scores are read, output scales on both sides
    of the switch between the two ways the running O is kept, blocks of 128 and of 64 keys, full and ragged ends,
    both head sizes: the sixteen x two full-range instantiations of the kernel."""
    for d in (64, 128):
        for S in (256, 320, 250, 300):
            c = fc.make_inputs(2, 2, (S + 63) // 64 * 64, d, pad="scatter", seed=81)
            c["mask"][:, 0] = 0
            c = dict(c, k=np.ascontiguousarray(c["k"][:, :, :S]), v=np.ascontiguousarray(c["v"][:, :, :S]),
                     mask=np.ascontiguousarray(c["mask"][:, :S]), q=fc.make_inputs(2, 2, 200, d, seed=82)["q"])
            for q_scale in (1.0, 60.0):
                for v_amax, o_amax in ((c["v_amax"], 1.0), (8.0, 0.25)):
                    scales = (c["q_amax"] * q_scale, c["k_amax"], v_amax, o_amax)
                    want = orc.fmha_i8_blockwise_cross(c["q"], c["k"], c["v"], c["mask"], *scales, full_range_p=True)
                    st = fc.parity_stats(_gpu(pkg, dev, c, scales), want)
                    # (with v_amax/o_amax = 32 one output LSB is a 32nd of a V step: the gate is wider there)
                    limit = 2 if v_amax / o_amax < 8 else 6
                    assert st["max"] <= limit and st["within1"] >= (0.999 if limit == 2 else 0.97), (d, S, scales, st)


@pytest.mark.gpu
def test_full_range_p_random_shapes(pkg, orc, dev):
    rng = np.random.default_rng(2025)
    for it in range(40):
        d = int(rng.choice([64, 128]))
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        S = int(rng.choice([rng.integers(1, 130), rng.integers(1, 700), rng.integers(500, 2600), 64 * rng.integers(1, 40)]))
        Sq = S if rng.random() < 0.4 else int(rng.choice([rng.integers(1, 70), rng.integers(1, 600), rng.integers(200, 1500)]))
        pad = str(rng.choice(["none", "scatter", "tail", "dead"]))
        c = fc.make_inputs(B, H, (S + 63) // 64 * 64, d, pad="scatter" if pad == "scatter" else "none", seed=3000 + it,
                           dist=str(rng.choice(["normal", "student_t"])), sigma=float(rng.choice([0.5, 1.0])))
        mask = c["mask"][:, :S].copy()
        if pad == "tail":
            for b in range(B):
                mask[b, int(rng.integers(1, S + 1)):] = 1
        if pad == "dead" and S > 256:
            a = int(rng.integers(0, S - 130))
            mask[:, a:a + int(rng.integers(64, 400))] = 1
        mask[:, 0] = 0
        cc = dict(c, q=fc.make_inputs(B, H, Sq, d, seed=7000 + it)["q"], k=np.ascontiguousarray(c["k"][:, :, :S]),
                  v=np.ascontiguousarray(c["v"][:, :, :S]), mask=mask)
        scales = (c["q_amax"] * float(rng.choice([1, 1, 8, 40])), c["k_amax"], c["v_amax"], float(rng.choice([1.0, 2.0])))
        print("case", it, B, H, Sq, S, d, pad, flush=True)
        want = orc.fmha_i8_blockwise_cross(cc["q"], cc["k"], cc["v"], mask, *scales, full_range_p=True)
        _gate(_gpu(pkg, dev, cc, scales), want, "case %d" % it)


@pytest.mark.gpu
def test_full_range_p_at_the_benchmark_shape(pkg, orc, dev):
    # B4 H16 S1024 d128: four heads against the checker, and the output differs from the 128-step kernel's
    import torch
    c = fc.make_config("C3")
    got = _gpu(pkg, dev, c)
    heads = slice(0, 4)
    cut = dict(c, q=c["q"][:1, heads], k=c["k"][:1, heads], v=c["v"][:1, heads], mask=c["mask"][:1])
    _gate(got[:1, heads], _full(orc, cut), "C3 heads 0..3")
    t = [torch.from_numpy(c[n]).to(dev) for n in ("q", "k", "v", "mask")]
    narrow = pkg.fmha_infer_i8(*t, *_scales(c)).cpu().numpy()
    delta = np.abs(narrow.astype(int) - got.astype(int))
    assert delta.max() <= 2 and 0 < (delta != 0).mean() < 0.5
    assert np.array_equal(_gpu(pkg, dev, c), got)  # the same bytes on a second call


@pytest.mark.gpu
def test_full_range_p_exponent_offsets_of_the_order_of_a_hundred_thousand(pkg, orc, dev):
    """Heavy-tailed Q, K and a forty-fold score scale: block maxima of 10^5 in base-2 units, where one unit in the last
    place of the exponent offset is a percent of p.  The largest p of a row must quantise to at most 255: a 256 would
    wrap to the byte 0 and drop the very key the row attends to most."""
    c = fc.make_inputs(2, 3, 1152, 64, dist="student_t", sigma=1.0, seed=1128)
    c = dict(c, q=fc.make_inputs(2, 3, 470, 64, seed=5128)["q"])
    scales = (c["q_amax"] * 40.0, c["k_amax"], c["v_amax"], 1.0)
    want = orc.fmha_i8_blockwise_cross(c["q"], c["k"], c["v"], c["mask"], *scales, full_range_p=True)
    _gate(_gpu(pkg, dev, c, scales), want, "large offsets")


@pytest.mark.gpu
@pytest.mark.parametrize("S,d", [(65536, 64), (16384, 128)])
def test_full_range_p_longest_sequences_by_closed_forms(pkg, dev, S, d):
    """The longest sequences the library takes: no CPU pass of that size finishes in seconds, so the checks are closed
    forms.  Q == 0: attention is uniform over the unmasked keys, every P is 255 and the column sums carry half the
    result; a one-key needle: O is the V row of that key, exactly."""
    rng = np.random.default_rng(S + d + 1)
    valid = S - 3 * 64 - 17
    v = rng.integers(-127, 128, (1, 1, S, d), dtype=np.int8)
    k = rng.integers(-20, 21, (1, 1, S, d), dtype=np.int8)
    mask = np.zeros((1, S), np.int8)
    mask[0, valid:] = 1
    got = _gpu(pkg, dev, dict(q=np.zeros((1, 1, S, d), np.int8), k=k, v=v, mask=mask), (1.0, 1.0, 2.0, 1.0)).astype(np.int64)
    y = 2.0 * v[0, 0, :valid].astype(np.float64).mean(axis=0)
    want = np.broadcast_to(np.clip(np.rint(y), -127, 127), got.shape)
    assert np.abs(got - want).max() <= 1 and (got == want).mean() > 0.99
    j0 = (valid // 2) | 1
    kn = k.copy()
    kn[0, 0, j0] = 127
    q = np.full((1, 1, S, d), 127, np.int8)
    got = _gpu(pkg, dev, dict(q=q, k=kn, v=v, mask=mask), (30.0, 30.0, 1.0, 1.0)).astype(np.int64)
    assert np.array_equal(got[0, 0], np.broadcast_to(v[0, 0, j0].astype(np.int64), (S, d)))


import glob  # noqa: E402
import os  # noqa: E402

FIXTURES = sorted(glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "*.npz")))


@pytest.mark.gpu
@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p) for p in FIXTURES])
def test_full_range_p_golden_fixture(pkg, dev, path):
    f = np.load(path)  # allow_pickle stays False
    c = dict(q=f["q"], k=f["k"], v=f["v"], mask=f["mask"])
    _gate(_gpu(pkg, dev, c, tuple(float(x) for x in f["amax"])), f["o_full_range_p"], os.path.basename(path))


@pytest.mark.gpu
def test_full_range_p_through_the_cpp_harness(tmp_path):
    """Host C++ calling FMHAInferI8CrossFullRangeP the way the reference's driver calls its launch function: the
    reference's own sweep (B = H = 1, its eleven lengths, both head sizes) and the smallest benchmark configuration,
    each checked inside the harness against the checker's 255-step mode."""
    import json
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "bin", "test_fmha_i8")
    assert os.path.exists(exe), "tests/bin/test_fmha_i8 is not built (python -c 'import __graft_entry__ as g; g.build()')"
    js = str(tmp_path / "harness.json")
    r = subprocess.run([exe, "--config", "1", "--sweep", "--full-range-p", "--iters", "20", "--warmup", "20", "--cpu-heads", "0",
                        "--json", js], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    print(r.stdout[-3000:])
    assert r.returncode == 0
    recs = [json.loads(l) for l in open(js)]
    assert len(recs) == 23 and all(x["pass"] for x in recs)
