"""Queries and keys that differ in number (the reference lists "S_src != S_dst" as planned, README.md:13; its kernel
sizes Q, K, V and the mask by one SEQ_LEN, inc/fmha_i8.cuh:45,88-89).  Nothing in the reference computes this case,
so parity is anchored on what the reference's arithmetic fixes: a query row never sees another query row
(inc/fmha_i8.cuh:120-332 keeps m, l and O per row), hence attention of any set of query rows over a key set equals the
same rows of a self-attention problem over that key set.  The CPU tests pin the checker's cross-length entry to its
self-attention entry (itself pinned by closed forms and the reference's headers); the GPU tests hold the HIP kernel to
the checker with the usual gate, and to its own self-attention output bit for bit."""
import numpy as np
import pytest

import fmha_cases as fc

WITHIN1_MIN = 0.999
MAX_ABS_LSB = 2


def _scales(c):
    return c["q_amax"], c["k_amax"], c["v_amax"], c["o_amax"]


def _self(orc, c):
    S = c["k"].shape[2]
    return orc.fmha_i8_blockwise(c["q"], c["k"], c["v"], c["mask"], *_scales(c), block=128 if S % 128 == 0 else 64)


# ---- the checker -------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("S,d,pad", [(256, 64, "none"), (192, 128, "scatter"), (384, 64, "scatter")])
def test_checker_cross_equals_self_on_equal_lengths(orc, S, d, pad):
    c = fc.make_inputs(2, 2, S, d, pad=pad, seed=31)
    assert np.array_equal(orc.fmha_i8_blockwise_cross(c["q"], c["k"], c["v"], c["mask"], *_scales(c)), _self(orc, c))


@pytest.mark.parametrize("rows", [1, 37, 64, 200])
def test_checker_fewer_queries_are_a_prefix_of_self_attention(orc, rows):
    c = fc.make_inputs(2, 3, 256, 64, pad="scatter", seed=32)
    full = _self(orc, c)
    got = orc.fmha_i8_blockwise_cross(c["q"][:, :, :rows], c["k"], c["v"], c["mask"], *_scales(c))
    assert got.shape == (2, 3, rows, 64) and np.array_equal(got, full[:, :, :rows])


def test_checker_more_queries_than_keys(orc):
    # 3 x 128 query rows over 128 keys: each third is a self-attention problem with the same K, V and mask
    ck = fc.make_inputs(1, 2, 128, 128, pad="scatter", seed=33)
    qs = [fc.make_inputs(1, 2, 128, 128, seed=40 + i)["q"] for i in range(3)]
    got = orc.fmha_i8_blockwise_cross(np.concatenate(qs, axis=2), ck["k"], ck["v"], ck["mask"], *_scales(ck))
    for i, q in enumerate(qs):
        assert np.array_equal(got[:, :, 128 * i:128 * (i + 1)], _self(orc, dict(ck, q=q)))


def test_checker_uniform_attention_closed_form(orc):
    # Q == 0: every unmasked key weighs the same, O = rne(v_amax/o_amax * mean of the unmasked V rows), for any Sq
    ck = fc.make_inputs(1, 2, 192, 64, seed=34, valid_lengths=[150])
    q = np.zeros((1, 2, 77, 64), np.int8)
    got = orc.fmha_i8_blockwise_cross(q, ck["k"], ck["v"], ck["mask"], 1.0, 1.0, 3.0, 1.5).astype(np.int64)
    y = 2.0 * ck["v"][:, :, :150].astype(np.float64).mean(axis=2, keepdims=True)
    want = np.broadcast_to(np.clip(np.rint(y), -127, 127), got.shape)
    near_tie = np.broadcast_to(np.abs(np.abs(y - np.floor(y)) - 0.5) < 1e-3, got.shape)
    assert np.array_equal(got[~near_tie], want[~near_tie]) and np.abs(got - want).max() <= 1


def test_cross_argument_checks_without_a_gpu(pkg):
    p = pkg.FMHAParamI8(1.0, 1.0, 1.0, 1.0, 1.0)
    ok = 0x1000

    def chk(B, Sq, S, H, d, q=ok, k=ok, v=ok, m=ok, o=ok):
        return pkg.FMHAInferI8CrossCheckArgs(p, pkg.FMHACrossAttnDescriptor(B, Sq, S, H, d), q, k, v, m, o)

    assert chk(1, 1, 64, 1, 64) == pkg.FMHA_I8_OK
    assert chk(2, 65536, 65536, 3, 128) == pkg.FMHA_I8_OK
    assert chk(1, 300, 192, 1, 64) == pkg.FMHA_I8_OK
    assert chk(1, 0, 64, 1, 64) == pkg.FMHA_I8_ERR_SEQ_LEN
    assert chk(1, 65537, 64, 1, 64) == pkg.FMHA_I8_ERR_SEQ_LEN
    assert chk(1, 64, 96, 1, 64) == pkg.FMHA_I8_OK                # any key count
    assert chk(1, 64, 65537, 1, 64) == pkg.FMHA_I8_ERR_SEQ_LEN
    assert chk(1, 64, 0, 1, 64) == pkg.FMHA_I8_ERR_SEQ_LEN
    assert chk(1, 64, 64, 1, 96) == pkg.FMHA_I8_ERR_HEAD_DIM
    assert chk(0, 64, 64, 1, 64) == pkg.FMHA_I8_ERR_BATCH_HEAD
    assert chk(1, 64, 64, 1, 64, q=ok + 8) == pkg.FMHA_I8_ERR_ALIGNMENT
    assert chk(1, 64, 64, 1, 64, m=None) == pkg.FMHA_I8_ERR_NULL_POINTER


# ---- the HIP kernel ----------------------------------------------------------------------------------------------
def _gpu(pkg, dev, q, c, canary=False):
    import torch
    t = [torch.from_numpy(np.ascontiguousarray(a)).to(dev) for a in (q, c["k"], c["v"], c["mask"])]
    out = None
    if canary:
        # rows past the last query must stay untouched: the output buffer is followed by marked bytes
        buf = torch.full((q.size + 4096,), 77, dtype=torch.int8, device=dev)
        out = buf[:q.size].view(q.shape)
    o = pkg.fmha_infer_i8(*t, *_scales(c), out=out)
    torch.cuda.synchronize()
    if canary:
        assert (buf[q.size:] == 77).all().item()
    return o.cpu().numpy()


def _gate(got, want, what):
    st = fc.parity_stats(got, want)
    print(what, st, flush=True)
    assert st["within1"] >= WITHIN1_MIN and st["max"] <= MAX_ABS_LSB, (what, st)


@pytest.mark.gpu
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("Sq,S,pad", [(1, 64, "none"), (31, 128, "scatter"), (33, 192, "scatter"), (100, 512, "none"),
                                      (256, 128, "scatter"), (257, 320, "tail"), (777, 1024, "scatter"),
                                      (1024, 64, "none"), (1300, 256, "scatter")])
def test_cross_attention_against_the_checker(pkg, orc, dev, Sq, S, d, pad):
    B, H = 2, 3
    ck = fc.make_inputs(B, H, S, d, pad="scatter" if pad == "scatter" else "none", seed=50,
                        valid_lengths=[S - 40, S - 64] if pad == "tail" else None)
    q = fc.make_inputs(B, H, Sq, d, seed=51)["q"]  # quantised normal data, like the keys
    want = orc.fmha_i8_blockwise_cross(q, ck["k"], ck["v"], ck["mask"], *_scales(ck))
    _gate(_gpu(pkg, dev, q, ck, canary=True), want, "cross Sq=%d S=%d d=%d %s" % (Sq, S, d, pad))


@pytest.mark.gpu
@pytest.mark.parametrize("S,d", [(512, 128), (320, 64)])
def test_cross_attention_is_rows_of_self_attention_bit_for_bit(pkg, dev, S, d):
    """The same kernel computes every query row from the same K, V tiles in the same order whatever the number of
    rows, so fewer (or regrouped) query rows must reproduce the self-attention bytes exactly."""
    c = fc.make_inputs(2, 2, S, d, pad="scatter", seed=52)
    full = _gpu(pkg, dev, c["q"], c)
    for rows in (1, 32, 45, 256, 300):
        assert np.array_equal(_gpu(pkg, dev, c["q"][:, :, :rows], c, canary=True), full[:, :, :rows]), rows
    # more queries than keys: the self-attention queries twice over, the second copy reversed
    q2 = np.concatenate([c["q"], c["q"][:, :, ::-1]], axis=2)
    got = _gpu(pkg, dev, q2, c)
    assert np.array_equal(got[:, :, :S], full) and np.array_equal(got[:, :, S:], full[:, :, ::-1])


@pytest.mark.gpu
def test_cross_attention_decode_shape_at_full_size(pkg, dev):
    """One query row per head over 65536 keys (the longest key sequence): uniform attention has a closed form."""
    import torch
    B, H, S, d = 1, 4, 65536, 64
    rng = np.random.default_rng(53)
    v = rng.integers(-127, 128, (B, H, S, d)).astype(np.int8)
    k = rng.integers(-127, 128, (B, H, S, d)).astype(np.int8)
    mask = np.zeros((B, S), np.int8)
    mask[0, 50000:] = 1
    q = np.zeros((B, H, 1, d), np.int8)
    c = dict(k=k, v=v, mask=mask, q_amax=1.0, k_amax=1.0, v_amax=40.0, o_amax=1.0)
    got = _gpu(pkg, dev, q, c, canary=True).astype(np.int64)
    y = 40.0 * v[:, :, :50000].astype(np.float64).mean(axis=2, keepdims=True)
    assert np.abs(got - np.clip(np.rint(y), -127, 127)).max() <= 1
    torch.cuda.synchronize()


# ---- key counts that are not multiples of 64 -----------------------------------------------------------------------
def test_checker_ragged_key_count_means_padding_with_masked_keys(orc):
    c = fc.make_inputs(1, 2, 192, 64, pad="scatter", seed=60)
    q = c["q"][:, :, :50]
    for S in (129, 150, 191):
        got = orc.fmha_i8_blockwise_cross(q, c["k"][:, :, :S], c["v"][:, :, :S], c["mask"][:, :S], *_scales(c))
        m = c["mask"].copy()
        m[:, S:] = 1  # same keys, the rest masked: what lies in K and V behind a masked key cannot matter
        assert np.array_equal(got, orc.fmha_i8_blockwise_cross(q, c["k"], c["v"], m, *_scales(c))), S


@pytest.mark.gpu
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("S", [1, 3, 4, 5, 63, 65, 100, 127, 129, 191, 193, 255, 257, 1000, 1023, 1025, 2049])
def test_any_key_count(pkg, orc, dev, S, d):
    """Self-attention and cross-attention with a key count that is no multiple of 64: the HIP kernel against the
    checker (gate), and against itself on inputs that the caller padded to the next multiple of 64 with masked keys
    and other bytes in the padding (so a read of padding that reaches the output shows)."""
    B, H = 2, 2
    Sp = (S + 63) // 64 * 64
    c = fc.make_inputs(B, H, Sp, d, pad="scatter" if S > 8 else "none", seed=61)
    if S > 8:
        c["mask"][:, 0] = 0  # at least one key that every batch entry attends to
    cut = dict(c, k=c["k"][:, :, :S], v=c["v"][:, :, :S], mask=c["mask"][:, :S])
    cut = {n: (np.ascontiguousarray(a) if isinstance(a, np.ndarray) else a) for n, a in cut.items()}
    padded = dict(c, mask=c["mask"].copy())
    padded["mask"][:, S:] = 1
    for Sq in sorted({S, 77}):
        q = fc.make_inputs(B, H, Sq, d, seed=62)["q"]
        got = _gpu(pkg, dev, q, cut, canary=True)
        _gate(got, orc.fmha_i8_blockwise_cross(q, cut["k"], cut["v"], cut["mask"], *_scales(c)),
              "S=%d Sq=%d d=%d" % (S, Sq, d))
        # (not bit for bit: the last block's keys sit in other lanes than in the padded run, so the float row sum
        # adds them in another order)
        st = fc.parity_stats(got, _gpu(pkg, dev, q, padded))
        assert st["max"] <= 1 and st["exact"] >= 0.999, (S, Sq, st)


@pytest.mark.gpu
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("S", [15, 16, 17, 31, 33, 4100, 4111])
def test_mask_bytes_of_the_lane_that_straddles_the_end_of_the_row(pkg, orc, dev, S, d):
    """The kernel classifies the mask sixteen bytes per lane; the lane whose sixteen keys straddle the end of the row
    takes its bytes from the row's last sixteen (one load that ends where the row ends), rows shorter than sixteen
    bytes are read byte by byte, and rows of more than 4096 keys are classified in several passes.  A scattered mask,
    so that every one of those bytes shows in the output."""
    B, H, Sq = 2, 2, 77
    Sp = (S + 63) // 64 * 64
    c = fc.make_inputs(B, H, Sp, d, pad="scatter", seed=66)
    c["mask"][:, 0] = 0
    c["mask"][0, S - 1] = 0  # the last key of the row: attended to in one batch entry, masked out in the other
    c["mask"][1, S - 1] = 1
    cut = dict(c, k=c["k"][:, :, :S], v=c["v"][:, :, :S], mask=c["mask"][:, :S])
    cut = {n: (np.ascontiguousarray(a) if isinstance(a, np.ndarray) else a) for n, a in cut.items()}
    q = fc.make_inputs(B, H, Sq, d, seed=67)["q"]
    _gate(_gpu(pkg, dev, q, cut, canary=True), orc.fmha_i8_blockwise_cross(q, cut["k"], cut["v"], cut["mask"], *_scales(c)),
          "S=%d d=%d" % (S, d))


@pytest.mark.gpu
def test_any_key_count_at_the_end_of_an_allocation(pkg, orc, dev):
    """K, V and the mask end exactly where their device allocations end: a tile load or a mask read that ran past the
    last key would leave the buffers (the last head of the last batch entry is the one that matters)."""
    import torch
    B, H, S, d = 1, 2, 70, 128
    c = fc.make_inputs(B, H, 128, d, seed=63)
    k, v, m = (np.ascontiguousarray(a) for a in (c["k"][:, :, :S], c["v"][:, :, :S], c["mask"][:, :S]))
    q = c["q"][:, :, :40]
    want = orc.fmha_i8_blockwise_cross(q, k, v, m, *_scales(c))
    bufs = []
    for a in (k, v, m):
        n = a.size
        buf = torch.empty(((n + 4095) // 4096) * 4096, dtype=torch.int8, device=dev)
        view = buf[buf.numel() - n:].view(a.shape) if n % 16 == 0 else None
        if view is None:  # the mask has no alignment requirement: put it at the very end, whatever its size
            view = buf[buf.numel() - n:].view(a.shape)
        view.copy_(torch.from_numpy(a))
        bufs.append((buf, view))
    qd = torch.from_numpy(np.ascontiguousarray(q)).to(dev)
    o = pkg.fmha_infer_i8(qd, bufs[0][1], bufs[1][1], bufs[2][1], *_scales(c))
    torch.cuda.synchronize()
    _gate(o.cpu().numpy(), want, "end of allocation")


@pytest.mark.gpu
@pytest.mark.parametrize("S,d", [(3, 64), (19, 128), (58, 64), (100, 128)])
def test_sequences_shorter_than_one_block_with_many_query_blocks(pkg, orc, dev, S, d):
    """A key sequence shorter than one block has a single tile, which every later issue point of the key loop fetches
    again: each of those fetches has to stop at the last key like the first one does (tiny K and V tensors, several
    heads and query blocks, so that a full-tile fetch would run far past their end)."""
    B, H, Sq = 3, 3, 319
    c = fc.make_inputs(B, H, 128, d, seed=64)
    k, v = (np.ascontiguousarray(c[n][:, :, :S]) for n in ("k", "v"))
    mask = np.zeros((B, S), np.int8)
    mask[1, S // 2 + 1:] = 1
    q = fc.make_inputs(B, H, Sq, d, seed=65)["q"]
    cc = dict(c, k=k, v=v, mask=mask)
    _gate(_gpu(pkg, dev, q, cc, canary=True), orc.fmha_i8_blockwise_cross(q, k, v, mask, *_scales(c)),
          "short S=%d d=%d" % (S, d))


@pytest.mark.gpu
def test_random_shapes(pkg, orc, dev):
    """Sixty seeded random problems - any query count, any key count, every kind of mask (none, scattered, ragged
    tails, a run of fully masked blocks in the middle), both head sizes, both distributions, three score scales -
    against the checker with the usual gate."""
    import torch
    rng = np.random.default_rng(2024)
    for it in range(60):
        d = int(rng.choice([64, 128]))
        B, H = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        S = int(rng.choice([rng.integers(1, 130), rng.integers(1, 700), rng.integers(500, 2600), 64 * rng.integers(1, 40)]))
        Sq = S if rng.random() < 0.4 else int(rng.choice([rng.integers(1, 70), rng.integers(1, 600), rng.integers(200, 1500)]))
        pad = str(rng.choice(["none", "scatter", "tail", "dead"]))
        c = fc.make_inputs(B, H, (S + 63) // 64 * 64, d, pad="scatter" if pad == "scatter" else "none", seed=1000 + it,
                           dist=str(rng.choice(["normal", "student_t"])), sigma=float(rng.choice([0.5, 1.0])))
        mask = c["mask"][:, :S].copy()
        if pad == "tail":
            for b in range(B):
                mask[b, int(rng.integers(1, S + 1)):] = 1
        if pad == "dead" and S > 256:
            a = int(rng.integers(0, S - 130))
            mask[:, a:a + int(rng.integers(64, 400))] = 1
        mask[:, 0] = 0
        k, v = (np.ascontiguousarray(c[n][:, :, :S]) for n in ("k", "v"))
        q = fc.make_inputs(B, H, Sq, d, seed=5000 + it)["q"]
        scales = (c["q_amax"] * float(rng.choice([1, 1, 8, 40])), c["k_amax"], c["v_amax"], float(rng.choice([1.0, 2.0])))
        print("case", it, B, H, Sq, S, d, pad, flush=True)
        want = orc.fmha_i8_blockwise_cross(q, k, v, mask, *scales)
        t = [torch.from_numpy(np.ascontiguousarray(a)).to(dev) for a in (q, k, v, mask)]
        got = pkg.fmha_infer_i8(*t, *scales)
        torch.cuda.synchronize()
        _gate(got.cpu().numpy(), want, "random case %d" % it)
