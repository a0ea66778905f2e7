"""Seeded synthetic workloads: the five benchmark configurations and the reference test's own data style.

Mask bytes use the API polarity of the reference kernel: nonzero = key masked OUT (inc/fmha_i8.cuh:189-192), so a
workload described by valid lengths L_b becomes mask[b][j] = (j >= L_b) and "no padding" is all zeros.
"""
import numpy as np

MASTER_SEED = 2023  # test_fmha_i8.cpp:49

# name -> (B, H, S, d, distribution, padding)
CONFIGS = {
    "C1": dict(B=1, H=2, S=128, d=64, dist="normal", sigma=1.0, pad="none"),
    "C2": dict(B=8, H=12, S=512, d=64, dist="normal", sigma=1.0, pad="bert"),
    "C3": dict(B=4, H=16, S=1024, d=128, dist="normal", sigma=1.0, pad="none"),
    "C4": dict(B=1, H=32, S=4096, d=128, dist="normal", sigma=0.5, pad="tail256"),
    "C5": dict(B=16, H=16, S=2048, d=64, dist="student_t", sigma=0.5, pad="none"),
}


def quantize_i8_np(x, amax):
    """inc/utils.hpp:23-29 in numpy: floorf(x * (127/amax) + 0.5): the add in double, rounded to float for floorf."""
    scale = np.float32(127.0) / np.float32(amax)
    scaled = (x.astype(np.float32) * scale).astype(np.float32)
    q = np.floor((scaled.astype(np.float64) + 0.5).astype(np.float32))
    return np.clip(q, -127, 127).astype(np.int8)


def make_inputs(B, H, S, d, dist="normal", sigma=1.0, pad="none", seed=MASTER_SEED, valid_lengths=None):
    """Returns dict(q,k,v int8 [B,H,S,d]; mask int8 [B,S]; q_amax,k_amax,v_amax,o_amax floats; qf,kf,vf floats)."""
    rng = np.random.default_rng([seed, B, H, S, d])
    shape = (B, H, S, d)
    if dist == "normal":
        qf, kf, vf = (np.float32(sigma) * rng.standard_normal(shape, dtype=np.float32) for _ in range(3))
    elif dist == "student_t":
        qf = (sigma * rng.standard_t(3, shape)).astype(np.float32)
        kf = (sigma * rng.standard_t(3, shape)).astype(np.float32)
        vf = rng.standard_normal(shape, dtype=np.float32)
    elif dist == "reference":  # test_fmha_i8.cpp:74-89: Q,K ~ U(-.5,.5), V = |U(-.5,.5)|
        qf = rng.uniform(-0.5, 0.5, shape).astype(np.float32)
        kf = rng.uniform(-0.5, 0.5, shape).astype(np.float32)
        vf = np.abs(rng.uniform(-0.5, 0.5, shape)).astype(np.float32)
    else:
        raise ValueError(dist)
    mask = np.zeros((B, S), np.int8)
    if valid_lengths is not None:
        for b in range(B):
            mask[b, valid_lengths[b]:] = 1
    elif pad == "bert":  # L_b uniform in [256, 512] rounded to a multiple of 64 (scaled to S for other lengths)
        for b in range(B):
            L = 64 * int(rng.integers(S // 128, S // 64 + 1))
            mask[b, L:] = 1
    elif pad == "tail256":
        mask[:, S - S // 16:] = 1
    elif pad == "scatter":  # test_fmha_i8.cpp:75-79: Bernoulli(0.2) scattered
        mask = (rng.random((B, S)) < 0.2).astype(np.int8)
    elif pad != "none":
        raise ValueError(pad)
    qa, ka, va = (float(np.max(np.abs(t))) for t in (qf, kf, vf))
    return dict(q=quantize_i8_np(qf, qa), k=quantize_i8_np(kf, ka), v=quantize_i8_np(vf, va), mask=mask, q_amax=qa,
                k_amax=ka, v_amax=va, o_amax=1.0, qf=qf, kf=kf, vf=vf)


def make_config(name, **override):
    cfg = dict(CONFIGS[name])
    cfg.update(override)
    return make_inputs(**cfg)


def parity_stats(got, want):
    """int8 O parity histogram: the gate is >= 99.9 % within +-1 LSB and max |delta| <= 2."""
    delta = np.abs(got.astype(np.int32) - want.astype(np.int32))
    return dict(exact=float((delta == 0).mean()), within1=float((delta <= 1).mean()), max=int(delta.max()),
                n=int(delta.size))


def assert_parity(got, want, what=""):
    st = parity_stats(got, want)
    assert st["within1"] >= 0.999 and st["max"] <= 2, "%s parity failed: %r" % (what, st)
    return st
