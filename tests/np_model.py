"""An independent, vectorised numpy restatement of the reference kernel's int8 pipeline (inc/fmha_i8.cuh:71-72,
181-253,298-332), written separately from oracle/fmha_oracle.hpp so that an indexing or ordering mistake in either
shows up as a disagreement.  It works on whole [S, block] tiles with matrix products, float32 throughout, and defers
nothing: O is kept normalised per block like the reference."""
import numpy as np

f32 = np.float32


def fmha_i8_head(q, k, v, mask, q_amax, k_amax, v_amax, o_amax, block=128, full_range_p=False):
    """full_range_p: P = rne(255 p) in [0, 255] (the variant README.md:15,186 plans) instead of rne(-128 p)."""
    S, d = q.shape
    row_scale = f32(1.0) / f32(np.sqrt(f32(d)))
    scale_qk = f32(q_amax) * f32(k_amax) / (f32(127.0) * f32(127.0))
    scale_v = f32(v_amax) * (f32(1.0) / (f32(o_amax) * f32(255.0 if full_range_p else 128.0)))
    qi = q.astype(np.int32)
    m_run = np.full(S, -1e6, f32)
    l_run = np.zeros(S, f32)
    o_f = np.zeros((S, d), f32)
    for k0 in range(0, S, block):
        mk = mask[k0:k0 + block] != 0
        if mk.all():
            continue
        s_int = qi @ k[k0:k0 + block].astype(np.int32).T  # [S, block] exact
        s_for_max = np.where(mk[None, :], np.int32(-1000000), s_int)
        m_blk = np.maximum(f32(-1e6), (row_scale * s_for_max.max(axis=1).astype(f32)) * scale_qk).astype(f32)
        x = ((row_scale * s_int.astype(f32)).astype(f32) * scale_qk).astype(f32) - m_blk[:, None]
        p = np.where(mk[None, :], f32(0), np.exp(x.astype(f32))).astype(f32)
        l_blk = p.sum(axis=1, dtype=f32)
        if full_range_p:
            p_i8 = -np.rint(np.clip(f32(255.0) * p, 0, 255)).astype(np.int32)  # (negated: the merge below subtracts)
        else:
            p_i8 = np.rint(np.clip(f32(-128.0) * p, -128, 0)).astype(np.int32)  # np.rint rounds half to even
        o_tilde = p_i8 @ v[k0:k0 + block].astype(np.int32)  # [S, d] exact
        m_new = np.maximum(m_run, m_blk)
        a = np.exp((m_run - m_new).astype(f32)).astype(f32)
        b = np.exp((m_blk - m_new).astype(f32)).astype(f32)
        l_new = (a * l_run + b * l_blk).astype(f32)
        o_f = ((f32(1.0) / l_new)[:, None] * ((l_run * a)[:, None] * o_f - b[:, None] * o_tilde.astype(f32))).astype(f32)
        l_run, m_run = l_new, m_new
    out = np.rint(np.clip(scale_v * o_f, -127, 127)).astype(np.int8)
    out[l_run <= 0] = 0
    return out


def fmha_i8(q, k, v, mask, q_amax, k_amax, v_amax, o_amax, block=128, full_range_p=False):
    B, H, S, d = q.shape
    o = np.zeros_like(q)
    for b in range(B):
        for h in range(H):
            o[b, h] = fmha_i8_head(q[b, h], k[b, h], v[b, h], mask[b], q_amax, k_amax, v_amax, o_amax, block,
                                   full_range_p)
    return o


def attention_fp64(qf, kf, vf, mask):
    """Plain softmax(Q K^T / sqrt(d)) V in float64 with masked keys removed: the textbook routine."""
    B, H, S, d = qf.shape
    o = np.zeros(qf.shape, np.float64)
    for b in range(B):
        keep = mask[b] == 0
        if not keep.any():
            continue
        for h in range(H):
            s = qf[b, h].astype(np.float64) @ kf[b, h].astype(np.float64)[keep].T / np.sqrt(d)
            s -= s.max(axis=1, keepdims=True)
            p = np.exp(s)
            p /= p.sum(axis=1, keepdims=True)
            o[b, h] = p @ vf[b, h].astype(np.float64)[keep]
    return o
