"""Quantisation-error study of INT8 attention: how much error each way of scaling the softmax matrix P costs.

Restates, seeded and with CSV output instead of interactive plots, the two simulations that the reference keeps beside
its kernel (fmha_i8_quant_error_seqlen.py:23-118: sum of |error| against the sequence length; fmha_i8_quant_deviation.py:
9-120: relative L2 deviation per token at one length), and adds the scheme the kernel really uses, which neither script
simulates:

  worst        P quantised against p_amax = 1                      (fmha_i8_quant_error_seqlen.py:62-76)
  static       P quantised against one p_amax for the whole matrix (…:82-96; the maximum of the float softmax)
  dynamic      P quantised against the maximum of its own row      (…:103-118)
  block_local  flash-style: per block of 128 keys (64 when the length is not a multiple of 128), p = exp(x - block
               maximum) quantised with scale 128, row sum kept un-quantised, blocks merged online
               (inc/fmha_i8.cuh:181-253,298-315)
  block_local_full
               the same with 255 steps: the "uint8 x int8" variant the reference plans (README.md:15,186), which on
               int8 matrix hardware is P - 128 as int8 plus 128 times the column sums of V per block
  kernel       (optional, --kernel) the HIP kernel itself through libfmha_i8.so, int8 output de-quantised with
               o_amax = max |float O|; adds the output quantisation on top of block_local; multiples of 64 only
  kernel_full  (with --kernel) the kernel's 255-step entry point, FMHAInferI8CrossFullRangeP: block_local_full plus
               the output quantisation

Everything else follows the scripts: Q, K, V standard normal, [S, d] (one head), symmetric int8 quantisation of Q, K, V
by abs-max with numpy's round-half-even, int32 Q.K^T, float softmax, P quantised to --levels steps, int32 P.V,
de-quantisation with v_amax / 127.  The scripts as they stand use 127 steps (SOFTMAX_QUANT_SCALE = 127, the default
here); the figures the reference publishes from them (fig/error_sum.png, fig/deviation_512.png: worst case 1430 at
1024 tokens, dynamic 55; worst-case deviation about 0.35 at 512 tokens, dynamic 0.02) are reproduced with 255 steps,
the full uint8 range that quantize_to_uint8 defaults to (fmha_i8_quant_error_seqlen.py:14).

    python quant_error_study.py seqlen    [--max-len 1024] [--step 16] [--head-dim 64] [--levels 127] [--seed 2023]
    python quant_error_study.py deviation [--seq-len 512] [--head-dim 64] [--levels 127] [--seed 2023]
    common: [--kernel] [--out FILE.csv]
"""
import argparse
import csv
import importlib.util
import os
import sys

import numpy as np

SOFTMAX_QUANT_SCALE = 127  # fmha_i8_quant_error_seqlen.py:4
SCHEMES = ("worst", "static", "dynamic", "block_local", "block_local_full")
f32 = np.float32


def quantize_to_int8(x, clip_max, quant_range=127):
    """fmha_i8_quant_error_seqlen.py:5-11: round(x * range / amax) clipped to +-range (numpy rounds half to even)."""
    scale = quant_range / clip_max
    return np.clip(np.round(x.astype(f32) * scale), -quant_range, quant_range).astype(np.int8)


def quantize_to_uint8(x, clip_max, quant_range=255):
    """fmha_i8_quant_error_seqlen.py:14-19; clip_max may be one number or one per row (shape [S, 1])."""
    scale = quant_range / clip_max
    return np.clip(np.round(x.astype(f32) * scale), 0, quant_range).astype(np.uint8)


def softmax_rows(s):
    """fmha_i8_quant_error_seqlen.py:38-42, all rows at once."""
    e = np.exp(s - s.max(axis=1, keepdims=True))
    return e / e.sum(axis=1, keepdims=True)


def block_keys_for(seq_len):
    return 128 if seq_len % 128 == 0 else 64  # src/fmha_i8.cu:39-154


def block_local_attention(s_f, v_i8, v_amax, block, steps=128):
    """The kernel's scheme on de-quantised scores s_f [S, S_kv] (float32) and int8 V: returns float O [S, d].
    steps: quantisation steps of P (128 in the kernel: p = 1 maps to -128)."""
    S = s_f.shape[0]
    m_run = np.full(S, -np.inf, f32)
    l_run = np.zeros(S, f32)
    o_run = np.zeros((S, v_i8.shape[1]), f32)  # un-normalised, in units of 1/128
    for k0 in range(0, s_f.shape[1], block):
        x = s_f[:, k0:k0 + block]
        m_blk = x.max(axis=1)
        p = np.exp(x - m_blk[:, None]).astype(f32)
        l_blk = p.sum(axis=1, dtype=f32)                                   # un-quantised (inc/fmha_i8.cuh:208-235)
        p_q = np.rint(np.clip(f32(steps) * p, 0, steps)).astype(np.int32)  # |P| of inc/fmha_i8.cuh:241,249
        o_blk = (p_q @ v_i8[k0:k0 + block].astype(np.int32)).astype(f32)   # exact int32
        m_new = np.maximum(m_run, m_blk)
        a, b = np.exp(m_run - m_new).astype(f32), np.exp(m_blk - m_new).astype(f32)
        l_run = a * l_run + b * l_blk
        o_run = a[:, None] * o_run + b[:, None] * o_blk
        m_run = m_new
    return (o_run / (f32(steps) * l_run)[:, None]) * f32(v_amax / 127.0)


def simulate(seq_len, head_dim, rng, kernel=None, levels=SOFTMAX_QUANT_SCALE):
    """One head of seq_len tokens.  Returns a dict with the float reference 'ref' [S, d], one float O per scheme, and
    the quantised tensors and scales ('q', 'k', 'v' int8; 'q_amax', 'k_amax', 'v_amax', 'o_amax')."""
    f_q, f_k, f_v = (rng.standard_normal((seq_len, head_dim)) for _ in range(3))
    f_p = softmax_rows((f_q @ f_k.T).astype(f32) / np.sqrt(head_dim))
    out = {"ref": (f_p @ f_v).astype(f32)}                                  # ground truth (…seqlen.py:33-45)
    q_amax, k_amax, v_amax = (float(np.abs(t).max()) for t in (f_q, f_k, f_v))
    i8_q, i8_k, i8_v = quantize_to_int8(f_q, q_amax), quantize_to_int8(f_k, k_amax), quantize_to_int8(f_v, v_amax)
    s_f = ((i8_q.astype(np.int32) @ i8_k.astype(np.int32).T) * q_amax / 127 * k_amax / 127) / np.sqrt(head_dim)
    p = softmax_rows(s_f).astype(f32)
    v32 = i8_v.astype(np.int32)

    def through_uint8(p_amax):  # …seqlen.py:71-74: quantise P, integer P.V, de-quantise
        u8 = quantize_to_uint8(p, p_amax, levels)
        return (u8.astype(np.int32) @ v32) * (np.asarray(p_amax, np.float64) / levels) * v_amax / 127

    out["worst"] = through_uint8(1.0)
    out["static"] = through_uint8(float(np.abs(f_p).max()))
    out["dynamic"] = through_uint8(p.max(axis=1, keepdims=True))
    out["block_local"] = block_local_attention(s_f.astype(f32), i8_v, v_amax, block_keys_for(seq_len))
    out["block_local_full"] = block_local_attention(s_f.astype(f32), i8_v, v_amax, block_keys_for(seq_len), steps=255)
    o_amax = float(np.abs(out["ref"]).max())
    out.update(q=i8_q, k=i8_k, v=i8_v, q_amax=q_amax, k_amax=k_amax, v_amax=v_amax, o_amax=o_amax)
    if kernel is not None and seq_len % 64 == 0:
        out["kernel"] = kernel(i8_q, i8_k, i8_v, q_amax, k_amax, v_amax, o_amax)
        out["kernel_full"] = kernel(i8_q, i8_k, i8_v, q_amax, k_amax, v_amax, o_amax, full_range_p=True)
    return out


def error_sum(o, ref):
    return float(np.abs(o - ref).sum())                                     # …seqlen.py:76,96,118


def row_deviation(o, ref):
    return np.linalg.norm(o - ref, ord=2, axis=1) / np.linalg.norm(ref, ord=2, axis=1)  # …deviation.py:75,97,120


def hip_kernel_runner():
    """Returns f(q, k, v int8 [S, d], scales) -> float O [S, d] computed by the HIP kernel (raises without a GPU or the
    built library: there is no substitute path)."""
    import torch
    here = os.path.dirname(os.path.abspath(__file__))
    name = "fmha_i8_amd_for_study"
    if name not in sys.modules:
        spec = importlib.util.spec_from_file_location(name, os.path.join(here, "__init__.py"),
                                                      submodule_search_locations=[here])
        mod = importlib.util.module_from_spec(spec)
        sys.modules[name] = mod
        spec.loader.exec_module(mod)
    pkg = sys.modules[name]
    pkg.load_library()
    if not torch.cuda.is_available():
        raise RuntimeError("--kernel needs a GPU")
    dev = torch.device("cuda:0")

    def run(q, k, v, q_amax, k_amax, v_amax, o_amax, full_range_p=False):
        t = [torch.from_numpy(np.ascontiguousarray(a[None, None])).to(dev) for a in (q, k, v)]
        mask = torch.zeros((1, k.shape[0]), dtype=torch.int8, device=dev)
        o = pkg.fmha_infer_i8(t[0], t[1], t[2], mask, q_amax, k_amax, v_amax, o_amax, full_range_p=full_range_p)
        torch.cuda.synchronize()
        return o[0, 0].cpu().numpy().astype(f32) / f32(127.0) * f32(o_amax)  # inc/utils.hpp:53

    return run


def table_seqlen(lengths, head_dim, seed, kernel=None, levels=SOFTMAX_QUANT_SCALE):
    """Rows (seq_len, sum |error| per scheme): what fmha_i8_quant_error_seqlen.py:119-130 plots."""
    cols = SCHEMES + (("kernel", "kernel_full") if kernel is not None else ())
    rows = []
    for S in lengths:
        r = simulate(S, head_dim, np.random.default_rng([seed, S, head_dim]), kernel, levels)
        rows.append([S] + [error_sum(r[c], r["ref"]) if c in r else "" for c in cols])
    return ("seq_len",) + cols, rows


def table_deviation(seq_len, head_dim, seed, kernel=None, levels=SOFTMAX_QUANT_SCALE):
    """Rows (token, relative L2 deviation per scheme): what fmha_i8_quant_deviation.py:75-126 plots."""
    cols = SCHEMES + (("kernel", "kernel_full") if kernel is not None else ())
    r = simulate(seq_len, head_dim, np.random.default_rng([seed, seq_len, head_dim]), kernel, levels)
    dev = [row_deviation(r[c], r["ref"]) for c in cols if c in r]
    return ("token",) + tuple(c for c in cols if c in r), [[i] + [float(d[i]) for d in dev] for i in range(seq_len)]


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("mode", choices=("seqlen", "deviation"))
    ap.add_argument("--max-len", type=int, default=1024)   # SEQLEN_LIST = 16 .. 1024 (…seqlen.py:21)
    ap.add_argument("--step", type=int, default=16)
    ap.add_argument("--seq-len", type=int, default=512)    # …deviation.py:9
    ap.add_argument("--head-dim", type=int, default=64)    # both scripts
    ap.add_argument("--levels", type=int, default=SOFTMAX_QUANT_SCALE, help="quantisation steps of P in the three "
                    "non-flash schemes: 127 as the scripts stand, 255 reproduces the published figures")
    ap.add_argument("--seed", type=int, default=2023)
    ap.add_argument("--kernel", action="store_true", help="add a column computed by the HIP kernel (needs the GPU)")
    ap.add_argument("--out", default="-")
    a = ap.parse_args(argv)
    kernel = hip_kernel_runner() if a.kernel else None
    if a.mode == "seqlen":
        header, rows = table_seqlen(range(a.step, a.max_len + 1, a.step), a.head_dim, a.seed, kernel, a.levels)
    else:
        header, rows = table_deviation(a.seq_len, a.head_dim, a.seed, kernel, a.levels)
    f = sys.stdout if a.out == "-" else open(a.out, "w", newline="")
    w = csv.writer(f)
    w.writerow(header)
    w.writerows(rows)
    if f is not sys.stdout:
        f.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
