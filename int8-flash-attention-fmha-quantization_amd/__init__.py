"""Host-side mirror (Python) of the INT8 fused attention launch API on MI355X.

The product is the C-ABI library ``libfmha_i8.so`` built from ``csrc/`` (see ``include/fmha_i8.h``).  This module binds
it with ctypes and keeps the reference's names and argument order (inc/fmha_i8.h:7-15, inc/fmha_param_i8.h:3-17):

    FMHAInferI8(stream, fmha_param, attn_desc, q, k, v, padding_mask, o, use_tcu)

``q, k, v, padding_mask, o`` are device pointers (ints) or objects with ``data_ptr()`` (torch tensors on the GPU);
``stream`` is a ``hipStream_t`` value (int), a ``torch.cuda.Stream`` or None for the null stream.  There is no CPU
fallback: if the library is missing or cannot be loaded, every call raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfmha_i8.so")

EXPORTED_SYMBOLS = ("FMHAInferI8", "FMHAInferI8Status", "FMHAInferI8CheckArgs", "FMHAInferI8StatusString",
                    "FMHAInferI8Version", "FMHAInferI8Cross", "FMHAInferI8CrossCheckArgs",
                    "FMHAInferI8CrossFullRangeP", "FMHAAbsMaxF32", "FMHAQuantizeI8", "FMHADequantizeI8",
                    "FMHAAbsMaxBF16", "FMHAQuantizeI8BF16", "FMHADequantizeI8BF16")

FMHA_I8_OK = 0
FMHA_I8_ERR_NULL_POINTER = 1
FMHA_I8_ERR_HEAD_DIM = 2
FMHA_I8_ERR_SEQ_LEN = 3
FMHA_I8_ERR_BATCH_HEAD = 4
FMHA_I8_ERR_ALIGNMENT = 5
FMHA_I8_ERR_SCALE = 6
FMHA_I8_ERR_HIP_BASE = 1000


class AttnDataDescriptor(C.Structure):
    """inc/fmha_param_i8.h:3-8 — same field order and defaults."""
    _fields_ = [("batch_num", C.c_int), ("seq_len", C.c_int), ("head_num", C.c_int), ("head_dim", C.c_int)]

    def __init__(self, batch_num=1, seq_len=64, head_num=4, head_dim=64):
        super().__init__(batch_num, seq_len, head_num, head_dim)


class FMHACrossAttnDescriptor(C.Structure):
    """include/fmha_i8.h: queries and keys differ in number (README.md:13 lists "S_src != S_dst" as planned)."""
    _fields_ = [("batch_num", C.c_int), ("seq_len_q", C.c_int), ("seq_len_kv", C.c_int), ("head_num", C.c_int),
                ("head_dim", C.c_int)]


class FMHAParamI8(C.Structure):
    """inc/fmha_param_i8.h:10-17 — same field order and defaults; s_max is carried but unused."""
    _fields_ = [("q_amax", C.c_float), ("k_amax", C.c_float), ("v_amax", C.c_float), ("o_amax", C.c_float),
                ("s_max", C.c_float)]

    def __init__(self, q_amax=0.0, k_amax=0.0, v_amax=0.0, o_amax=1.0, s_max=1.0):
        super().__init__(q_amax, k_amax, v_amax, o_amax, s_max)


class FMHAError(RuntimeError):
    def __init__(self, status, text):
        super().__init__("FMHAInferI8 failed with status %d: %s" % (status, text))
        self.status = status


_lib = None


def load_library(path=None):
    """dlopen libfmha_i8.so and declare the prototypes of include/fmha_i8.h.  Raises if the library is absent."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise FileNotFoundError(
            "%s is not built; run `python -c 'import __graft_entry__ as g; g.build()'` at the repository root "
            "(there is no CPU fallback for this path)" % p)
    # A process must hold ONE HIP runtime.  PyTorch-ROCm wheels carry their own libamdhip64.so.7; importing torch first
    # makes the dynamic linker satisfy this library's libamdhip64.so.7 dependency with that already-loaded copy.  The
    # opposite order (system runtime first, torch's second) leaves the process with a runtime that finds no device.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = C.CDLL(p)
    ptr = C.c_void_p
    L.FMHAInferI8.argtypes = [ptr, FMHAParamI8, AttnDataDescriptor, ptr, ptr, ptr, ptr, ptr, C.c_bool]
    L.FMHAInferI8.restype = None
    L.FMHAInferI8Status.argtypes = L.FMHAInferI8.argtypes
    L.FMHAInferI8Status.restype = C.c_int
    L.FMHAInferI8CheckArgs.argtypes = [FMHAParamI8, AttnDataDescriptor, ptr, ptr, ptr, ptr, ptr]
    L.FMHAInferI8CheckArgs.restype = C.c_int
    L.FMHAInferI8StatusString.argtypes = [C.c_int]
    L.FMHAInferI8StatusString.restype = C.c_char_p
    L.FMHAInferI8Version.argtypes = []
    L.FMHAInferI8Version.restype = C.c_char_p
    L.FMHAInferI8Cross.argtypes = [ptr, FMHAParamI8, FMHACrossAttnDescriptor, ptr, ptr, ptr, ptr, ptr]
    L.FMHAInferI8Cross.restype = C.c_int
    L.FMHAInferI8CrossFullRangeP.argtypes = L.FMHAInferI8Cross.argtypes
    L.FMHAInferI8CrossFullRangeP.restype = C.c_int
    L.FMHAInferI8CrossCheckArgs.argtypes = [FMHAParamI8, FMHACrossAttnDescriptor, ptr, ptr, ptr, ptr, ptr]
    L.FMHAInferI8CrossCheckArgs.restype = C.c_int
    # include/fmha_quant.h
    L.FMHAAbsMaxF32.argtypes = [ptr, ptr, C.c_longlong, ptr]
    L.FMHAAbsMaxF32.restype = C.c_int
    L.FMHAQuantizeI8.argtypes = [ptr, ptr, C.c_longlong, C.c_float, ptr, ptr]
    L.FMHAQuantizeI8.restype = C.c_int
    L.FMHADequantizeI8.argtypes = [ptr, ptr, C.c_longlong, C.c_float, ptr]
    L.FMHADequantizeI8.restype = C.c_int
    L.FMHAAbsMaxBF16.argtypes = L.FMHAAbsMaxF32.argtypes
    L.FMHAAbsMaxBF16.restype = C.c_int
    L.FMHAQuantizeI8BF16.argtypes = L.FMHAQuantizeI8.argtypes
    L.FMHAQuantizeI8BF16.restype = C.c_int
    L.FMHADequantizeI8BF16.argtypes = L.FMHADequantizeI8.argtypes
    L.FMHADequantizeI8BF16.restype = C.c_int
    if path is None:
        _lib = L
    return L


def _ptr(x):
    if x is None:
        return None
    if hasattr(x, "data_ptr"):
        return x.data_ptr()
    return int(x)


def _stream(s):
    if s is None:
        return None
    if hasattr(s, "cuda_stream"):
        return s.cuda_stream
    return int(s)


def FMHAInferI8(stream, fmha_param, attn_desc, q, k, v, padding_mask, o, use_tcu=True):
    """Drop-in for gpuImpl::FMHAInferI8 (src/fmha_i8.cu:157-173): enqueue, return nothing, never synchronise."""
    load_library().FMHAInferI8(_stream(stream), fmha_param, attn_desc, _ptr(q), _ptr(k), _ptr(v), _ptr(padding_mask),
                               _ptr(o), bool(use_tcu))


def FMHAInferI8Status(stream, fmha_param, attn_desc, q, k, v, padding_mask, o, use_tcu=True):
    """Same launch, returning the status code of include/fmha_i8.h."""
    return int(load_library().FMHAInferI8Status(_stream(stream), fmha_param, attn_desc, _ptr(q), _ptr(k), _ptr(v),
                                                _ptr(padding_mask), _ptr(o), bool(use_tcu)))


def FMHAInferI8CheckArgs(fmha_param, attn_desc, q, k, v, padding_mask, o):
    return int(load_library().FMHAInferI8CheckArgs(fmha_param, attn_desc, _ptr(q), _ptr(k), _ptr(v),
                                                   _ptr(padding_mask), _ptr(o)))


def FMHAInferI8Cross(stream, fmha_param, desc, q, k, v, padding_mask, o):
    """seq_len_q queries over seq_len_kv keys; status code of include/fmha_i8.h."""
    return int(load_library().FMHAInferI8Cross(_stream(stream), fmha_param, desc, _ptr(q), _ptr(k), _ptr(v),
                                               _ptr(padding_mask), _ptr(o)))


def FMHAInferI8CrossFullRangeP(stream, fmha_param, desc, q, k, v, padding_mask, o):
    """FMHAInferI8Cross with P = rne(255 p) on all 255 steps of a byte (README.md:15,186 of the reference plans it)."""
    return int(load_library().FMHAInferI8CrossFullRangeP(_stream(stream), fmha_param, desc, _ptr(q), _ptr(k), _ptr(v),
                                                         _ptr(padding_mask), _ptr(o)))


def FMHAInferI8CrossCheckArgs(fmha_param, desc, q, k, v, padding_mask, o):
    return int(load_library().FMHAInferI8CrossCheckArgs(fmha_param, desc, _ptr(q), _ptr(k), _ptr(v),
                                                        _ptr(padding_mask), _ptr(o)))


def status_string(status):
    return load_library().FMHAInferI8StatusString(int(status)).decode()


def version():
    return load_library().FMHAInferI8Version().decode()


def _check(status):
    if status != FMHA_I8_OK:
        raise FMHAError(status, status_string(status) if status < 1000 else "HIP error %d" % (status - 1000))


def FMHAAbsMaxF32(stream, x, n, amax_out):
    """abs_max (inc/utils.hpp:31-39) on the GPU: *amax_out = max |x[i]|, device pointers, status code."""
    return int(load_library().FMHAAbsMaxF32(_stream(stream), _ptr(x), int(n), _ptr(amax_out)))


def FMHAQuantizeI8(stream, x, n, amax_host, amax_dev, out):
    """float_quant2_int8 (inc/utils.hpp:23-29) over n floats on the GPU; amax from device memory when amax_dev is given."""
    return int(load_library().FMHAQuantizeI8(_stream(stream), _ptr(x), int(n), float(amax_host), _ptr(amax_dev), _ptr(out)))


def FMHADequantizeI8(stream, x, n, amax, out):
    """(float)x / 127 * amax (inc/utils.hpp:53) over n int8 values on the GPU."""
    return int(load_library().FMHADequantizeI8(_stream(stream), _ptr(x), int(n), float(amax), _ptr(out)))


def FMHAAbsMaxBF16(stream, x, n, amax_out):
    """FMHAAbsMaxF32 for a bfloat16 tensor (raw 16-bit patterns)."""
    return int(load_library().FMHAAbsMaxBF16(_stream(stream), _ptr(x), int(n), _ptr(amax_out)))


def FMHAQuantizeI8BF16(stream, x, n, amax_host, amax_dev, out):
    """FMHAQuantizeI8 for a bfloat16 tensor: same roundings as on the widened floats."""
    return int(load_library().FMHAQuantizeI8BF16(_stream(stream), _ptr(x), int(n), float(amax_host), _ptr(amax_dev), _ptr(out)))


def FMHADequantizeI8BF16(stream, x, n, amax, out):
    """FMHADequantizeI8 with the result rounded to bfloat16 (nearest even)."""
    return int(load_library().FMHADequantizeI8BF16(_stream(stream), _ptr(x), int(n), float(amax), _ptr(out)))


def quantize_tensor(x, amax=None, stream=None):
    """Convenience for a contiguous float32 or bfloat16 torch tensor on the GPU: returns (int8 tensor, amax as a
    1-element float32 device tensor).  With amax=None the maximum is measured on the GPU and never visits the host."""
    import torch
    if not (x.is_cuda and x.dtype in (torch.float32, torch.bfloat16) and x.is_contiguous()):
        raise ValueError("x must be a contiguous float32 or bfloat16 tensor on the GPU")
    absmax, quant = (FMHAAbsMaxF32, FMHAQuantizeI8) if x.dtype == torch.float32 else (FMHAAbsMaxBF16, FMHAQuantizeI8BF16)
    st = stream if stream is not None else torch.cuda.current_stream(x.device)
    out = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    if amax is None:
        a = torch.empty(1, dtype=torch.float32, device=x.device)
        _check(absmax(st, x, x.numel(), a))
        _check(quant(st, x, x.numel(), 0.0, a, out))
    else:
        a = torch.full((1,), float(amax), dtype=torch.float32, device=x.device)
        _check(quant(st, x, x.numel(), float(amax), None, out))
    return out, a


def dequantize_tensor(x, amax, stream=None, dtype=None):
    """int8 torch tensor on the GPU -> float32 (default) or bfloat16, (float)x / 127 * amax."""
    import torch
    if not (x.is_cuda and x.dtype == torch.int8 and x.is_contiguous()):
        raise ValueError("x must be a contiguous int8 tensor on the GPU")
    dtype = dtype or torch.float32
    if dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("dtype must be float32 or bfloat16")
    st = stream if stream is not None else torch.cuda.current_stream(x.device)
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    _check((FMHADequantizeI8 if dtype == torch.float32 else FMHADequantizeI8BF16)(st, x, x.numel(), float(amax), out))
    return out


def fmha_infer_i8(q, k, v, padding_mask, q_amax, k_amax, v_amax, o_amax=1.0, out=None, stream=None,
                  full_range_p=False):
    """Convenience over FMHAInferI8Status for torch int8 tensors on the GPU.

    q: int8 [B, H, Sq, d]; k, v: int8 [B, H, S, d], all contiguous; padding_mask: int8 [B, S], nonzero = key masked
    out (inc/fmha_i8.cuh:189-192).  Returns int8 O [B, H, Sq, d].  Sq == S goes through the reference's entry point
    (FMHAInferI8Status), anything else through FMHAInferI8Cross; full_range_p=True selects
    FMHAInferI8CrossFullRangeP (P on 255 steps instead of 128).  Raises FMHAError on a nonzero status."""
    import torch

    for name, t in (("q", q), ("k", k), ("v", v), ("padding_mask", padding_mask)):
        if not (t.is_cuda and t.dtype == torch.int8 and t.is_contiguous()):
            raise ValueError("%s must be a contiguous int8 tensor on the GPU" % name)
    B, H, Sq, d = q.shape
    S = k.shape[2] if k.dim() == 4 else -1
    if tuple(k.shape) != (B, H, S, d) or v.shape != k.shape or tuple(padding_mask.shape) != (B, S):
        raise ValueError("shape mismatch: q [B,H,Sq,d], k/v [B,H,S,d] and padding_mask [B,S] expected")
    if out is None:
        out = torch.empty_like(q)
    elif not (out.is_cuda and out.dtype == torch.int8 and out.is_contiguous() and out.shape == q.shape):
        raise ValueError("out must be a contiguous int8 tensor on the GPU, shaped like q")
    if stream is None:
        stream = torch.cuda.current_stream(q.device)
    param = FMHAParamI8(q_amax, k_amax, v_amax, o_amax, 1.0)
    if full_range_p:
        st = FMHAInferI8CrossFullRangeP(stream, param, FMHACrossAttnDescriptor(B, Sq, S, H, d), q, k, v, padding_mask,
                                        out)
    elif Sq == S:
        st = FMHAInferI8Status(stream, param, AttnDataDescriptor(B, S, H, d), q, k, v, padding_mask, out, True)
    else:
        st = FMHAInferI8Cross(stream, param, FMHACrossAttnDescriptor(B, Sq, S, H, d), q, k, v, padding_mask, out)
    if st != FMHA_I8_OK:
        raise FMHAError(st, status_string(st))
    return out


def fmha_infer_from_float(q, k, v, padding_mask, o_amax, out_dtype=None, stream=None, full_range_p=False):
    """The flow of the reference's driver with every step on the GPU (test_fmha_i8.cpp:91-110 quantises Q, K and V on the
    host by their abs-max, :204-222 launches the kernel, inc/utils.hpp:53 de-quantises O): q [B,H,Sq,d] and k, v
    [B,H,S,d] are contiguous float32 or bfloat16 tensors on the GPU, padding_mask int8 [B,S] (nonzero = masked out),
    o_amax the range the int8 output is scaled to (the driver takes max |O| of its float path).  Returns
    (O as out_dtype - default: q's dtype -, int8 O, (q_amax, k_amax, v_amax)).  The three maxima are read back in one
    copy because FMHAParamI8 is passed by value, as in the reference; nothing else leaves the device."""
    import torch
    if stream is None:
        st = torch.cuda.current_stream(q.device)
    elif isinstance(stream, torch.cuda.Stream):
        st = stream
    else:
        # Every tensor of the flow is allocated by torch's caching allocator, which orders the reuse of a block by the
        # stream it was allocated under; a raw handle gives it nothing to order by.
        raise TypeError("stream must be a torch.cuda.Stream (or None for the current one), not %r" % type(stream))
    # The whole flow runs with `st` as torch's current stream: the intermediate and output tensors are then allocated
    # under the stream that the kernels writing them are queued on.
    with torch.cuda.stream(st):
        (qi, qa), (ki, ka), (vi, va) = (quantize_tensor(t, stream=st) for t in (q, k, v))
        amax = [float(x) for x in torch.cat((qa, ka, va)).cpu()]  # the one synchronisation of the flow
        if min(amax) <= 0.0:
            raise ValueError("q, k and v must each hold a nonzero value (abs-max %r)" % (amax,))
        o_i8 = fmha_infer_i8(qi, ki, vi, padding_mask, amax[0], amax[1], amax[2], o_amax, stream=st,
                             full_range_p=full_range_p)
        o = dequantize_tensor(o_i8, o_amax, stream=st, dtype=out_dtype or q.dtype)
    return o, o_i8, tuple(amax)
