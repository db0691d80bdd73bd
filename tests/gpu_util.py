"""Helpers for the GPU parity tests: torch is used only to own device memory
and the stream; every computation goes through the C ABI of libbr_hip.so."""
import ctypes

import numpy as np
import torch

from blackriver_amd import hip

F32, F16, BF16, I32 = hip.F32, hip.F16, hip.BF16, hip.I32


_KEEP = []


def dev(a):
    """numpy array -> device tensor (fp16 passes as torch.float16).  The
    tensor is kept alive until release() so that `ptr(dev(x))` is safe: a
    temporary freed before the asynchronous kernel runs could be handed out
    again by torch's caching allocator."""
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    _KEEP.append(t)
    return t


def release():
    torch.cuda.synchronize()
    _KEEP.clear()


def empty(shape, dtype=torch.float32):
    return torch.empty(shape, dtype=dtype, device="cuda")


def host(t):
    torch.cuda.synchronize()
    return t.detach().cpu().numpy()


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def call(name, *args):
    hip.call(name, *args)


def workspace(nbytes):
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device="cuda")


def f16_ulp(ref):
    """Spacing of fp16 numbers around |ref| (subnormal spacing below 2^-14)."""
    a = np.abs(np.asarray(ref, np.float64))
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -14)))
    return 2.0 ** (e - 10)


def assert_close_f16(got, ref, rtol, what=""):
    """For fp16-stored results of fp32 math: the fp32 bound of assert_close
    plus half an fp16 ulp of the reference for the final rounding (0.52 to
    leave room for the double rounding fp64 -> fp32 -> fp16)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape
    assert np.all(np.isfinite(got)), what
    rms = float(np.sqrt(np.mean(ref * ref)))
    bound = rtol * (np.abs(ref) + rms) + 0.52 * f16_ulp(ref)
    worst = float(np.max(np.abs(got - ref) / bound))
    assert worst <= 1.0, "%s: worst error %.3g x the bound" % (what, worst)
