"""ctypes/numpy front end of the CPU oracle (``libbr_oracle.so``).

TEST INFRASTRUCTURE ONLY: the parity checker and the timed CPU baseline.  The
shipped package never imports this module.

Every wrapper takes and returns C-contiguous numpy arrays (fp32, int32) and
forwards to the C restatement in ``br_oracle.c``; see ``br_oracle.h`` for the
reference file:line each function follows.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libbr_oracle.so")
if os.environ.get("BR_SANITIZE") == "1":   # the ASan + UBSan build made by `python -m blackriver_amd.build --sanitize`
    _LIB_PATH = os.path.join(os.path.dirname(_HERE), "blackriver_amd", "lib", "sanitize", "libbr_oracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_i32p = ctypes.POINTER(ctypes.c_int32)
_i64p = ctypes.POINTER(ctypes.c_int64)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_i64 = ctypes.c_int64
_f32 = ctypes.c_float


def build() -> str:
    """Compile the oracle with its Makefile and return the library path."""
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_loss_labels.restype = _i64
        _lib.orc_loss_groups.restype = _i64
        _lib.orc_loss_backward.restype = _f32
        _lib.orc_logsoftmax_nll.restype = _f32
        _lib.orc_threads.restype = ctypes.c_int
    return _lib


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _i(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _p(a):
    if a is None:
        return None
    if a.dtype == np.float32:
        return a.ctypes.data_as(_f32p)
    if a.dtype == np.int32:
        return a.ctypes.data_as(_i32p)
    if a.dtype == np.int64:
        return a.ctypes.data_as(_i64p)
    if a.dtype == np.uint16:
        return a.ctypes.data_as(_u16p)
    raise TypeError(a.dtype)


def threads() -> int:
    return int(lib().orc_threads())


# ---------------------------------------------------------------- LayerNorm
def layernorm_fwd(x, gamma, beta, eps):
    x, gamma, beta = _f(x), _f(gamma), _f(beta)
    cols = x.shape[-1]
    rows = x.size // cols
    y = np.empty_like(x)
    mean = np.empty(rows, np.float32)
    var = np.empty(rows, np.float32)
    lib().orc_layernorm_fwd(_p(x), _p(gamma), _p(beta), _p(y), _p(mean), _p(var),
                            _i64(rows), _i64(cols), _f32(eps))
    return y, mean, var


def layernorm_bwd(dy, y, gamma, beta, var, eps):
    dy, y, gamma, beta, var = _f(dy), _f(y), _f(gamma), _f(beta), _f(var)
    cols = dy.shape[-1]
    rows = dy.size // cols
    dgamma = np.empty(cols, np.float32)
    dbeta = np.empty(cols, np.float32)
    dx = np.empty_like(dy)
    lib().orc_layernorm_bwd(_p(dy), _p(y), _p(gamma), _p(beta), _p(var), _p(dgamma),
                            _p(dbeta), _p(dx), _i64(rows), _i64(cols), _f32(eps))
    return dx, dgamma, dbeta


# --------------------------------------------------------------------- GELU
def gelu_fwd(x):
    x = _f(x)
    y = np.empty_like(x)
    lib().orc_gelu_fwd(_p(x), _p(y), _i64(x.size))
    return y


def gelu_bwd(dy, x):
    dy, x = _f(dy), _f(x)
    dx = np.empty_like(x)
    lib().orc_gelu_bwd(_p(dy), _p(x), _p(dx), _i64(x.size))
    return dx


def bias_gelu_fwd(x, bias):
    x, bias = _f(x), _f(bias)
    cols = x.shape[-1]
    y = np.empty_like(x)
    lib().orc_bias_gelu_fwd(_p(x), _p(bias), _p(y), _i64(x.size // cols), _i64(cols))
    return y


def bias_gelu_bwd(dy, x, bias):
    dy, x, bias = _f(dy), _f(x), _f(bias)
    cols = x.shape[-1]
    dx = np.empty_like(x)
    dbias = np.empty(cols, np.float32)
    lib().orc_bias_gelu_bwd(_p(dy), _p(x), _p(bias), _p(dx), _p(dbias),
                            _i64(x.size // cols), _i64(cols))
    return dx, dbias


# ------------------------------------------------------------------- Linear
def linear_fwd(x, w, b):
    x, w, b = _f(x), _f(w), _f(b)
    out, inn = w.shape
    n = x.size // inn
    y = np.empty(x.shape[:-1] + (out,), np.float32)
    lib().orc_linear_fwd(_p(x), _p(w), _p(b), _p(y), _i64(n), _i64(inn), _i64(out))
    return y


def linear_bwd(dy, x, w):
    dy, x, w = _f(dy), _f(x), _f(w)
    out, inn = w.shape
    n = x.size // inn
    dx = np.empty_like(x)
    dw = np.empty_like(w)
    db = np.empty(out, np.float32)
    lib().orc_linear_bwd(_p(dy), _p(x), _p(w), _p(dx), _p(dw), _p(db), _i64(n),
                         _i64(inn), _i64(out))
    return dx, dw, db


# ---------------------------------------------------------- shape shuffling
def transpose_0213(x):
    x = _f(x)
    s0, s1, s2, s3 = x.shape
    y = np.empty((s0, s2, s1, s3), np.float32)
    lib().orc_transpose_0213(_p(x), _p(y), _i64(s0), _i64(s1), _i64(s2), _i64(s3))
    return y


def _shape4(shape):
    """Rank <= 4 to rank 4, the way the reference builds cuDNN descriptors
    (blackriver/cuda_tensor.hpp:39-49)."""
    s = list(shape)
    if len(s) == 4:
        return s
    if len(s) == 3:
        return [s[0], s[1], 1, s[2]]
    if len(s) == 2:
        return [s[0], s[1], 1, 1]
    if len(s) == 1:
        return [1, s[0], 1, 1]
    raise ValueError(shape)


def add_bcast(a, b):
    a, b = _f(a), _f(b)
    ash = np.array(_shape4(a.shape), np.int64)
    bsh = np.array(_shape4(b.shape), np.int64)
    for x, y in zip(ash, bsh):
        if y != 1 and x != y:
            raise ValueError("b must match a or be 1 in every dimension")
    c = np.empty_like(a)
    lib().orc_add_bcast(_p(a), _p(ash), _p(b), _p(bsh), _p(c))
    return c


# ---------------------------------------------------------------- attention
def qk(q, k):
    q, k = _f(q), _f(k)
    b, h, t, hd = q.shape
    s = np.empty((b, h, t, t), np.float32)
    lib().orc_qk(_p(q), _p(k), _p(s), _i64(b * h), _i64(t), _i64(hd))
    return s


def softmax_fwd(x):
    x = _f(x)
    cols = x.shape[-1]
    y = np.empty_like(x)
    lib().orc_softmax_fwd(_p(x), _p(y), _i64(x.size // cols), _i64(cols))
    return y


def softmax_bwd(dy, y):
    dy, y = _f(dy), _f(y)
    cols = y.shape[-1]
    dx = np.empty_like(y)
    lib().orc_softmax_bwd(_p(dy), _p(y), _p(dx), _i64(y.size // cols), _i64(cols))
    return dx


def attn(p, v):
    p, v = _f(p), _f(v)
    b, h, t, hd = v.shape
    o = np.empty_like(v)
    lib().orc_attn(_p(p), _p(v), _p(o), _i64(b * h), _i64(t), _i64(hd))
    return o


def attn_bwd(d_o, p, v):
    d_o, p, v = _f(d_o), _f(p), _f(v)
    b, h, t, hd = v.shape
    dp = np.empty_like(p)
    dv = np.empty_like(v)
    lib().orc_attn_bwd(_p(d_o), _p(p), _p(v), _p(dp), _p(dv), _i64(b * h), _i64(t), _i64(hd))
    return dp, dv


def softmax_attn_bwd(d_o, p, v):
    d_o, p, v = _f(d_o), _f(p), _f(v)
    b, h, t, hd = v.shape
    ds = np.empty_like(p)
    dv = np.empty_like(v)
    lib().orc_softmax_attn_bwd(_p(d_o), _p(p), _p(v), _p(ds), _p(dv), _i64(b * h),
                               _i64(t), _i64(hd))
    return ds, dv


def qk_bwd(ds, q, k):
    ds, q, k = _f(ds), _f(q), _f(k)
    b, h, t, hd = q.shape
    dq = np.empty_like(q)
    dk = np.empty_like(k)
    lib().orc_qk_bwd(_p(ds), _p(q), _p(k), _p(dq), _p(dk), _i64(b * h), _i64(t), _i64(hd))
    return dq, dk


# ---------------------------------------------------------------- loss head
def last_logits(x, mask, lm_head):
    x, mask, lm_head = _f(x), _i(mask), _f(lm_head)
    b, t, h = x.shape
    v = lm_head.shape[0]
    out = np.empty((b, v), np.float32)
    lib().orc_last_logits(_p(x), _p(mask), _p(lm_head), _p(out), _i64(b), _i64(t),
                          _i64(h), _i64(v))
    return out


def loss_labels(ids, mask):
    ids, mask = _i(ids), _i(mask)
    b, t = ids.shape
    labels = np.empty((b, t), np.int32)
    count = lib().orc_loss_labels(_p(ids), _p(mask), _i64(b), _i64(t), _p(labels))
    return labels, int(count)


def loss_groups(mask, group_max):
    mask = _i(mask)
    b, t = mask.shape
    cap = b * (t // max(1, group_max) + 2)
    triples = np.zeros((cap, 3), np.int64)
    n = lib().orc_loss_groups(_p(mask), _i64(b), _i64(t), _i64(group_max), _p(triples),
                              _i64(cap))
    return triples[:n].copy()


def loss_backward(x, ids, mask, lm_head, lm_head_g=None, want_dlogits=False):
    x, ids, mask, lm_head = _f(x), _i(ids), _i(mask), _f(lm_head)
    b, t, h = x.shape
    v = lm_head.shape[0]
    x_g = np.empty_like(x)
    if lm_head_g is None:
        lm_head_g = np.zeros_like(lm_head)
    else:
        lm_head_g = _f(lm_head_g).copy()
    dl = np.empty((b * t, v), np.float32) if want_dlogits else None
    loss = lib().orc_loss_backward(_p(x), _p(ids), _p(mask), _p(lm_head), _p(x_g),
                                   _p(lm_head_g), _p(dl), _i64(b), _i64(t), _i64(h), _i64(v))
    return float(loss), x_g, lm_head_g, dl


def logsoftmax_nll(logits, target, keep, want_dlogits=True):
    logits, target, keep = _f(logits), _i(target), _i(keep)
    rows, vocab = logits.shape
    lse = np.empty(rows, np.float32)
    dl = np.empty_like(logits) if want_dlogits else None
    loss = lib().orc_logsoftmax_nll(_p(logits), _p(target), _p(keep), _p(lse), _p(dl),
                                    _i64(rows), _i64(vocab))
    return float(loss), lse, dl


# --------------------------------------------------------------- fetch_data
def embedding_gather(vocab, ids):
    vocab, ids = _f(vocab), _i(ids)
    h = vocab.shape[1]
    out = np.empty(ids.shape + (h,), np.float32)
    lib().orc_embedding_gather(_p(vocab), _p(ids), _p(out), _i64(ids.size), _i64(h))
    return out


def embedding_scatter_add(grad, dx, ids):
    """grad[ids[i]] += dx[i] in ascending i, in place on a copy; returns it."""
    grad = np.array(_f(grad), copy=True)
    dx, ids = _f(dx), _i(ids)
    lib().orc_embedding_scatter_add(_p(grad), _p(dx), _p(ids), _i64(ids.size), _i64(grad.shape[1]),
                                    _i64(grad.shape[0]))
    return grad


def alibi(heads, tokens):
    out = np.empty((heads, tokens), np.float32)
    lib().orc_alibi(_p(out), _i64(heads), _i64(tokens))
    return out


def xmask(mask):
    mask = _i(mask)
    b, t = mask.shape
    out = np.empty((b, t, t), np.float32)
    lib().orc_xmask(_p(mask), _p(out), _i64(b), _i64(t))
    return out


# ---------------------------------------------------------------------- f16
def f32_to_f16_bits(x):
    x = _f(x)
    y = np.empty(x.shape, np.uint16)
    lib().orc_f32_to_f16(_p(x), _p(y), _i64(x.size))
    return y


def f16_bits_to_f32(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    y = np.empty(x.shape, np.float32)
    lib().orc_f16_to_f32(_p(x), _p(y), _i64(x.size))
    return y


def adamw_step(param, grad, m, v, lr, beta1, beta2, eps, weight_decay, step):
    """One AdamW step in fp32, operation for operation the single-tensor update
    of torch.optim.AdamW (decoupled decay, lerp for the first moment, bias
    corrections from python floats).  The reference has no optimizer; pinned
    against torch.optim.AdamW itself in tests/test_oracle_ops.py.
    Returns (param, m, v) as new fp32 arrays."""
    f = np.float32
    p = _f(param) * f(1.0 - lr * weight_decay)
    g = _f(grad)
    m = _f(m) + (g - _f(m)) * f(1.0 - beta1)
    v = _f(v) * f(beta2) + (f(1.0 - beta2) * g) * g
    bc1 = 1.0 - beta1 ** step
    bc2 = 1.0 - beta2 ** step
    denom = np.sqrt(v) / f(bc2 ** 0.5) + f(eps)
    p = p - f(lr / bc1) * (m / denom)
    return p.astype(np.float32), m.astype(np.float32), v.astype(np.float32)
