"""ctypes binding of ``libblackriver.so`` (the C embedding API declared in
include/br_host.h): boot the C++ host runtime, run word scripts, move tensor
contents.  Plumbing for drivers, tests and benchmarks written in Python; no
fallback exists if the library has not been built.
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
# BR_SANITIZE=1 selects the ASan + UBSan build of the host runtime
# (`python -m blackriver_amd.build --sanitize`; the interpreter then needs
# libasan preloaded)
LIB_PATH = os.path.join(_PKG, "lib", "sanitize" if os.environ.get("BR_SANITIZE") == "1" else "", "libblackriver.so")
WORDS_DIR = os.path.join(_PKG, "words")

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_cp = ctypes.c_char_p
_dp = ctypes.POINTER(ctypes.c_double)
_ip = ctypes.POINTER(_int)
_f32p = ctypes.POINTER(ctypes.c_float)
_i32p = ctypes.POINTER(ctypes.c_int32)

SIGNATURES = {
    "br_host_boot": (_int, [_int, ctypes.c_size_t]),
    "br_host_shutdown": (_int, []),
    "br_host_last_error": (_cp, []),
    "br_host_stream": (_vp, []),
    "br_host_sync": (_int, []),
    "br_host_set_fp32_gemm_compute": (_int, [_int]),
    "br_env_create": (_vp, [_int]),
    "br_env_destroy": (None, [_vp]),
    "br_env_execute": (_int, [_vp, _cp]),
    "br_env_build": (_int, [_vp, _cp, _ip]),
    "br_env_run": (_int, [_vp, _int]),
    "br_env_disassemble_fused": (_int, [_vp, _cp, ctypes.c_char_p, ctypes.c_size_t]),
    "br_env_change_hash": (_int, [_vp, _int]),
    "br_env_current_hash": (_int, [_vp]),
    "br_env_set_number": (_int, [_vp, _cp, ctypes.c_double]),
    "br_env_set_string": (_int, [_vp, _cp, _cp]),
    "br_env_get_number": (_int, [_vp, _cp, _dp]),
    "br_env_has": (_int, [_vp, _cp]),
    "br_env_stack_size": (_int, [_vp]),
    "br_env_stack_clear": (_int, [_vp]),
    "br_env_stack_pop_number": (_int, [_vp, _dp]),
    "br_env_disassemble": (_int, [_vp, _cp, ctypes.c_char_p, ctypes.c_size_t]),
    "br_env_tensor_info": (_int, [_vp, _cp, _ip, _ip, _ip, ctypes.POINTER(_i64), ctypes.POINTER(_vp)]),
    "br_env_tensor_write": (_int, [_vp, _cp, _f32p, _i64]),
    "br_env_tensor_read": (_int, [_vp, _cp, _f32p, _i64]),
    "br_env_tensor_write_i32": (_int, [_vp, _cp, _i32p, _i64]),
    "br_env_tensor_read_i32": (_int, [_vp, _cp, _i32p, _i64]),
    "br_host_set_echo_loss": (_int, [_int]),
    "br_bloom_model_create": (_int, [_vp, _int, _i64, _i64, _i64, _i64, _i64, ctypes.c_float, _cp, _cp]),
    "br_bloom_model_set_fused_attention": (_int, [_vp, _int]),
    "br_bloom_model_init": (_int, [_vp, ctypes.c_uint64, ctypes.c_float]),
    "br_bloom_model_step": (_int, [_vp, _i32p, _i32p, ctypes.POINTER(ctypes.c_float)]),
    "br_bloom_model_grad_lift": (_int, [_vp, ctypes.POINTER(ctypes.c_float)]),
    "br_bloom_model_optimizer_create": (_int, [_vp] + [ctypes.c_float] * 5),
    "br_bloom_model_optimizer_step": (_int, [_vp]),
    "br_bloom_fetch_data": (_int, [_i32p, _i32p, _i64, _i64, _f32p, _i64, _i64, _f32p, _f32p, _f32p]),
}

_lib = None


class HostError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HostError("%s is missing: build it with `python -m blackriver_amd.build`" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def _check(rc, what):
    if rc != 0:
        raise HostError("%s: %s" % (what, load().br_host_last_error().decode(errors="replace")))


_booted = False


def boot(device: int = 0, host_arena_bytes: int = 1 << 30) -> None:
    """Boot the runtime once per process (device < 0: host only)."""
    global _booted
    if _booted:
        raise HostError("runtime already booted")
    _check(load().br_host_boot(device, host_arena_bytes), "br_host_boot")
    _booted = True


def shutdown() -> None:
    global _booted
    if _booted:
        _check(load().br_host_shutdown(), "br_host_shutdown")
        _booted = False


def booted() -> bool:
    return _booted


def stream():
    return load().br_host_stream()


def sync() -> None:
    _check(load().br_host_sync(), "br_host_sync")


def set_echo_loss(on: bool) -> None:
    """Whether op.loss_backward prints its '#################  count loss' line."""
    load().br_host_set_echo_loss(1 if on else 0)


def words_text(name: str) -> str:
    """Text of one of the word scripts shipped with the package."""
    with open(os.path.join(WORDS_DIR, name)) as f:
        return f.read()


class Env:
    """An Enviroment with the io.*, op.* and bloom.* words loaded."""

    def __init__(self, hashes: int = 1):
        self._lib = load()
        self._h = self._lib.br_env_create(hashes)
        if not self._h:
            raise HostError("br_env_create: " + self._lib.br_host_last_error().decode())

    def close(self):
        if self._h:
            self._lib.br_env_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def execute(self, text: str) -> None:
        rc = self._lib.br_env_execute(self._h, text.encode())
        if rc != 0:
            self._lib.br_env_stack_clear(self._h)
        _check(rc, "execute")

    def build(self, text: str) -> int:
        prog = _int(-1)
        _check(self._lib.br_env_build(self._h, text.encode(), ctypes.byref(prog)), "build")
        return prog.value

    def run(self, program: int) -> None:
        _check(self._lib.br_env_run(self._h, program), "run")

    def change_hash(self, h: int) -> None:
        _check(self._lib.br_env_change_hash(self._h, h), "change_hash")

    @property
    def current_hash(self) -> int:
        return self._lib.br_env_current_hash(self._h)

    def set(self, name: str, value) -> None:
        if isinstance(value, str):
            _check(self._lib.br_env_set_string(self._h, name.encode(), value.encode()), "set")
        else:
            _check(self._lib.br_env_set_number(self._h, name.encode(), float(value)), "set")

    def number(self, name: str) -> float:
        v = ctypes.c_double()
        _check(self._lib.br_env_get_number(self._h, name.encode(), ctypes.byref(v)), "number")
        return v.value

    def has(self, name: str) -> bool:
        return bool(self._lib.br_env_has(self._h, name.encode()))

    @property
    def stack_size(self) -> int:
        return self._lib.br_env_stack_size(self._h)

    def stack_clear(self) -> None:
        self._lib.br_env_stack_clear(self._h)

    def pop_number(self) -> float:
        v = ctypes.c_double()
        _check(self._lib.br_env_stack_pop_number(self._h, ctypes.byref(v)), "pop_number")
        return v.value

    def disassemble(self, text: str, fused: bool = False) -> list:
        """Compile and link `text`; return the flat step list as strings
        (after the fusion pass when `fused`)."""
        size = 1 << 20
        fn = self._lib.br_env_disassemble_fused if fused else self._lib.br_env_disassemble
        while True:
            buf = ctypes.create_string_buffer(size)
            rc = fn(self._h, text.encode(), buf, size)
            if rc == -2:
                size *= 4
                continue
            _check(rc, "disassemble")
            return buf.value.decode().split("\n")[:-1]

    def info(self, name: str):
        """(dtype code, on_device, shape tuple, data pointer) of a tensor."""
        dtype, dev, rank = _int(), _int(), _int()
        shape = (_i64 * 8)()
        data = _vp()
        _check(self._lib.br_env_tensor_info(self._h, name.encode(), ctypes.byref(dtype), ctypes.byref(dev),
                                            ctypes.byref(rank), shape, ctypes.byref(data)), "info(%s)" % name)
        return dtype.value, bool(dev.value), tuple(shape[i] for i in range(rank.value)), data.value

    def write(self, name: str, array) -> None:
        a = np.ascontiguousarray(array)
        if a.dtype == np.int32:
            _check(self._lib.br_env_tensor_write_i32(self._h, name.encode(), a.ctypes.data_as(_i32p), a.size),
                   "write(%s)" % name)
        else:
            a = np.ascontiguousarray(a, dtype=np.float32)
            _check(self._lib.br_env_tensor_write(self._h, name.encode(), a.ctypes.data_as(_f32p), a.size),
                   "write(%s)" % name)

    def read(self, name: str) -> np.ndarray:
        dtype, _, shape, _ = self.info(name)
        if dtype == 3:
            out = np.empty(shape, np.int32)
            _check(self._lib.br_env_tensor_read_i32(self._h, name.encode(), out.ctypes.data_as(_i32p), out.size),
                   "read(%s)" % name)
        else:
            out = np.empty(shape, np.float32)
            _check(self._lib.br_env_tensor_read(self._h, name.encode(), out.ctypes.data_as(_f32p), out.size),
                   "read(%s)" % name)
        return out


class BloomModel:
    """A whole BLOOM model on one GPU (C++ driver BloomTrainer): block i in
    hash i of `env`, embedding / final LayerNorm / LM head in hash 0."""

    def __init__(self, layers, batch, tokens, hidden=4096, heads=32, vocab=250880, eps=1e-5, weight_dtype="f16",
                 gemm_precision="f16", fused_attention=True):
        self.layers, self.batch, self.tokens = layers, batch, tokens
        self.hidden, self.heads, self.vocab, self.eps = hidden, heads, vocab, eps
        self.env = Env(layers + 1)
        self.env.execute(words_text("bloom.words"))
        self.env.execute(words_text("bloom_model.words"))
        _check(load().br_bloom_model_set_fused_attention(self.env._h, 1 if fused_attention else 0), "model_attention")
        _check(load().br_bloom_model_create(self.env._h, layers, batch, tokens, hidden, heads, vocab, eps,
                                            weight_dtype.encode(), gemm_precision.encode()), "model_create")

    def init(self, seed=0, std=0.02):
        _check(load().br_bloom_model_init(self.env._h, seed, std), "model_init")

    def step(self, ids, mask) -> float:
        ids = np.ascontiguousarray(ids, np.int32)
        mask = np.ascontiguousarray(mask, np.int32)
        assert ids.shape == (self.batch, self.tokens) and mask.shape == ids.shape
        loss = ctypes.c_float()
        _check(load().br_bloom_model_step(self.env._h, ids.ctypes.data_as(_i32p), mask.ctypes.data_as(_i32p),
                                          ctypes.byref(loss)), "model_step")
        return loss.value

    def grad_lift(self) -> float:
        """Power of two the last step's activation gradients were carried at
        (parameter gradients are at their true scale)."""
        v = ctypes.c_float()
        _check(load().br_bloom_model_grad_lift(self.env._h, ctypes.byref(v)), "grad_lift")
        return v.value

    def create_optimizer(self, lr=1e-4, beta1=0.9, beta2=0.95, eps=1e-8, weight_decay=0.0):
        """AdamW state (moments, fp32 masters of 16-bit matrices).  Call after
        the weights have their starting values."""
        _check(load().br_bloom_model_optimizer_create(self.env._h, lr, beta1, beta2, eps, weight_decay),
               "optimizer_create")

    def optimizer_step(self):
        _check(load().br_bloom_model_optimizer_step(self.env._h), "optimizer_step")

    def read(self, layer, name):
        self.env.change_hash(layer)
        out = self.env.read(name)
        self.env.change_hash(0)
        return out

    def write(self, layer, name, array):
        self.env.change_hash(layer)
        self.env.write(name, array)
        self.env.change_hash(0)

    def close(self):
        self.env.close()


def fetch_data(ids, mask, heads, vocab=None):
    """Host batch preparation: (xinput or None, alibi[heads,T], xmask[B,T,T])."""
    ids = np.ascontiguousarray(ids, np.int32)
    mask = np.ascontiguousarray(mask, np.int32)
    b, t = ids.shape
    alibi = np.empty((heads, t), np.float32)
    xmask = np.empty((b, t, t), np.float32)
    xinput = None
    vp, hidden = None, 0
    if vocab is not None:
        vocab = np.ascontiguousarray(vocab, np.float32)
        hidden = vocab.shape[1]
        xinput = np.empty((b, t, hidden), np.float32)
        vp = vocab.ctypes.data_as(_f32p)
    _check(load().br_bloom_fetch_data(ids.ctypes.data_as(_i32p), mask.ctypes.data_as(_i32p), b, t, vp, hidden, heads,
                                      xinput.ctypes.data_as(_f32p) if xinput is not None else None,
                                      alibi.ctypes.data_as(_f32p), xmask.ctypes.data_as(_f32p)), "fetch_data")
    return xinput, alibi, xmask
