"""MFMA GEMM kernel against fp64 products through the C ABI: every operand
layout, storage type and compute type, odd sizes, batching, bias, alpha and
accumulation.  Tolerances: 2e-2 relative for fp16 / bf16 operands, 1e-5 for
the fp32-operand kernel."""
import numpy as np
import pytest
import torch

from conftest import assert_close
from gpu_util import BF16, F16, F32, call, dev, empty, host, ptr, stream
from blackriver_amd import hip

pytestmark = pytest.mark.gpu

TORCH_T = {F32: torch.float32, F16: torch.float16, BF16: torch.bfloat16}


def to_dev(a, dtype):
    return torch.from_numpy(np.ascontiguousarray(a, np.float32)).cuda().to(TORCH_T[dtype]).contiguous()


def to_host64(t):
    torch.cuda.synchronize()
    return t.detach().float().cpu().numpy().astype(np.float64)


def run_gemm(ta, tb, m, n, k, a, b, a_dt, b_dt, c_dt, compute, alpha=1.0, bias=None, c0=None, batch=1):
    da, db_ = to_dev(a, a_dt), to_dev(b, b_dt)
    if c0 is not None:
        c = to_dev(c0, c_dt)
    else:
        c = torch.full((batch, m, n), float("nan"), dtype=TORCH_T[c_dt], device="cuda")
    dbias = dev(bias) if bias is not None else None
    lda = m if ta else k
    ldb = k if tb else n
    call("br_hip_gemm", int(ta), int(tb), m, n, k, alpha, ptr(da), a_dt, lda, m * k, ptr(db_), b_dt, ldb, n * k,
         1 if c0 is not None else 0, ptr(c), c_dt, n, m * n, ptr(dbias), batch, compute, stream())
    # reference from the operands as the kernel saw them (after storage rounding)
    A = to_host64(da).reshape(batch, *((k, m) if ta else (m, k)))
    B = to_host64(db_).reshape(batch, *((n, k) if tb else (k, n)))
    if ta:
        A = A.transpose(0, 2, 1)
    if tb:
        B = B.transpose(0, 2, 1)
    ref = alpha * np.einsum("bik,bkj->bij", A, B)
    if bias is not None:
        ref = ref + bias.astype(np.float64)[None, None, :]
    if c0 is not None:
        ref = ref + to_host64(to_dev(c0, c_dt)).reshape(batch, m, n)
    return to_host64(c).reshape(batch, m, n), ref


def operands(rng, ta, tb, m, n, k, batch=1):
    a = rng.standard_normal((batch,) + ((k, m) if ta else (m, k))).astype(np.float32)
    b = rng.standard_normal((batch,) + ((n, k) if tb else (k, n))).astype(np.float32)
    return a, b


@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("a_dt,b_dt,c_dt", [(F32, F32, F32), (F32, F16, F32), (F16, F16, F16), (F16, F32, F32)])
def test_gemm_f16_layouts_and_storage_types(ta, tb, a_dt, b_dt, c_dt):
    rng = np.random.default_rng(0)
    m, n, k = 256, 384, 160
    print("case ta=%d tb=%d dtypes=%s" % (ta, tb, (a_dt, b_dt, c_dt)), flush=True)
    a, b = operands(rng, ta, tb, m, n, k)
    got, ref = run_gemm(ta, tb, m, n, k, a, b, a_dt, b_dt, c_dt, hip.GEMM_F16)
    assert_close(got, ref, 2e-2, "gemm f16")
    # typical error is far below the bound: fp16 operand rounding only
    assert np.sqrt(np.mean((got - ref) ** 2)) < 3e-3 * np.sqrt(np.mean(ref ** 2)) + (1e-2 if c_dt == F16 else 0)


@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (5, 7, 3), (33, 65, 17), (130, 129, 40), (12, 12, 16), (128, 128, 32),
                                   (200, 100, 1000)])
def test_gemm_odd_sizes(ta, tb, m, n, k):
    rng = np.random.default_rng(1)
    print("case ta=%d tb=%d m=%d n=%d k=%d" % (ta, tb, m, n, k), flush=True)
    a, b = operands(rng, ta, tb, m, n, k)
    got, ref = run_gemm(ta, tb, m, n, k, a, b, F32, F32, F32, hip.GEMM_F16)
    assert_close(got, ref, 2e-2, "gemm f16 odd sizes")
    got, ref = run_gemm(ta, tb, m, n, k, a, b, F32, F32, F32, hip.GEMM_F32)
    assert_close(got, ref, 1e-5, "gemm fp32 odd sizes")


def test_gemm_bias_alpha_accumulate_batched():
    rng = np.random.default_rng(2)
    m, n, k, batch = 96, 80, 64, 5
    a, b = operands(rng, 0, 1, m, n, k, batch)
    bias = rng.standard_normal(n).astype(np.float32)
    c0 = rng.standard_normal((batch, m, n)).astype(np.float32)
    for compute, tol in ((hip.GEMM_F16, 2e-2), (hip.GEMM_F32, 1e-5)):
        got, ref = run_gemm(0, 1, m, n, k, a, b, F32, F32, F32, compute, alpha=0.25, bias=bias, c0=c0, batch=batch)
        assert_close(got, ref, tol, "alpha/bias/accumulate/batch compute=%d" % compute)


def test_gemm_bf16():
    rng = np.random.default_rng(3)
    m, n, k = 192, 160, 96
    for ta, tb in ((0, 1), (1, 0)):
        a, b = operands(rng, ta, tb, m, n, k)
        got, ref = run_gemm(ta, tb, m, n, k, a, b, BF16, F32, BF16, hip.GEMM_BF16)
        assert_close(got, ref, 2e-2, "gemm bf16")


def test_gemm_fp32_kernel_is_fp32_faithful_at_block_sizes():
    rng = np.random.default_rng(4)
    m, n, k = 512, 1024, 4096
    a, b = operands(rng, 0, 1, m, n, k)
    got, ref = run_gemm(0, 1, m, n, k, a, b, F32, F32, F32, hip.GEMM_F32)
    assert_close(got, ref, 1e-5, "fp32 gemm, k=4096")


def test_gemm_rejects_bad_arguments():
    lib = hip.load()
    t = empty(64)
    args = lambda **kw: None
    assert lib.br_hip_gemm(0, 1, 8, 8, 8, 1.0, ptr(t), F32, 4, 0, ptr(t), F32, 8, 0, 0, ptr(t), F32, 8, 0, None, 1,
                           hip.GEMM_F16, stream()) == -4          # lda < k
    assert lib.br_hip_gemm(0, 1, 8, 8, 8, 1.0, ptr(t), F16, 8, 0, ptr(t), F32, 8, 0, 0, ptr(t), F32, 8, 0, None, 1,
                           hip.GEMM_BF16, stream()) == -1         # fp16 storage with bf16 compute
    assert lib.br_hip_gemm(0, 1, 8, 8, 8, 1.0, ptr(t), F32, 8, 0, ptr(t), F32, 8, 0, 0, None, F32, 8, 0, None, 1,
                           hip.GEMM_F16, stream()) == -3
    torch.cuda.synchronize()
