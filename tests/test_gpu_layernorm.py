"""LayerNorm forward / backward HIP kernels against the CPU oracle, through
the C ABI.  Tolerance: 1e-5 relative (see conftest.assert_close), the bound
stated for fp32 operators."""
import numpy as np
import pytest
import torch

import oracle as orc
from conftest import assert_close
from gpu_util import BF16, F16, F32, call, dev, empty, host, ptr, stream, workspace
from blackriver_amd import hip

pytestmark = pytest.mark.gpu

RTOL = 1e-5


def run_fwd(x, g, b, eps, offset=0):
    rows, cols = x.shape
    if offset:   # place x at an address that is not 16-byte aligned
        buf = empty(x.size + offset)
        buf[offset:] = dev(x).flatten()
        dx_ = buf[offset:]
    else:
        dx_ = dev(x)
    y, mean, var = empty((rows, cols)), empty(rows), empty(rows)
    dg, db = dev(g), dev(b)
    call("br_hip_layernorm_fwd", ptr(dx_), ptr(dg), ptr(db), ptr(y), ptr(mean), ptr(var), rows, cols, eps, stream())
    return host(y), host(mean), host(var)


def run_bwd(dy, y, g, b, var, eps, param_scale=1.0):
    rows, cols = dy.shape
    dgam, dbet, dx = empty(cols), empty(cols), empty((rows, cols))
    ws = workspace(hip.load().br_hip_layernorm_bwd_workspace(rows, cols))
    t = [dev(a) for a in (dy, y, g, b, var)]
    call("br_hip_layernorm_bwd", ptr(t[0]), ptr(t[1]), ptr(t[2]), ptr(t[3]), ptr(t[4]), ptr(dgam), ptr(dbet),
         ptr(dx), rows, cols, eps, param_scale, ptr(ws), ws.numel(), stream())
    return host(dx), host(dgam), host(dbet)


def make(rows, cols, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    g = (1 + 0.02 * rng.standard_normal(cols)).astype(np.float32)
    b = (0.02 * rng.standard_normal(cols)).astype(np.float32)
    dy = rng.standard_normal((rows, cols)).astype(np.float32)
    return x, g, b, dy


@pytest.mark.parametrize("rows,cols", [
    (2048, 4096),    # the headline configuration
    (1, 4096), (3, 64), (37, 1024), (5, 8192), (7, 1000), (9, 1001), (4, 12), (2, 20000),
])
def test_layernorm_fwd_bwd_against_oracle(rows, cols):
    print("case rows=%d cols=%d" % (rows, cols), flush=True)
    x, g, b, dy = make(rows, cols, seed=0)
    eps = 1e-5
    y_ref, mean_ref, var_ref = orc.layernorm_fwd(x, g, b, eps)
    y, mean, var = run_fwd(x, g, b, eps)
    assert_close(y, y_ref, RTOL, "y")
    assert_close(mean, mean_ref, RTOL, "mean")
    assert_close(var, var_ref, RTOL, "var (sigma^2 + eps)")
    # backward consumes the forward's own output and statistic, like the scripts do
    dx_ref, dg_ref, db_ref = orc.layernorm_bwd(dy, y_ref, g, b, var_ref, eps)
    dx, dg, db = run_bwd(dy, y_ref, g, b, var_ref, eps)
    assert_close(dx, dx_ref, RTOL, "dx")
    assert_close(dg, dg_ref, RTOL, "dgamma")
    assert_close(db, db_ref, RTOL, "dbeta")


def test_layernorm_unaligned_input_and_large_mean():
    x, g, b, _ = make(6, 512, seed=1)
    x = x * 0.1 + 50.0       # variance tiny next to the mean: needs the centred form
    y_ref, _, var_ref = orc.layernorm_fwd(x, g, b, 1e-5)
    y, _, var = run_fwd(x, g, b, 1e-5, offset=1)
    assert_close(y, y_ref, 1e-4, "y, mean 50 / std 0.1")     # x itself carries 2^-24 * 50 / 0.1 of noise
    assert_close(var, var_ref, 1e-4, "var")


def test_layernorm_bwd_overwrites_grads_and_handles_tiny_gamma():
    x, g, b, dy = make(16, 256, seed=2)
    g[3], g[4] = 1e-7, -1e-7
    eps = 1e-5
    y_ref, _, var_ref = orc.layernorm_fwd(x, g, b, eps)
    dx_ref, dg_ref, db_ref = orc.layernorm_bwd(dy, y_ref, g, b, var_ref, eps)
    dx, dg, db = run_bwd(dy, y_ref, g, b, var_ref, eps)
    assert_close(dx, dx_ref, RTOL, "dx")
    assert_close(dg, dg_ref, RTOL, "dgamma with |gamma| < eps")
    assert_close(db, db_ref, RTOL, "dbeta")


def test_layernorm_rejects_bad_arguments():
    lib = hip.load()
    t = empty(16)
    assert lib.br_hip_layernorm_fwd(None, ptr(t), ptr(t), ptr(t), None, None, 1, 16, 1e-5, stream()) == -2
    assert lib.br_hip_layernorm_fwd(ptr(t), ptr(t), ptr(t), None, None, None, 1, 16, 1e-5, stream()) == -3
    assert lib.br_hip_layernorm_fwd(ptr(t), ptr(t), ptr(t), ptr(t), None, None, 1, 0, 1e-5, stream()) == -4
    assert lib.br_hip_layernorm_bwd(ptr(t), ptr(t), ptr(t), ptr(t), ptr(t), ptr(t), ptr(t), ptr(t), 1, 16, 1e-5,
                                    1.0, None, 0, stream()) == -4
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype,tdtype", [(F16, torch.float16), (BF16, torch.bfloat16)])
@pytest.mark.parametrize("rows,cols", [(2048, 4096), (3, 64), (5, 8192), (9, 1000)])
def test_layernorm_fwd_with_16_bit_copy(rows, cols, dtype, tdtype):
    """The forward that also writes a 16-bit image of y: y, mean and var are
    bit for bit the plain forward's, and the image is bit for bit the cast of
    y (so scripts may use either form)."""
    print("case rows=%d cols=%d dtype=%d" % (rows, cols, dtype), flush=True)
    x, g, b, _ = make(rows, cols, seed=3)
    eps = 1e-5
    y_plain, mean_plain, var_plain = run_fwd(x, g, b, eps)
    y, mean, var = empty((rows, cols)), empty(rows), empty(rows)
    y16 = empty((rows, cols), tdtype)
    call("br_hip_layernorm_fwd_copy16", ptr(dev(x)), ptr(dev(g)), ptr(dev(b)), ptr(y), ptr(y16), dtype, ptr(mean),
         ptr(var), rows, cols, eps, stream())
    assert np.array_equal(host(y), y_plain)
    assert np.array_equal(host(mean), mean_plain) and np.array_equal(host(var), var_plain)
    cast = empty((rows, cols), tdtype)
    call("br_hip_cast", ptr(y), F32, ptr(cast), dtype, rows * cols, stream())
    assert torch.equal(y16.view(torch.int16), cast.view(torch.int16))
    assert torch.equal(y16, y.to(tdtype))   # round to nearest even of the fp32 output


def test_layernorm_fwd_with_16_bit_copy_declines_what_the_row_kernel_cannot_do():
    lib = hip.load()
    rows, cols = 4, 1001   # not a multiple of 4: general kernel, no copy
    t = empty(rows * cols)
    g = empty(cols)
    h = empty(rows * cols, torch.float16)
    assert lib.br_hip_layernorm_fwd_copy16(ptr(t), ptr(g), ptr(g), ptr(t), ptr(h), F16, None, None, rows, cols, 1e-5,
                                           stream()) == -1
    assert lib.br_hip_layernorm_fwd_copy16(ptr(t), ptr(g), ptr(g), ptr(t), ptr(h), F32, None, None, rows, 1000, 1e-5,
                                           stream()) == -1
    assert lib.br_hip_layernorm_fwd_copy16(ptr(t), ptr(g), ptr(g), ptr(t), None, F16, None, None, rows, 1000, 1e-5,
                                           stream()) == -3
    torch.cuda.synchronize()


@pytest.mark.parametrize("rows,cols", [(2048, 4096), (37, 1024), (5, 8192)])
def test_layernorm_bwd_with_residual_equals_backward_then_add(rows, cols):
    """dx = layernorm_backward(...) + residual in one pass: bit for bit the
    plain backward followed by an fp32 add, also when dx is written over the
    residual or over dy; dgamma / dbeta are unchanged."""
    print("case rows=%d cols=%d" % (rows, cols), flush=True)
    x, g, b, dy = make(rows, cols, seed=5)
    res = np.random.default_rng(6).standard_normal((rows, cols)).astype(np.float32)
    eps = 1e-5
    y_ref, _, var_ref = orc.layernorm_fwd(x, g, b, eps)
    dx_plain, dg_plain, db_plain = run_bwd(dy, y_ref, g, b, var_ref, eps)
    want = dx_plain + res
    ws = workspace(hip.load().br_hip_layernorm_bwd_workspace(rows, cols))
    for alias in ("none", "residual", "dy"):
        t_dy, t_y, t_g, t_b, t_var, t_res = (dev(a) for a in (dy, y_ref, g, b, var_ref, res))
        dgam, dbet = empty(cols), empty(cols)
        out = {"none": empty((rows, cols)), "residual": t_res, "dy": t_dy}[alias]
        call("br_hip_layernorm_bwd_residual", ptr(t_dy), ptr(t_y), ptr(t_g), ptr(t_b), ptr(t_var), ptr(t_res),
             ptr(dgam), ptr(dbet), ptr(out), rows, cols, eps, 1.0, ptr(ws), ws.numel(), stream())
        assert np.array_equal(host(out), want), alias
        assert np.array_equal(host(dgam), dg_plain) and np.array_equal(host(dbet), db_plain), alias
    # shapes the row kernel cannot take are declined
    t = empty(4 * 1001)
    gg = empty(1001)
    assert hip.load().br_hip_layernorm_bwd_residual(ptr(t), ptr(t), ptr(gg), ptr(gg), ptr(gg), ptr(t), ptr(gg), ptr(gg),
                                                    ptr(t), 4, 1001, eps, 1.0, ptr(ws), ws.numel(), stream()) == -1
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype,tdtype", [(F16, torch.float16), (BF16, torch.bfloat16)])
@pytest.mark.parametrize("rows,cols", [(2048, 4096), (512, 4096), (37, 1024), (3, 256)])
def test_layernorm_bwd_with_residual_sums_and_16_bit_copy(rows, cols, dtype, tdtype):
    """The backward + residual that also leaves the 16-bit image and the column sums of its result (the first pass
    of the linear backward below it): dx, dgamma, dbeta bit for bit those of br_hip_layernorm_bwd_residual, the
    image bit for bit dx rounded once, the sums (times param_scale) against a float64 sum of dx as stored --
    through the lifted-gradient factor too."""
    print("case rows=%d cols=%d dtype=%d" % (rows, cols, dtype), flush=True)
    x, g, b, dy = make(rows, cols, seed=7)
    res = np.random.default_rng(8).standard_normal((rows, cols)).astype(np.float32)
    eps = 1e-5
    y_ref, _, var_ref = orc.layernorm_fwd(x, g, b, eps)
    lib = hip.load()
    ws = workspace(lib.br_hip_layernorm_bwd_sums_workspace(rows, cols))
    assert lib.br_hip_layernorm_bwd_sums_workspace(rows, cols) >= lib.br_hip_layernorm_bwd_workspace(rows, cols)
    for scale in (1.0, 1.0 / 1024):
        t_dy, t_y, t_g, t_b, t_var, t_res = (dev(a) for a in (dy, y_ref, g, b, var_ref, res))
        dgam, dbet, dx = empty(cols), empty(cols), empty((rows, cols))
        call("br_hip_layernorm_bwd_residual", ptr(t_dy), ptr(t_y), ptr(t_g), ptr(t_b), ptr(t_var), ptr(t_res),
             ptr(dgam), ptr(dbet), ptr(dx), rows, cols, eps, scale, ptr(ws), ws.numel(), stream())
        dgam2, dbet2, dx2, sums = empty(cols), empty(cols), empty((rows, cols)), empty(cols)
        dx16 = torch.zeros((rows, cols), dtype=tdtype, device="cuda")
        call("br_hip_layernorm_bwd_residual_sums", ptr(t_dy), ptr(t_y), ptr(t_g), ptr(t_b), ptr(t_var), ptr(t_res),
             ptr(dgam2), ptr(dbet2), ptr(dx2), ptr(dx16), dtype, ptr(sums), rows, cols, eps, scale, ptr(ws), ws.numel(),
             stream())
        assert torch.equal(dx2, dx) and torch.equal(dgam2, dgam) and torch.equal(dbet2, dbet)
        assert torch.equal(dx16, dx.to(tdtype))
        want = host(dx).astype(np.float64).sum(0) * scale
        # fp32 sums in a fixed tree: a few ulps of the sum of magnitudes
        bound = 1e-6 * np.abs(host(dx)).astype(np.float64).sum(0) * scale + 1e-30
        assert np.all(np.abs(host(sums) - want) <= bound), float((np.abs(host(sums) - want) / bound).max())
    # declined: rows wider than 4096 columns, a misaligned sums pointer; missing outputs are an error
    t = empty(2 * 8192)
    gg = empty(8192 + 4)
    h = torch.zeros(2 * 8192, dtype=tdtype, device="cuda")
    ws2 = workspace(lib.br_hip_layernorm_bwd_sums_workspace(2, 8192))
    args = lambda sums_ptr, h_ptr, c: (ptr(t), ptr(t), ptr(gg), ptr(gg), ptr(gg), ptr(t), ptr(gg), ptr(gg), ptr(t), h_ptr,
                                       dtype, sums_ptr, 2, c, eps, 1.0, ptr(ws2), ws2.numel(), stream())
    assert lib.br_hip_layernorm_bwd_residual_sums(*args(ptr(gg), ptr(h), 8192)) == -1
    import ctypes
    assert lib.br_hip_layernorm_bwd_residual_sums(*args(ctypes.c_void_p(gg.data_ptr() + 4), ptr(h), 4096)) == -1
    assert lib.br_hip_layernorm_bwd_residual_sums(*args(None, ptr(h), 4096)) == -3
    assert lib.br_hip_layernorm_bwd_residual_sums(*args(ptr(gg), None, 4096)) == -3
    torch.cuda.synchronize()


def test_layernorm_bwd_param_scale_is_an_exact_power_of_two_factor():
    """dy lifted by S = 1024 with param_scale = 1/S: dx comes out S times the
    plain one and dgamma / dbeta equal the plain ones, all bit for bit (scaling
    by a power of two commutes with every rounding on the way)."""
    rng = np.random.default_rng(31)
    rows, cols, eps = 96, 1024, 1e-5
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(cols)).astype(np.float32)
    b = (0.1 * rng.standard_normal(cols)).astype(np.float32)
    dy = rng.standard_normal((rows, cols)).astype(np.float32)
    y, _, var = run_fwd(x, g, b, eps)
    dx, dg, db = run_bwd(dy, y, g, b, var, eps)
    dx2, dg2, db2 = run_bwd(dy * np.float32(1024), y, g, b, var, eps, param_scale=1.0 / 1024)
    assert np.array_equal(dx2, dx * np.float32(1024))
    assert np.array_equal(dg2, dg) and np.array_equal(db2, db)
