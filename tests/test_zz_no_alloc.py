"""br_hip_layernorm_bwd_static, the entry point that allocates nothing: same
kernels as br_hip_layernorm_bwd with the partial sums in a buffer built into
the library, so every output must equal the workspace entry's bit for bit --
on two calls in a row, the second on a smaller input (the buffer keeps the
first call's contents), and sizes beyond the buffer are refused."""
import numpy as np
import pytest
import torch

import oracle as orc
from conftest import assert_close
from gpu_util import call, dev, empty, host, ptr, stream, workspace
from blackriver_amd import hip

pytestmark = pytest.mark.gpu


def both_entries(rows, cols, seed, param_scale=1.0, eps=1e-5):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(cols)).astype(np.float32)
    b = (0.1 * rng.standard_normal(cols)).astype(np.float32)
    dy = rng.standard_normal((rows, cols)).astype(np.float32)
    y, _, var = orc.layernorm_fwd(x.reshape(1, rows, cols), g, b, eps)
    y, var = y.reshape(rows, cols), var.reshape(rows)
    t = [dev(a) for a in (dy, y, g, b, var)]
    lib = hip.load()
    ws = workspace(lib.br_hip_layernorm_bwd_workspace(rows, cols))
    dg0, db0, dx0 = empty(cols), empty(cols), empty((rows, cols))
    call("br_hip_layernorm_bwd", ptr(t[0]), ptr(t[1]), ptr(t[2]), ptr(t[3]), ptr(t[4]), ptr(dg0), ptr(db0), ptr(dx0),
         rows, cols, eps, param_scale, ptr(ws), ws.numel(), stream())
    dg1, db1, dx1 = empty(cols), empty(cols), empty((rows, cols))
    for o in (dg1, db1, dx1):
        o.fill_(float("nan"))
    # One warm call first (the first call on a device looks the buffer's address up and loads the kernels), then
    # the device's free memory as the driver reports it (hipMemGetInfo: it sees an allocation made by anyone in the
    # process, inside the library or by the runtime for a kernel's private segment, not only the test's own pool)
    # must be the same before and after a call.
    call("br_hip_layernorm_bwd_static", ptr(t[0]), ptr(t[1]), ptr(t[2]), ptr(t[3]), ptr(t[4]), ptr(dg1), ptr(db1),
         ptr(dx1), rows, cols, eps, param_scale, stream())
    for o in (dg1, db1, dx1):
        o.fill_(float("nan"))
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    call("br_hip_layernorm_bwd_static", ptr(t[0]), ptr(t[1]), ptr(t[2]), ptr(t[3]), ptr(t[4]), ptr(dg1), ptr(db1),
         ptr(dx1), rows, cols, eps, param_scale, stream())
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, "device memory changed by %d bytes across the call" % (free_before - free_after)
    got = host(dx1), host(dg1), host(db1)
    want = host(dx0), host(dg0), host(db0)
    for a, w, name in zip(got, want, ("dx", "dgamma", "dbeta")):
        assert np.array_equal(a, w), (rows, cols, name)
    # and the pair is right, not merely equal: against the oracle
    dx_ref, dg_ref, db_ref = orc.layernorm_bwd(dy.reshape(1, rows, cols), y.reshape(1, rows, cols), g, b, var, eps)
    assert_close(got[0], dx_ref.reshape(rows, cols), 1e-5, "dx")
    assert_close(got[1], dg_ref * param_scale, 1e-5, "dgamma")
    assert_close(got[2], db_ref * param_scale, 1e-5, "dbeta")


def test_static_entry_equals_the_workspace_entry_twice_in_a_row():
    print("case rows=2048 cols=8192, then rows=300 cols=1024", flush=True)
    both_entries(2048, 8192, seed=41)                      # fills the whole 16 MiB buffer
    both_entries(300, 1024, seed=42, param_scale=0.25)     # smaller: stale partials beyond its own must not matter
    both_entries(7, 1001, seed=43)                         # the general kernels (width not a multiple of 4)


def test_static_entry_refuses_what_does_not_fit():
    lib = hip.load()
    assert lib.br_hip_layernorm_bwd_static_limit() == 16 << 20
    t = empty(16)
    rc = lib.br_hip_layernorm_bwd_static(ptr(t), ptr(t), ptr(t), ptr(t), ptr(t), ptr(t), ptr(t), ptr(t), 2048, 16384, 1e-5,
                                         1.0, stream())
    assert rc == -5
    assert b"scratch" in lib.br_hip_error_string(rc)
    torch.cuda.synchronize()
