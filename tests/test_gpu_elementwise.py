"""Elementwise / data-movement HIP kernels against the CPU oracle through the
C ABI: GELU and bias-GELU (fp32 and fp16 storage), broadcast add, transpose,
column sums, casts and the bit-exact data-preparation tables."""
import ctypes

import numpy as np
import pytest
import torch

import oracle as orc
from conftest import assert_close
from gpu_util import (BF16, F16, F32, I32, assert_close_f16, call, dev, empty, host, ptr, stream, workspace)
from blackriver_amd import hip

pytestmark = pytest.mark.gpu
RTOL = 1e-5
FLT_MAX = np.finfo(np.float32).max


# ------------------------------------------------------------------- GELU
@pytest.mark.parametrize("n", [8 * 1000, 1000003, 5])
def test_gelu_f32_fwd_bwd(n):
    rng = np.random.default_rng(0)
    x = (1.5 * rng.standard_normal(n)).astype(np.float32)
    x[:4] = [-12.0, 12.0, 0.0, -30.0][: min(4, n)]
    dy = rng.standard_normal(n).astype(np.float32)
    dx_, dy_ = dev(x), dev(dy)
    y, g = empty(n), empty(n)
    call("br_hip_gelu_fwd", ptr(dx_), ptr(y), F32, n, stream())
    call("br_hip_gelu_bwd", ptr(dy_), ptr(dx_), ptr(g), F32, n, stream())
    assert_close(host(y), orc.gelu_fwd(x), RTOL, "gelu fwd")
    assert_close(host(g), orc.gelu_bwd(dy, x), RTOL, "gelu bwd")
    # in place on x, the aliasing the scripts use (train.words:200)
    call("br_hip_gelu_bwd", ptr(dy_), ptr(dx_), ptr(dx_), F32, n, stream())
    assert np.array_equal(host(dx_), host(g))


def test_bias_gelu_f16_headline_shape():
    """x[2048,16384] fp16 ~N(0,1.5), bias ~N(0,0.02), dy ~N(0,1), seed 1."""
    rng = np.random.default_rng(1)
    rows, cols = 2048, 16384
    x = (1.5 * rng.standard_normal((rows, cols))).astype(np.float16)
    bias = (0.02 * rng.standard_normal(cols)).astype(np.float32)
    dy = rng.standard_normal((rows, cols)).astype(np.float16)
    dx_, db_, dy_ = dev(x), dev(bias), dev(dy)
    y = empty((rows, cols), torch.float16)
    g = empty((rows, cols), torch.float16)
    dbias = empty(cols)
    call("br_hip_bias_gelu_fwd", ptr(dx_), ptr(db_), ptr(y), F16, rows, cols, stream())
    ws = workspace(hip.load().br_hip_bias_gelu_bwd_workspace(rows, cols))
    call("br_hip_bias_gelu_bwd", ptr(dy_), ptr(dx_), ptr(db_), ptr(g), ptr(dbias), F16, rows, cols, 1.0, ptr(ws),
         ws.numel(), stream())
    x32, dy32 = x.astype(np.float32), dy.astype(np.float32)
    assert_close_f16(host(y), orc.bias_gelu_fwd(x32, bias), RTOL, "bias gelu fwd (fp16 storage)")
    g_ref, _ = orc.bias_gelu_bwd(dy32, x32, bias)
    got_g = host(g)
    assert_close_f16(got_g, g_ref, RTOL, "bias gelu bwd (fp16 storage)")
    # dbias sums what was stored (the fp16-rounded dx)
    assert_close(host(dbias), got_g.astype(np.float64).sum(0), RTOL, "dbias")


@pytest.mark.parametrize("rows,cols,dtype", [(33, 1024, "f32"), (7, 100, "f32"), (5, 24, "f16"), (9, 31, "f16"),
                                             (130, 6152, "f16"), (300, 3080, "f32"), (512, 16384, "f16")])
def test_bias_gelu_small_and_unaligned(rows, cols, dtype):
    rng = np.random.default_rng(2)
    np_t, code, t_t = (np.float32, F32, torch.float32) if dtype == "f32" else (np.float16, F16, torch.float16)
    x = (1.5 * rng.standard_normal((rows, cols))).astype(np_t)
    bias = rng.standard_normal(cols).astype(np.float32)
    dy = rng.standard_normal((rows, cols)).astype(np_t)
    dx_, db_, dy_ = dev(x), dev(bias), dev(dy)
    y, g, dbias = empty((rows, cols), t_t), empty((rows, cols), t_t), empty(cols)
    call("br_hip_bias_gelu_fwd", ptr(dx_), ptr(db_), ptr(y), code, rows, cols, stream())
    ws = workspace(hip.load().br_hip_bias_gelu_bwd_workspace(rows, cols))
    call("br_hip_bias_gelu_bwd", ptr(dy_), ptr(dx_), ptr(db_), ptr(g), ptr(dbias), code, rows, cols, 1.0, ptr(ws),
         ws.numel(), stream())
    y_ref = orc.bias_gelu_fwd(x.astype(np.float32), bias)
    g_ref, dbias_ref = orc.bias_gelu_bwd(dy.astype(np.float32), x.astype(np.float32), bias)
    if dtype == "f32":
        assert_close(host(y), y_ref, RTOL, "fwd")
        assert_close(host(g), g_ref, RTOL, "bwd")
        assert_close(host(dbias), dbias_ref, RTOL, "dbias")
    else:
        assert_close_f16(host(y), y_ref, RTOL, "fwd")
        assert_close_f16(host(g), g_ref, RTOL, "bwd")
        assert_close(host(dbias), host(g).astype(np.float64).sum(0), RTOL, "dbias")


# ---------------------------------------------------------- broadcast add
@pytest.mark.parametrize("ashape,bshape", [
    ((4, 32, 128, 128), (1, 32, 1, 128)),   # alibi
    ((4, 32, 128, 128), (4, 1, 128, 128)),  # xmask
    ((2, 512, 4096), (2, 512, 4096)),       # residual
    ((2, 3, 5, 7), (1, 3, 1, 7)), ((2, 3, 5, 7), (2, 1, 5, 7)), ((6, 10), (1, 10)), ((2, 3, 4, 8), (2, 3, 4, 1)),
])
def test_add_bcast_bit_exact(ashape, bshape):
    rng = np.random.default_rng(3)
    a = rng.standard_normal(ashape).astype(np.float32)
    b = rng.standard_normal(bshape).astype(np.float32)
    if bshape[-1] == ashape[-1] and len(bshape) == 4 and bshape[1] == 1:
        b[b > 1.0] = -FLT_MAX          # behave like the additive mask
    da, db_ = dev(a), dev(b)
    c = empty(ashape)
    call("br_hip_add_bcast", ptr(da), ptr(db_), ptr(c), F32, hip.shape4(ashape), hip.shape4(bshape), stream())
    ref = orc.add_bcast(a, b)
    assert np.array_equal(host(c), ref)
    # c aliasing a (train.words:158)
    call("br_hip_add_bcast", ptr(da), ptr(db_), ptr(da), F32, hip.shape4(ashape), hip.shape4(bshape), stream())
    assert np.array_equal(host(da), ref)


def test_add_f16_same_shape():
    rng = np.random.default_rng(4)
    a = rng.standard_normal((3, 40, 64)).astype(np.float16)
    b = rng.standard_normal((3, 40, 64)).astype(np.float16)
    c = empty(a.shape, torch.float16)
    da, db_ = dev(a), dev(b)          # keep the operands alive until the kernel has run
    call("br_hip_add_bcast", ptr(da), ptr(db_), ptr(c), F16, hip.shape4(a.shape), hip.shape4(b.shape), stream())
    assert np.array_equal(host(c), (a.astype(np.float32) + b.astype(np.float32)).astype(np.float16))


# ----------------------------------------------------- transpose / colsum
@pytest.mark.parametrize("shape,eb", [((4, 512, 32, 128), 4), ((2, 7, 3, 5), 4), ((2, 16, 4, 8), 2), ((1, 3, 5, 3), 2)])
def test_transpose_0213_bit_exact(shape, eb):
    rng = np.random.default_rng(5)
    x = rng.standard_normal(shape).astype(np.float32 if eb == 4 else np.float16)
    y = empty((shape[0], shape[2], shape[1], shape[3]), torch.float32 if eb == 4 else torch.float16)
    call("br_hip_transpose_0213", ptr(dev(x)), ptr(y), eb, *shape, stream())
    assert np.array_equal(host(y), np.ascontiguousarray(x.transpose(0, 2, 1, 3)))


@pytest.mark.parametrize("rows,cols", [(2048, 4096), (77, 130), (1, 8), (512, 4096), (1000, 3080)])
def test_colsum(rows, cols):
    rng = np.random.default_rng(6)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    out = empty(cols)
    ws = workspace(hip.load().br_hip_colsum_workspace(rows, cols))
    call("br_hip_colsum", ptr(dev(x)), F32, ptr(out), rows, cols, 1.0, ptr(ws), ws.numel(), stream())
    assert_close(host(out), x.astype(np.float64).sum(0), RTOL, "colsum")


@pytest.mark.parametrize("rows,cols,dtype", [(2048, 12288, "f16"), (130, 6152, "f16"), (513, 16384, "bf16"),
                                             (77, 6144, "bf16"), (1, 6144, "f16"), (40, 1024, "f16")])
def test_colsum_16_bit(rows, cols, dtype):
    """Column sums of 16-bit tensors (the bias gradient of a linear layer whose
    output gradient is kept in 16 bits): shapes wide enough for the
    single-launch form (a workgroup per 64 columns walking all rows; ragged
    last block, rows that do not fill a pass) and one that takes two launches."""
    from gpu_util import BF16
    rng = np.random.default_rng(61)
    t, code = (torch.float16, F16) if dtype == "f16" else (torch.bfloat16, BF16)
    x = torch.from_numpy(rng.standard_normal((rows, cols)).astype(np.float32)).cuda().to(t)
    out = empty(cols)
    ws = workspace(hip.load().br_hip_colsum_workspace(rows, cols))
    call("br_hip_colsum", ptr(x), code, ptr(out), rows, cols, 0.5, ptr(ws), ws.numel(), stream())
    assert_close(host(out), 0.5 * x.float().cpu().numpy().astype(np.float64).sum(0), RTOL, "colsum " + dtype)


@pytest.mark.parametrize("rows,cols", [(2048, 4096), (300, 1000), (5, 8), (1, 4), (512, 4096), (300, 3080), (1, 3072)])
def test_colsum_cast_equals_colsum_plus_cast(rows, cols):
    """One pass giving the column sums and the fp16 copy: the sums must equal
    br_hip_colsum's bit for bit (same strips, same order), the copy the cast's."""
    rng = np.random.default_rng(8)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    dx = dev(x)
    ws = workspace(hip.load().br_hip_colsum_workspace(rows, cols))
    sums, sums2, h = empty(cols), empty(cols), empty((rows, cols), torch.float16)
    call("br_hip_colsum", ptr(dx), F32, ptr(sums), rows, cols, 1.0, ptr(ws), ws.numel(), stream())
    call("br_hip_colsum_cast", ptr(dx), ptr(sums2), ptr(h), F16, rows, cols, 1.0, ptr(ws), ws.numel(), stream())
    assert np.array_equal(host(sums2), host(sums))
    assert np.array_equal(host(h).view(np.uint16), x.astype(np.float16).view(np.uint16))
    assert_close(host(sums2), x.astype(np.float64).sum(0), RTOL, "colsum")


def test_gelu_fwd_f32_to_16_rounds_the_fp32_result_once():
    from gpu_util import BF16
    rng = np.random.default_rng(9)
    n = 8 * 4099
    x = (2.0 * rng.standard_normal(n)).astype(np.float32)
    dx = dev(x)
    y32, y16, yb = empty(n), empty(n, torch.float16), empty(n, torch.bfloat16)
    call("br_hip_gelu_fwd", ptr(dx), ptr(y32), F32, n, stream())
    call("br_hip_gelu_fwd_f32_to_16", ptr(dx), ptr(y16), F16, n, stream())
    call("br_hip_gelu_fwd_f32_to_16", ptr(dx), ptr(yb), BF16, n, stream())
    assert np.array_equal(host(y16).view(np.uint16), host(y32).astype(np.float16).view(np.uint16))
    torch.cuda.synchronize()
    assert torch.equal(yb, y32.to(torch.bfloat16))
    lib = hip.load()
    assert lib.br_hip_gelu_fwd_f32_to_16(ptr(dx), ptr(y16), F16, 12, stream()) == -1   # n % 8 != 0: not this entry's job
    assert lib.br_hip_gelu_fwd_f32_to_16(ptr(dx), ptr(y16), F32, 16, stream()) == -1
    assert lib.br_hip_gelu_fwd_f32_to_16(ptr(dx), ptr(y16), F16, 0, stream()) == 0
    torch.cuda.synchronize()


def test_normal_fill_is_a_function_of_seed_and_index():
    n = 1 << 20
    a, b, c = empty(n), empty(n), empty(n)
    h = empty(n, torch.float16)
    call("br_hip_normal", ptr(a), F32, 1.0, 0.5, 7, n, stream())
    call("br_hip_normal", ptr(b), F32, 1.0, 0.5, 7, n, stream())
    call("br_hip_normal", ptr(c), F32, 1.0, 0.5, 8, n, stream())
    call("br_hip_normal", ptr(h), F16, 1.0, 0.5, 7, n, stream())
    va, vb, vc = host(a).astype(np.float64), host(b), host(c)
    assert np.array_equal(host(a), vb) and not np.array_equal(host(a), vc)
    assert np.array_equal(host(h).view(np.uint16), host(a).astype(np.float16).view(np.uint16))
    # a prefix is the same whatever the length (value depends on the index only)
    short = empty(1000)
    call("br_hip_normal", ptr(short), F32, 1.0, 0.5, 7, 1000, stream())
    assert np.array_equal(host(short), host(a)[:1000])
    z = (va - 1.0) / 0.5
    assert abs(z.mean()) < 5e-3 and abs(z.std() - 1.0) < 5e-3
    assert abs((z ** 3).mean()) < 2e-2 and abs((z ** 4).mean() - 3.0) < 5e-2      # skewness 0, kurtosis 3
    assert abs(np.corrcoef(z[:-1], z[1:])[0, 1]) < 5e-3                            # neighbours uncorrelated
    assert np.all(np.isfinite(va))


def test_fill_and_cast_roundtrip():
    n = 100003
    t = empty(n)
    call("br_hip_fill", ptr(t), F32, 2.5, n, stream())
    assert np.all(host(t) == 2.5)
    rng = np.random.default_rng(7)
    x = (rng.standard_normal(n) * 10.0 ** rng.integers(-6, 5, n)).astype(np.float32)
    h = empty(n, torch.float16)
    call("br_hip_cast", ptr(dev(x)), F32, ptr(h), F16, n, stream())
    with np.errstate(over="ignore"):
        assert np.array_equal(host(h).view(np.uint16), x.astype(np.float16).view(np.uint16))
    back = empty(n)
    call("br_hip_cast", ptr(h), F16, ptr(back), F32, n, stream())
    assert np.array_equal(host(back), host(h).astype(np.float32))


# ------------------------------------------------ data preparation tables
def test_embedding_gather_bit_exact(fixture_ids_mask):
    ids, _ = fixture_ids_mask
    rng = np.random.default_rng(8)
    vocab, hidden = 4099, 4096
    table = rng.standard_normal((vocab, hidden)).astype(np.float32)
    small = (ids % vocab).astype(np.int32)
    out = empty((2, 512, hidden))
    call("br_hip_embedding_gather", ptr(dev(table)), ptr(dev(small)), ptr(out), 4, small.size, hidden, vocab, stream())
    assert np.array_equal(host(out), orc.embedding_gather(table, small))


@pytest.mark.parametrize("heads,tokens", [(32, 512), (8, 7), (160, 33)])
def test_alibi_table_bit_exact(heads, tokens):
    out = empty((heads, tokens))
    call("br_hip_alibi_table", ptr(out), heads, tokens, stream())
    assert np.array_equal(host(out), orc.alibi(heads, tokens))


def test_xmask_table_bit_exact(fixture_ids_mask):
    _, mask = fixture_ids_mask
    m = mask.copy()
    out = empty((2, 512, 512))
    call("br_hip_xmask_table", ptr(dev(m)), ptr(out), 2, 512, stream())
    assert np.array_equal(host(out), orc.xmask(m))
    holes = np.array([[1, 1, 0, 1, 1], [0, 1, 1, 1, 1], [1, 1, 1, 1, 1]], np.int32)
    out2 = empty((3, 5, 5))
    call("br_hip_xmask_table", ptr(dev(holes)), ptr(out2), 3, 5, stream())
    assert np.array_equal(host(out2), orc.xmask(holes))


@pytest.mark.parametrize("n,hidden,vocab", [(2048, 4096, 512), (37, 100, 11), (64, 256, 1), (5, 8, 1000)])
def test_embedding_scatter_add_is_the_sequential_scatter(n, hidden, vocab):
    """Backward of the embedding gather: bit-exact against the oracle's
    sequential loop (repeated ids are summed in position order), with many
    repeats (vocab < n), a single row taking everything (vocab 1), ids outside
    the table skipped, and a non-zero starting gradient."""
    print("case n=%d hidden=%d vocab=%d" % (n, hidden, vocab), flush=True)
    rng = np.random.default_rng(31)
    ids = rng.integers(0, vocab, n).astype(np.int32)
    if n > 4:
        ids[1], ids[3] = -1, vocab       # outside the table
    dx = rng.standard_normal((n, hidden)).astype(np.float32)
    grad = rng.standard_normal((vocab, hidden)).astype(np.float32)
    want = orc.embedding_scatter_add(grad, dx, ids)
    d_grad = dev(grad)
    call("br_hip_embedding_scatter_add", ptr(dev(dx)), ptr(dev(ids)), ptr(d_grad), n, hidden, vocab, 1.0, stream())
    assert np.array_equal(host(d_grad), want)


@pytest.mark.parametrize("dtype,master", [(F32, False), (F16, True), (F16, False), (BF16, True)])
@pytest.mark.parametrize("n", [4096 * 1024, 1001])
def test_adamw_against_oracle(n, dtype, master):
    """Three AdamW steps against the oracle's fp32 restatement (itself pinned to
    torch.optim.AdamW): parameter / master and both moments within 1e-5; a
    16-bit parameter is exactly the rounding of its master copy."""
    print("case n=%d dtype=%d master=%s" % (n, dtype, master), flush=True)
    rng = np.random.default_rng(17)
    tdt = {F32: torch.float32, F16: torch.float16, BF16: torch.bfloat16}[dtype]
    p0 = torch.from_numpy(rng.standard_normal(n).astype(np.float32)).to(tdt)
    d_p = p0.cuda()
    d_master = p0.float().cuda() if master else None
    d_m, d_v = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    p, m, v = p0.float().numpy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    lr, b1, b2, eps, wd = 1e-2, 0.9, 0.95, 1e-8, 0.1
    for step in range(1, 4):
        g = rng.standard_normal(n).astype(np.float32)
        call("br_hip_adamw", ptr(d_p), dtype, ptr(d_master), ptr(dev(g)), ptr(d_m), ptr(d_v), n, lr, b1, b2, eps, wd,
             step, stream())
        p, m, v = orc.adamw_step(p, g, m, v, lr, b1, b2, eps, wd, step)
        assert_close(host(d_m), m, 1e-5, "first moment, step %d" % step)
        assert_close(host(d_v), v, 1e-5, "second moment, step %d" % step)
        if dtype == F32:
            assert_close(host(d_p), p, 1e-5, "parameter, step %d" % step)
        elif master:
            assert_close(host(d_master), p, 1e-5, "master copy, step %d" % step)
            assert torch.equal(d_p, d_master.to(tdt))
        else:
            # the 16-bit value is the only state: the oracle follows the same rounding
            p = torch.from_numpy(p).to(tdt).float().numpy()
            got = host(d_p.float())
            ulp = np.abs(p) * (2.0 ** -10 if dtype == F16 else 2.0 ** -7)
            assert np.all(np.abs(got - p) <= ulp + 1e-6)
            p = got


def test_adamw_rejects_bad_arguments():
    lib = hip.load()
    t = empty(16)
    args = (16, 1e-3, 0.9, 0.95, 1e-8, 0.0)
    assert lib.br_hip_adamw(ptr(t), F32, ptr(t), ptr(t), ptr(t), ptr(t), *args, 1, stream()) == -4   # fp32 + master
    assert lib.br_hip_adamw(ptr(t), F32, None, ptr(t), ptr(t), ptr(t), *args, 0, stream()) == -4      # step from 1
    assert lib.br_hip_adamw(ptr(t), F32, None, None, ptr(t), ptr(t), *args, 1, stream()) == -2
    assert lib.br_hip_adamw(None, F32, None, ptr(t), ptr(t), ptr(t), *args, 1, stream()) == -3
    assert lib.br_hip_adamw(ptr(t), I32, None, ptr(t), ptr(t), ptr(t), *args, 1, stream()) == -1
    torch.cuda.synchronize()


@pytest.mark.parametrize("offset,nbytes", [(0, 1 << 20), (3, 1000), (5, 7), (16, 4096 + 9), (1, 0)])
def test_memset_fills_exactly_the_requested_bytes(offset, nbytes):
    """br_hip_memset is a fill kernel (16-byte stores over the aligned middle,
    single bytes at the ends): every requested byte is set, none around it."""
    buf = torch.full((nbytes + 64,), 0x11, dtype=torch.uint8, device="cuda")
    call("br_hip_memset", ctypes.c_void_p(buf.data_ptr() + offset), 0xAB, nbytes, stream())
    got = host(buf)
    assert np.all(got[offset:offset + nbytes] == 0xAB)
    assert np.all(got[:offset] == 0x11) and np.all(got[offset + nbytes:] == 0x11)


@pytest.mark.parametrize("dtype,tdtype", [(F16, torch.float16), (BF16, torch.bfloat16)])
@pytest.mark.parametrize("rows,cols", [(2048, 16384), (37, 64), (5, 1000), (512, 16384), (300, 3080)])
def test_gelu_bwd_colsum_cast_equals_the_separate_kernels(rows, cols, dtype, tdtype):
    """One pass producing the GELU gradient, its 16-bit copy and its column
    sums: each bit for bit what br_hip_gelu_bwd followed by br_hip_colsum_cast
    gives, also in place on x."""
    print("case rows=%d cols=%d dtype=%d" % (rows, cols, dtype), flush=True)
    rng = np.random.default_rng(23)
    x = (1.5 * rng.standard_normal((rows, cols))).astype(np.float32)
    dy = rng.standard_normal((rows, cols)).astype(np.float32)
    d_x, d_dy = dev(x), dev(dy)
    n = rows * cols
    dx_sep = empty((rows, cols))
    call("br_hip_gelu_bwd", ptr(d_dy), ptr(d_x), ptr(dx_sep), F32, n, stream())
    ws = workspace(hip.load().br_hip_colsum_workspace(rows, cols))
    sums_sep, x16_sep = empty(cols), empty((rows, cols), tdtype)
    call("br_hip_colsum_cast", ptr(dx_sep), ptr(sums_sep), ptr(x16_sep), dtype, rows, cols, 1.0, ptr(ws), ws.numel(), stream())
    for in_place in (False, True):
        d_u = dev(x)
        dx = d_u if in_place else empty((rows, cols))
        sums, x16 = empty(cols), empty((rows, cols), tdtype)
        call("br_hip_gelu_bwd_colsum_cast", ptr(d_dy), ptr(d_u), ptr(dx), ptr(sums), ptr(x16), dtype, rows, cols,
             1.0, ptr(ws), ws.numel(), stream())
        assert torch.equal(dx, dx_sep), in_place
        assert torch.equal(x16.view(torch.int16), x16_sep.view(torch.int16)), in_place
        assert torch.equal(sums, sums_sep), in_place
    assert hip.load().br_hip_gelu_bwd_colsum_cast(ptr(d_dy), ptr(d_x), ptr(dx_sep), ptr(sums_sep), ptr(x16_sep), dtype,
                                                  4, 1001, 1.0, ptr(ws), ws.numel(), stream()) == -1
    torch.cuda.synchronize()
