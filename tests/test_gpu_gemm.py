"""MFMA GEMM kernel against fp64 products through the C ABI: every operand
layout, storage type and compute type, odd sizes, batching, bias, alpha and
accumulation.  Tolerances: 2e-2 relative for fp16 / bf16 operands, 1e-5 for
the fp32-operand kernel."""
import ctypes

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
    ref = alpha * np.matmul(A, B)
    if bias is not None:
        ref = ref + bias.astype(np.float64)[None, None, :]
    if c0 is not None:
        ref = ref + to_host64(to_dev(c0, c_dt)).reshape(batch, m, n)
    return to_host64(c).reshape(batch, m, n), ref


def run_gemm_staged(ta, tb, m, n, k, a, b, a_dt, b_dt, c_dt, compute, batch=1, ws_bytes=None, bias=None):
    """br_hip_gemm_staged and br_hip_gemm on the same device operands."""
    da, db_ = to_dev(a, a_dt), to_dev(b, b_dt)
    dbias = dev(bias) if bias is not None else None
    lda = m if ta else k
    ldb = k if tb else n
    need = hip.load().br_hip_gemm_staged_workspace(int(ta), int(tb), m, n, k, a_dt, b_dt, batch)
    if ws_bytes is None:
        ws_bytes = need
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
    outs = []
    for staged in (True, False):
        c = torch.full((batch, m, n), float("nan"), dtype=TORCH_T[c_dt], device="cuda")
        common = (int(ta), int(tb), m, n, k, 1.0, ptr(da), a_dt, lda, m * k, ptr(db_), b_dt, ldb, n * k, 0, ptr(c),
                  c_dt, n, m * n, ptr(dbias), batch, compute)
        if staged:
            call("br_hip_gemm_staged", *common, ptr(ws), ws_bytes, stream())
        else:
            call("br_hip_gemm", *common, stream())
        outs.append(to_host64(c).reshape(batch, m, n))
    return outs[0], outs[1], need


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


# Shapes that make the dispatcher pick each direct-to-LDS tile configuration
# (256x256, 256x128, 128x128 with 64-wide K steps; 128x128 with 32-wide steps
# when K % 64 != 0), with rows / columns that do not fill the last tile.
DTL_SHAPES = [
    ("256x256", 512, 512, 128, 64),
    ("256x256 ragged", 488, 520, 192, 64),
    ("256x128", 256, 128, 512, 1),
    ("256x128 ragged", 1000, 1048, 256, 1),
    ("128x128", 128, 51200, 64, 1),
    ("128x128 k32", 264, 392, 96, 3),
    ("one k step", 256, 256, 64, 1),
    ("one k step k32", 256, 256, 32, 1),
]


@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("name,m,n,k,batch", DTL_SHAPES)
def test_gemm_direct_to_lds_kernel(ta, tb, name, m, n, k, batch):
    rng = np.random.default_rng(5)
    print("case %s ta=%d tb=%d m=%d n=%d k=%d batch=%d" % (name, ta, tb, m, n, k, batch), flush=True)
    a, b = operands(rng, ta, tb, m, n, k, batch)
    got, ref = run_gemm(ta, tb, m, n, k, a, b, F16, F16, F32, hip.GEMM_F16, batch=batch)
    assert_close(got, ref, 2e-2, "dtl gemm " + name)
    assert np.sqrt(np.mean((got - ref) ** 2)) < 1e-5 * np.sqrt(np.mean(ref ** 2)) * np.sqrt(k)


def test_gemm_direct_to_lds_epilogue_and_types():
    rng = np.random.default_rng(6)
    m, n, k, batch = 320, 256, 256, 2
    a, b = operands(rng, 0, 1, m, n, k, batch)
    bias = rng.standard_normal(n).astype(np.float32)
    c0 = rng.standard_normal((batch, m, n)).astype(np.float32)
    got, ref = run_gemm(0, 1, m, n, k, a, b, F16, F16, F32, hip.GEMM_F16, alpha=0.5, bias=bias, c0=c0, batch=batch)
    assert_close(got, ref, 2e-2, "dtl alpha/bias/accumulate")
    got, ref = run_gemm(0, 1, m, n, k, a, b, F16, F16, F16, hip.GEMM_F16, bias=bias, batch=batch)
    assert_close(got, ref, 2e-2, "dtl fp16 output")
    for ta, tb in ((0, 1), (0, 0), (1, 0), (1, 1)):
        a, b = operands(rng, ta, tb, m, n, k, batch)
        got, ref = run_gemm(ta, tb, m, n, k, a, b, BF16, BF16, BF16, hip.GEMM_BF16, batch=batch)
        assert_close(got, ref, 2e-2, "dtl bf16")


def test_gemm_direct_to_lds_at_linear_layer_shape():
    """BLOOM-7B1 h -> 4h at a quarter of the token count; checked on a sample
    of rows against fp64 and, for every element, through linearity:
    (A1 + A2) B == A1 B + A2 B up to fp32 accumulation error when the sums are
    exact in fp16."""
    rng = np.random.default_rng(7)
    m, n, k = 512, 16384, 4096
    a1 = rng.integers(-8, 9, (1, m, k)).astype(np.float32)
    a2 = rng.integers(-8, 9, (1, m, k)).astype(np.float32)
    b = rng.integers(-4, 5, (1, n, k)).astype(np.float32)
    c1, _ = run_gemm(0, 1, m, n, k, a1, b, F16, F16, F32, hip.GEMM_F16)
    c2, _ = run_gemm(0, 1, m, n, k, a2, b, F16, F16, F32, hip.GEMM_F16)
    c12, ref = run_gemm(0, 1, m, n, k, a1 + a2, b, F16, F16, F32, hip.GEMM_F16)
    # small integers: every product and partial sum is exact in fp32
    assert np.array_equal(c12, ref)
    assert np.array_equal(c1 + c2, c12)


@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k,c_dt", [
    (2048, 8192, 192, F32),     # 256 tiles: one per workgroup, three K steps
    (2048, 16384, 128, F16),    # 512 tiles: two per workgroup, 16-bit C
    (3072, 16384, 64, F32),     # 768 tiles of a single K step
    (2816, 6144, 320, F32),     # 264 tiles: 33 per XCD for 32 workgroups, one of them walks twice
])
def test_gemm_workgroups_that_walk_the_tiles(ta, tb, m, n, k, c_dt):
    """Plain products (no bias, nothing accumulated) of 256 or more interior
    256 x 256 tiles run on 256 workgroups that each walk several tiles, loading
    the next tile's first K stages ahead of the current tile's stores.  Against
    fp64, and for an fp32 C bit for bit against the same product with a bias of
    zeros, which takes the one-workgroup-per-tile kernel."""
    rng = np.random.default_rng(31)
    print("case ta=%d tb=%d m=%d n=%d k=%d c_dt=%d" % (ta, tb, m, n, k, c_dt), flush=True)
    a, b = operands(rng, ta, tb, m, n, k)
    got, ref = run_gemm(ta, tb, m, n, k, a, b, F16, F16, c_dt, hip.GEMM_F16, alpha=0.5)
    assert_close(got, ref, 2e-2, "walking workgroups")
    per_tile, _ = run_gemm(ta, tb, m, n, k, a, b, F16, F16, c_dt, hip.GEMM_F16, alpha=0.5, bias=np.zeros(n, np.float32))
    assert np.array_equal(got, per_tile)


@pytest.mark.parametrize("k", [512, 2048])
def test_gemm_walking_workgroups_at_the_weight_gradient_shape(k):
    """dW[16384, 4096] = dy[k, 16384]^T . x[k, 4096] (1024 tiles, four per
    workgroup) at both token counts of the benchmarks: bit for bit the
    one-workgroup-per-tile kernel (taken with a bias of zeros), three launches
    in a row on rotating operands, and a sample of rows against fp64."""
    torch.manual_seed(k)
    m, n = 16384, 4096
    sets = [(torch.randn((k, m), device="cuda").half(), torch.randn((k, n), device="cuda").half()) for _ in range(3)]
    zeros = torch.zeros(n, device="cuda")
    for a, b in sets:
        outs = []
        for bias in (None, zeros):
            c = torch.full((m, n), float("nan"), device="cuda")
            call("br_hip_gemm", 1, 0, m, n, k, 0.25, ptr(a), F16, m, 0, ptr(b), F16, n, 0, 0, ptr(c), F32, n, 0, ptr(bias),
                 1, hip.GEMM_F16, stream())
            outs.append(c)
        torch.cuda.synchronize()
        assert torch.equal(outs[0], outs[1])
        rows = torch.arange(0, m, 257, device="cuda")
        ref = 0.25 * (a[:, rows].double().t() @ b.double())
        err = (outs[0][rows].double() - ref).abs()
        assert bool((err <= 1e-5 * (ref.abs() + ref.pow(2).mean().sqrt()) * (k ** 0.5)).all())


@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("n,c_dt", [(12288, F16), (12248, F32)])
def test_gemm_round_and_a_half_of_tiles(ta, tb, n, c_dt):
    """[2048 x 12288] from K = 1024: 384 tiles of 256 x 256 are a round and a
    half on 256 CUs, which the dispatcher runs as two launches (8192 columns on
    256 x 256 tiles, the rest on 256 x 128 tiles).  Bias, alpha and an
    accumulated C cross the seam; the ragged case ends inside the second
    launch's last tile."""
    rng = np.random.default_rng(21)
    m, k = 2048, 1024
    print("case ta=%d tb=%d n=%d c_dt=%d" % (ta, tb, n, c_dt), flush=True)
    a, b = operands(rng, ta, tb, m, n, k)
    bias = rng.standard_normal(n).astype(np.float32)
    c0 = rng.standard_normal((1, m, n)).astype(np.float32)
    got, ref = run_gemm(ta, tb, m, n, k, a, b, F16, F16, c_dt, hip.GEMM_F16, alpha=0.5, bias=bias, c0=c0)
    assert_close(got, ref, 2e-2, "two-launch product")
    if c_dt == F32:
        assert np.sqrt(np.mean((got - ref) ** 2)) < 1e-5 * np.sqrt(np.mean(ref ** 2)) * np.sqrt(k)


@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("c_dt", [F32, F16])
def test_gemm_tile_on_two_groups_of_waves(ta, tb, c_dt):
    """[1024 x 8192] from K = 2048: 256 tiles of 256 x 128 and 32 K steps, which the dispatcher runs with the
    sub-steps of every K step dealt to two groups of four waves whose sums meet in LDS after the K loop.  Alpha,
    bias and an accumulated C; against fp64, and with small-integer operands (every partial sum exact) bit for
    bit."""
    rng = np.random.default_rng(33)
    m, n, k = 1024, 8192, 2048
    print("case ta=%d tb=%d c_dt=%d" % (ta, tb, c_dt), flush=True)
    a, b = operands(rng, ta, tb, m, n, k)
    bias = rng.standard_normal(n).astype(np.float32)
    c0 = rng.standard_normal((1, m, n)).astype(np.float32)
    got, ref = run_gemm(ta, tb, m, n, k, a, b, F16, F16, c_dt, hip.GEMM_F16, alpha=0.5, bias=bias, c0=c0)
    assert_close(got, ref, 2e-2, "two wave groups")
    if c_dt == F32:
        assert np.sqrt(np.mean((got - ref) ** 2)) < 1e-5 * np.sqrt(np.mean(ref ** 2)) * np.sqrt(k)
        ai = rng.integers(-8, 9, a.shape).astype(np.float32)
        bi = rng.integers(-4, 5, b.shape).astype(np.float32)
        got, ref = run_gemm(ta, tb, m, n, k, ai, bi, F16, F16, F32, hip.GEMM_F16)
        assert np.array_equal(got, ref)


@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("a_dt,b_dt", [(F32, F16), (F16, F32), (F32, F32)])
def test_gemm_staged_matches_plain_entry(ta, tb, a_dt, b_dt):
    rng = np.random.default_rng(8)
    m, n, k, batch = 384, 256, 128, 3
    print("case staged ta=%d tb=%d dtypes=%s" % (ta, tb, (a_dt, b_dt)), flush=True)
    a, b = operands(rng, ta, tb, m, n, k, batch)
    bias = rng.standard_normal(n).astype(np.float32)
    staged, plain, need = run_gemm_staged(ta, tb, m, n, k, a, b, a_dt, b_dt, F32, hip.GEMM_F16, batch=batch, bias=bias)
    assert need == sum(2 * batch * r * c for r, c, dt in ((m, k, a_dt), (k, n, b_dt)) if dt == F32)
    # same operand rounding, same products; only the summation order inside a
    # K step may differ between the two kernels
    assert_close(staged, plain, 1e-5, "staged vs plain")


@pytest.mark.parametrize("ta,tb", [(0, 1), (0, 0), (1, 0), (1, 1)])
@pytest.mark.parametrize("a_dt,b_dt,c_dt", [(F32, F16, F32), (F16, F16, F16), (F32, F32, F32)])
def test_gemm_staged_split_k(ta, tb, a_dt, b_dt, c_dt):
    """Few output tiles and a long K: the staged entry splits K (the workspace
    figure shows it) and must still give the plain product, with alpha, bias
    and accumulation applied once."""
    rng = np.random.default_rng(10)
    m, n, k = 256, 384, 4096
    print("case split-k ta=%d tb=%d dtypes=%s" % (ta, tb, (a_dt, b_dt, c_dt)), flush=True)
    a, b = operands(rng, ta, tb, m, n, k)
    bias = rng.standard_normal(n).astype(np.float32)
    c0 = rng.standard_normal((1, m, n)).astype(np.float32)
    da, db_, dbias = to_dev(a, a_dt), to_dev(b, b_dt), dev(bias)
    need = hip.load().br_hip_gemm_staged_workspace(int(ta), int(tb), m, n, k, a_dt, b_dt, 1)
    copies = sum(2 * r * c for r, c, dt in ((m, k, a_dt), (k, n, b_dt)) if dt == F32)
    splits = (need - copies) // (4 * m * n)
    assert splits >= 2 and need == copies + splits * 4 * m * n
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    c = to_dev(c0, c_dt)
    call("br_hip_gemm_staged", int(ta), int(tb), m, n, k, 0.5, ptr(da), a_dt, m if ta else k, 0, ptr(db_), b_dt,
         k if tb else n, 0, 1, ptr(c), c_dt, n, 0, ptr(dbias), 1, hip.GEMM_F16, ptr(ws), need, stream())
    A = to_host64(da).reshape((k, m) if ta else (m, k))
    B = to_host64(db_).reshape((n, k) if tb else (k, n))
    ref = 0.5 * ((A.T if ta else A) @ (B.T if tb else B)) + bias.astype(np.float64)[None, :] + \
        to_host64(to_dev(c0, c_dt)).reshape(m, n)
    assert_close(to_host64(c).reshape(m, n), ref, 2e-2, "split-k staged gemm")
    if c_dt == F32:
        assert np.sqrt(np.mean((to_host64(c).reshape(m, n) - ref) ** 2)) < 1e-3 * np.sqrt(np.mean(ref ** 2))


def test_gemm_split_in_two_on_two_streams_at_once():
    """The 4h -> h shape ([2048 x 4096] from K = 16384, split in two inside
    the kernel) on two streams at the same time, each with its own operands
    and workspace: the slices of a tile meet through a counter set per stream,
    so both streams give the bits they give alone."""
    torch.manual_seed(5)
    m, n, k = 2048, 4096, 16384
    lib = hip.load()
    need = lib.br_hip_gemm_staged_workspace(0, 1, m, n, k, F16, F16, 1)
    assert need >= m * n * 4          # room for the partial tiles: this shape takes the split
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    jobs = []
    for _ in streams:
        a = torch.randn((m, k), device="cuda").half()
        b = torch.randn((n, k), device="cuda").half()
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        jobs.append((a, b, ws))
    torch.cuda.synchronize()

    def launch(job, c, st):
        a, b, ws = job
        call("br_hip_gemm_staged", 0, 1, m, n, k, 1.0, ptr(a), F16, k, 0, ptr(b), F16, k, 0, 0, ptr(c), F32, n, 0, None, 1,
             hip.GEMM_F16, ptr(ws), need, ctypes.c_void_p(st.cuda_stream))
    alone = []
    for job, st in zip(jobs, streams):
        c = torch.full((m, n), float("nan"), device="cuda")
        launch(job, c, st)
        torch.cuda.synchronize()
        alone.append(c)
    together = [[torch.full((m, n), float("nan"), device="cuda") for _ in range(4)] for _ in streams]
    torch.cuda.synchronize()
    for r in range(4):
        for i, (job, st) in enumerate(zip(jobs, streams)):
            launch(job, together[i][r], st)
    torch.cuda.synchronize()
    for i in range(2):
        for r in range(4):
            assert torch.equal(together[i][r], alone[i]), (i, r)
    ref = jobs[0][0][:64].double() @ jobs[0][1].double().t()
    assert bool(((alone[0][:64].double() - ref).abs() <= 1e-5 * (ref.abs() + ref.pow(2).mean().sqrt()) * (k ** 0.5)).all())


def test_gemm_staged_falls_back():
    rng = np.random.default_rng(9)
    # K not a multiple of 32, fp32 compute, and a workspace that is too small
    for (m, n, k, compute, ws) in ((96, 80, 40, hip.GEMM_F16, None), (128, 128, 64, hip.GEMM_F32, None),
                                   (128, 128, 64, hip.GEMM_F16, 16)):
        a, b = operands(rng, 0, 1, m, n, k)
        staged, plain, _ = run_gemm_staged(0, 1, m, n, k, a, b, F32, F32, F32, compute, ws_bytes=ws)
        assert np.array_equal(staged, plain)


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


@pytest.mark.parametrize("dtype", [F16, BF16])
@pytest.mark.parametrize("rows,out,inn", [(512, 1024, 256), (200, 520, 96), (2048, 4096, 1024), (2048, 12288, 1024),
                                          (512, 16384, 2048)])   # the last: 256 x 128 tiles on two groups of waves
def test_linear_gelu_epilogue_writes_both_tensors(dtype, rows, out, inn):
    """br_hip_linear_gelu: u = x.W^T + bias and y = gelu(u) from one product.
    u against the fp64 product of the stored operands, y against the oracle's
    GELU of that fp64 u (the kernel takes the activation of the fp32 sum, so y
    does not inherit u's storage rounding); 2e-2 for 16-bit operands, plus the
    output's own rounding."""
    import oracle as orc
    print("case dtype=%d rows=%d out=%d in=%d" % (dtype, rows, out, inn), flush=True)
    rng = np.random.default_rng(rows + out)
    x = to_dev(rng.standard_normal((rows, inn)), dtype)
    w = to_dev(rng.standard_normal((out, inn)) / np.sqrt(inn) * 1.5, dtype)
    bias = (0.1 * rng.standard_normal(out)).astype(np.float32)
    u = torch.full((rows, out), float("nan"), dtype=TORCH_T[dtype], device="cuda")
    y = torch.full((rows, out), float("nan"), dtype=TORCH_T[dtype], device="cuda")
    call("br_hip_linear_gelu", ptr(x), ptr(w), ptr(dev(bias)), ptr(u), ptr(y), dtype, rows, out, inn, stream())
    ref_u = to_host64(x) @ to_host64(w).T + bias.astype(np.float64)
    ref_y = orc.gelu_fwd(ref_u.astype(np.float32)).astype(np.float64)
    tol = 2e-2 if dtype == F16 else 3e-2
    assert_close(to_host64(u), ref_u, tol, "pre-activation")
    assert_close(to_host64(y), ref_y, tol, "gelu")
    # shapes the direct-to-LDS kernel does not take are declined, nothing is written
    assert hip.load().br_hip_linear_gelu(ptr(x), ptr(w), None, ptr(u), ptr(y), dtype, rows, out, inn - 8, stream()) == -1
    assert hip.load().br_hip_linear_gelu(ptr(x), ptr(w), None, ptr(u), ptr(u), dtype, rows, out, inn, stream()) == -3
    torch.cuda.synchronize()
