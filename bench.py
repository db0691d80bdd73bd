#!/usr/bin/env python3
"""Benchmark of the BLOOM-7B1 training hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--leg all|block|model|roofline|elementwise|copy]

A "step" is one forward + backward pass of one BLOOM-7B1 decoder block
(hidden 4096, 32 heads x 128, FFN 16384, ALiBi causal attention, batch 4 x
seq 512, fp16 weights, fp32 activations and accumulation) run through the
product path: word script -> word machine -> TensorType -> HIPTensor -> HIP
kernels.  Inputs and weights are resident in HBM before the timed region.

One JSON line is printed.  Besides the step throughput it carries
  roofline      the dominant kernel (the direct-to-LDS MFMA GEMM in its
                weight-gradient form, at the h->4h shape of this block) timed
                on its own with HIP events on the launch stream
  elementwise   LayerNorm / bias-GELU / log-softmax+NLL kernels in GB/s
  gemms         every GEMM shape of the block in TFLOP/s (kernel alone, operand
                and output types as the headline words use them)
  cpu_baseline  the CPU oracle timed on the host cores on a bounded sample
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # dense fp16
# HBM bytes per launch of the roofline kernel at the roofline shape come from a
# committed rocprofv3 counter summary (FETCH_SIZE / WRITE_SIZE, each scaled by
# what the same counter reads on the copy leg), not from this run.
ROOFLINE_TRAFFIC_PROFILE = os.path.join("profiles", "gemm_dtl_f16_weight_gradient_hbm_traffic.txt")


def roofline_traffic():
    """(bytes per launch, source) from the line `traffic_bytes_per_launch = N`
    of the committed counter summary; (None, None) when it is absent."""
    try:
        with open(os.path.join(ROOT, ROOFLINE_TRAFFIC_PROFILE)) as f:
            for line in f:
                if line.lstrip("# ").startswith("traffic_bytes_per_launch"):
                    return float(line.split("=")[1].split()[0]), ROOFLINE_TRAFFIC_PROFILE
    except OSError:
        pass
    return None, None

H, NH, F, V = 4096, 32, 16384, 250880
B, T = 4, 512
N = B * T
# GEMM flops of one block, forward (attention counted dense T x T)
FWD_GEMM_FLOP = 2.0 * N * H * (3 * H + H + 2 * F) + 2 * 2.0 * B * NH * T * T * (H // NH)
STEP_GEMM_FLOP = 3.0 * FWD_GEMM_FLOP


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--leg", default="all", choices=["all", "block", "model", "roofline", "elementwise", "copy"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU-baseline leg")
    ap.add_argument("--block-words", default="flash", choices=["flash", "mixed", "plain"],
                    help="with --headline-words-only: which of the three word sets of the block leg to time "
                         "(for kernel profiles of the operator-chain paths)")
    ap.add_argument("--headline-words-only", action="store_true",
                    help="block leg: time only the word set `value` is quoted on (for kernel profiles of it alone)")
    return ap.parse_args()


class Timer:
    """HIP events recorded on the stream the kernels are launched on."""

    def __init__(self, hip, stream):
        self.hip, self.stream = hip, stream
        self.device_sync = None
        self.e0, self.e1 = ctypes.c_void_p(), ctypes.c_void_p()
        hip.call("br_hip_event_create", ctypes.byref(self.e0))
        hip.call("br_hip_event_create", ctypes.byref(self.e1))

    def run(self, fn, iters, warmup, blocker=None):
        """Seconds per call of fn.  `blocker` enqueues a long kernel right before
        the first event: the timed launches then pile up behind it in the queue and
        run back to back, so that for kernels of a few microseconds the time
        between the events is kernel time and not the host's launch rate."""
        if self.device_sync:
            self.device_sync()   # buffers made on another stream are complete
        for i in range(warmup):
            fn(i)
        self.hip.call("br_hip_stream_sync", self.stream)
        if blocker:
            blocker()
        self.hip.call("br_hip_event_record", self.e0, self.stream)
        for i in range(iters):
            fn(i)
        self.hip.call("br_hip_event_record", self.e1, self.stream)
        self.hip.call("br_hip_event_sync", self.e1)
        ms = ctypes.c_float()
        self.hip.call("br_hip_event_elapsed_ms", self.e0, self.e1, ctypes.byref(ms))
        return ms.value * 1e-3 / iters   # seconds per iteration


def block_leg(args, host, hip, timer):
    rng = np.random.default_rng(3)
    env = host.Env(2)
    env.execute(host.words_text("bloom.words"))
    env.execute("%d %d %d 1e-05 model_dims" % (H, NH, V))
    env.set("$DEVICE", "cuda")
    env.set("$WDTYPE", "f16")
    env.execute("'f16' op.gemm_precision")
    env.execute("create_layer_weight create_layer_grad zero_layer_grad")
    env.execute("%d %d dynamic_floats" % (B, T))
    floats = int(env.pop_number()) + V
    env.execute("%d create_var  %d %d create_dynamic" % (floats, B, T))
    env.execute("%d %d %d 3 'cuda' 'float' op.create 'yout_g0' !" % (B, T, H))

    def normal(shape, std, mean=0.0):
        return (mean + std * rng.standard_normal(shape)).astype(np.float32)

    for ln in ("input_layernorm", "post_attention_layernorm"):
        env.write(ln + ".weight", normal(H, 0.02, 1.0))
        env.write(ln + ".bias", normal(H, 0.02))
    for name, (o, i) in {"query_key_value": (3 * H, H), "dense": (H, H), "dense_h_to_4h": (F, H),
                         "dense_4h_to_h": (H, F)}.items():
        env.write(name + ".weight", normal((o, i), 0.02))
        env.write(name + ".bias", normal(o, 0.02))
    env.write("xinput", normal((B, T, H), 1.0))
    env.write("yout_g0", normal((B, T, H), 1.0))
    env.write("mask_", np.ones((B, T), np.int32))
    env.execute("create_operand_buffers create_flash_buffers prepare_batch_flash op.sync")
    # The operator-chain backward adds into yout_g in place, so each of its steps starts from a fresh copy;
    # the fused-attention backward leaves yout_g as it is (the next block's gradient is read where it lies).
    # block_step        the reference's operator sequence over the fp32 arena
    # block_step_mixed  the same sequence with product-only operands kept in fp16 buffers;
    #                   it produces the bits block_step produces (tests/test_gpu_block.py)
    # block_step_flash  block_step_mixed with the attention chain as one fused kernel per
    #                   direction (same tolerance against the oracle, not the same bits)
    env.execute("'yout_g' @ 'yout_g0' @ op.copy op.sync")
    step = env.build("block_step_flash")
    mixed = env.build("'yout_g' @ 'yout_g0' @ op.copy  block_step_mixed")
    plain = env.build("'yout_g' @ 'yout_g0' @ op.copy  block_step")
    if args.headline_words_only and args.block_words != "flash":
        sec = timer.run(lambda i: env.run(mixed if args.block_words == "mixed" else plain), args.steps, args.warmup)
        assert np.all(np.isfinite(env.read("xa"))), "block step produced non-finite values"
        env.close()
        return sec, None, None
    sec = timer.run(lambda i: env.run(step), args.steps, args.warmup)
    out_flash = env.read("xa")
    assert np.all(np.isfinite(out_flash)), "block step produced non-finite values"
    if args.headline_words_only:
        env.close()
        return sec, None, None
    few = max(3, args.steps // 4)
    sec_mixed = timer.run(lambda i: env.run(mixed), few, 1)
    out = env.read("xa")
    sec_plain = timer.run(lambda i: env.run(plain), few, 1)
    assert np.array_equal(env.read("xa"), out), "the two operator-chain word sets disagree"
    scale = float(np.sqrt(np.mean(out.astype(np.float64) ** 2)))
    assert float(np.max(np.abs(out_flash - out))) <= 2e-2 * (float(np.max(np.abs(out))) + scale), \
        "fused attention and the operator chain disagree"
    env.close()
    return sec, sec_mixed, sec_plain


def model_leg(args, host, timer):
    """BASELINE configs[4]: 30 blocks + embedding LayerNorm + final LayerNorm +
    LM-head loss, forward and backward, batch 1 x 512, every layer resident."""
    layers, batch, tokens = 30, 1, T
    model = host.BloomModel(layers, batch, tokens, H, NH, V, 1e-5, "f16", "f16")
    model.init(4, 0.02)
    rng = np.random.default_rng(4)
    ids = rng.integers(0, V, (batch, tokens)).astype(np.int32)
    mask = np.ones((batch, tokens), np.int32)
    mask[0, tokens - 37:] = 0                       # right padding, 37 of 512 masked
    steps = max(3, args.steps // 4)
    losses = []
    sec = timer.run(lambda i: losses.append(model.step(ids, mask)), steps, max(2, args.warmup // 4))
    assert all(np.isfinite(l) for l in losses), "model step produced a non-finite loss"
    n = batch * tokens
    fwd_block = 2.0 * n * H * (3 * H + H + 2 * F) + 2 * 2.0 * batch * NH * tokens * tokens * (H // NH)
    flop = 3.0 * (layers * fwd_block + 2.0 * n * H * V)
    model.close()
    return {"workload": "BLOOM-7B1, 30 blocks + LM head (BASELINE configs[4]), batch 1 x 512, fp16 weights, "
                        "no recomputation", "ms_per_step": sec * 1e3, "tokens_per_s": n / sec,
            "gemm_tflop_per_step": flop / 1e12, "gemm_tflops": flop / sec / 1e12, "loss": losses[-1],
            "steps": steps}


def gemm_case(hip, timer, torch, ta, tb, m, n, k, a_dt, b_dt, c_dt, batch=1, iters=20, staged=False, sets=1,
              warmup=40):
    """Times one product.  staged=True goes through br_hip_gemm_staged the way
    the tensor backend does (fp32 operands converted into a scratch block,
    conversion time included).  sets > 1 rotates that many operand / output
    sets so that no launch finds its operands in the last-level cache.  The
    warm-up is long on purpose: from idle the clock needs ~100 launches of
    this size to settle, and the first dozens run 20-25 % slower."""
    tt = {hip.F32: torch.float32, hip.F16: torch.float16}
    a = [torch.randn((batch, m * k), device="cuda").to(tt[a_dt]) for _ in range(sets)]
    b = [torch.randn((batch, n * k), device="cuda").to(tt[b_dt]) for _ in range(sets)]
    c = [torch.empty((batch, m * n), device="cuda", dtype=tt[c_dt]) for _ in range(sets)]
    lda, ldb = (m if ta else k), (k if tb else n)
    st = timer.stream

    def common(i):
        j = i % sets
        return (ta, tb, m, n, k, 1.0, ctypes.c_void_p(a[j].data_ptr()), a_dt, lda, m * k,
                ctypes.c_void_p(b[j].data_ptr()), b_dt, ldb, n * k, 0, ctypes.c_void_p(c[j].data_ptr()), c_dt, n, m * n,
                None, batch, hip.GEMM_F16)
    if staged:
        need = hip.load().br_hip_gemm_staged_workspace(ta, tb, m, n, k, a_dt, b_dt, batch)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")

        def fn(i):
            hip.call("br_hip_gemm_staged", *common(i), ctypes.c_void_p(ws.data_ptr()), need, st)
    else:
        def fn(i):
            hip.call("br_hip_gemm", *common(i), st)
    sec = timer.run(fn, iters, warmup)
    return sec, 2.0 * m * n * k * batch


def roofline_leg(hip, timer, torch, full):
    """Dominant kernel: the direct-to-LDS fp16 MFMA GEMM in its weight-gradient
    form (both operands row-contiguous, fp32 output), which takes the largest
    share of the block step (four launches, ~30 % of its time); timed at the
    h->4h weight gradient dW[16384, 4096] = dy[2048, 16384]^T . x[2048, 4096]
    with operands as the tensor backend hands them over (already fp16), four
    operand sets in rotation."""
    f32, f16 = hip.F32, hip.F16
    sec, flop = gemm_case(hip, timer, torch, 1, 0, F, H, N, f16, f16, f32, iters=60, sets=4, warmup=150)
    traffic, source = roofline_traffic()
    roof = {"bound": "mfma", "kernel": "gemm_dtl_walk_kernel, 256x256x64 tiles (A fp16 [k,m], B fp16 [k,n], C fp32)",
            "shape": "m=%d n=%d k=%d" % (F, H, N), "achieved": flop / sec / 1e12, "peak": MFMA_F16_PEAK_TFLOPS,
            "unit": "TFLOP/s", "frac": flop / sec / 1e12 / MFMA_F16_PEAK_TFLOPS, "us_per_launch": sec * 1e6,
            "traffic": traffic, "traffic_source": source}
    # what a bare MFMA loop (no memory traffic) reaches on this box with operands of zeros and of random values
    scratch = torch.empty(1 << 17, device="cuda")
    probe = ctypes.CDLL(os.path.join(ROOT, "blackriver_amd", "lib", "libbr_probe.so"))
    probe.br_probe_mfma_f16.restype = ctypes.c_int
    probe.br_probe_mfma_f16.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64,
                                        ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
    loop = {}
    for name, rnd in (("zeros", 0), ("random", 1)):
        tf = ctypes.c_double()
        rc = probe.br_probe_mfma_f16(rnd, 8000, ctypes.c_void_p(scratch.data_ptr()), scratch.numel(), ctypes.byref(tf),
                                     timer.stream)
        assert rc == 0, "MFMA calibration loop failed with %d" % rc
        loop[name] = round(tf.value, 1)
    roof["mfma_loop_tflops"] = loop
    roof["frac_of_random_operand_loop"] = roof["achieved"] / loop["random"]
    # yardstick, not product: the vendor library's product of the same shape (fp16 in, fp16 out) through torch
    a = torch.randn((N, F), device="cuda", dtype=torch.float16)
    b = torch.randn((N, H), device="cuda", dtype=torch.float16)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for i in range(150 + 30):
        if i == 150:
            e0.record()
        torch.matmul(a.t(), b)
    e1.record()
    torch.cuda.synchronize()
    roof["vendor_library_tflops_fp16_out"] = round(flop / (e0.elapsed_time(e1) * 1e-3 / 30) / 1e12, 1)
    gemms = []
    if full:
        hd = H // NH
        cases = [
            ("qkv fwd  y=xW^T", 0, 1, N, 3 * H, H, f16, f16, f16, 1),
            ("dense fwd", 0, 1, N, H, H, f16, f16, f32, 1),
            ("h->4h fwd (+GELU epilogue in the step)", 0, 1, N, F, H, f16, f16, f16, 1),
            ("4h->h fwd", 0, 1, N, H, F, f16, f16, f32, 1),
            ("dx=dy.W (4h->h)", 0, 0, N, F, H, f16, f16, f16, 1),
            ("dx=dy.W (h->4h)", 0, 0, N, H, F, f16, f16, f32, 1),
            ("dW=dy^T.x (h->4h)", 1, 0, F, H, N, f16, f16, f32, 1),
            ("dW=dy^T.x (dense)", 1, 0, H, H, N, f16, f16, f32, 1),
            ("QK^T (operator chain only)", 0, 1, T, T, hd, f16, f16, f32, B * NH),
            ("PV (operator chain only)", 0, 0, T, hd, T, f16, f16, f16, B * NH),
        ]
        for name, ta, tb, m, n, k, a_dt, b_dt, c_dt, batch in cases:
            # through the entry the tensor backend uses (16-bit operands are taken as they are; the workspace
            # gives a long-K product room for the partial tiles of a K split)
            s16, fl = gemm_case(hip, timer, torch, ta, tb, m, n, k, a_dt, b_dt, c_dt, batch, iters=12, sets=3,
                                staged=True)
            gemms.append({"name": name, "m": m, "n": n, "k": k, "batch": batch, "c": "f32" if c_dt == f32 else "f16",
                          "kernel_us": round(s16 * 1e6, 1), "kernel_tflops": round(fl / s16 / 1e12, 1),
                          "kernel_frac": round(fl / s16 / 1e12 / MFMA_F16_PEAK_TFLOPS, 3)})
    return roof, gemms


def elementwise_leg(hip, timer, torch):
    """C1-C3 kernels; buffers are rotated so the 256 MB last-level cache
    cannot serve the 33-134 MB working sets."""
    lib = hip.load()
    st = timer.stream
    vp = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
    out = {}

    def rec(name, sec, nbytes):
        gbs = nbytes / sec / 1e9
        out[name] = {"us": round(sec * 1e6, 2), "GB/s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 3),
                     "algorithmic_MB": round(nbytes / 1e6, 2)}

    # ~1.5 ms of fill kernels: longer than the host needs to enqueue 200 launches
    block_buf = torch.empty(1 << 30, device="cuda")

    def blocker():
        for _ in range(2):
            hip.call("br_hip_fill", vp(block_buf), hip.F32, 0.0, block_buf.numel(), st)

    nb = 8
    rows, cols = 2048, 4096
    xs = [torch.randn((rows, cols), device="cuda") for _ in range(nb)]
    ys = [torch.empty_like(x) for x in xs]
    dys = [torch.randn((rows, cols), device="cuda") for _ in range(nb)]
    dxs = [torch.empty_like(x) for x in xs]
    g = torch.randn(cols, device="cuda") * 0.02 + 1
    b = torch.randn(cols, device="cuda") * 0.02
    mean, var = torch.empty(rows, device="cuda"), torch.empty(rows, device="cuda")
    dg, db = torch.empty(cols, device="cuda"), torch.empty(cols, device="cuda")
    sec = timer.run(lambda i: hip.call("br_hip_layernorm_fwd", vp(xs[i % nb]), vp(g), vp(b), vp(ys[i % nb]), vp(mean),
                                       vp(var), rows, cols, 1e-5, st), 200, 10, blocker)
    rec("layernorm_fwd [2048,4096] f32", sec, 2 * rows * cols * 4)
    ws = torch.empty(lib.br_hip_layernorm_bwd_workspace(rows, cols), dtype=torch.uint8, device="cuda")
    sec = timer.run(lambda i: hip.call("br_hip_layernorm_bwd", vp(dys[i % nb]), vp(ys[i % nb]), vp(g), vp(b), vp(var),
                                       vp(dg), vp(db), vp(dxs[i % nb]), rows, cols, 1e-5, 1.0, vp(ws), ws.numel(), st),
                    200, 10, blocker)
    rec("layernorm_bwd [2048,4096] f32", sec, 3 * rows * cols * 4)
    # yardstick: a plain copy of the same tensors (same rotation, same timing method)
    sec = timer.run(lambda i: hip.call("br_hip_cast", vp(xs[i % nb]), hip.F32, vp(ys[i % nb]), hip.F32, rows * cols, st),
                    200, 10, blocker)
    rec("copy [2048,4096] f32 (yardstick)", sec, 2 * rows * cols * 4)
    del xs, ys, dys, dxs

    rows, cols = 2048, 16384
    xs = [(torch.randn((rows, cols), device="cuda") * 1.5).half() for _ in range(nb)]
    ys = [torch.empty_like(x) for x in xs]
    dys = [torch.randn((rows, cols), device="cuda").half() for _ in range(nb)]
    bias = torch.randn(cols, device="cuda") * 0.02
    dbias = torch.empty(cols, device="cuda")
    sec = timer.run(lambda i: hip.call("br_hip_bias_gelu_fwd", vp(xs[i % nb]), vp(bias), vp(ys[i % nb]), hip.F16, rows,
                                       cols, st), 200, 10, blocker)
    rec("bias_gelu_fwd [2048,16384] f16", sec, 2 * rows * cols * 2)
    ws = torch.empty(lib.br_hip_bias_gelu_bwd_workspace(rows, cols), dtype=torch.uint8, device="cuda")
    sec = timer.run(lambda i: hip.call("br_hip_bias_gelu_bwd", vp(dys[i % nb]), vp(xs[i % nb]), vp(bias), vp(ys[i % nb]),
                                       vp(dbias), hip.F16, rows, cols, 1.0, vp(ws), ws.numel(), st), 200, 10, blocker)
    rec("bias_gelu_bwd [2048,16384] f16 (+dbias)", sec, 3 * rows * cols * 2)
    del xs, ys, dys

    # ALiBi + causal / padding mask + softmax over the scores of config C4 in one pass (the kernel the word machine
    # puts in place of `op.add op.add op.softmax`), and the softmax backward of the same shape
    heads = NH
    ss = [torch.randn((B, heads, T, T), device="cuda") for _ in range(4)]
    pp = [torch.empty_like(x) for x in ss]
    alibi = torch.empty((heads, T), device="cuda")
    xmask = torch.empty((B, T, T), device="cuda")
    mask = torch.ones((B, T), device="cuda", dtype=torch.int32)
    mask[-1, T - T // 4:] = 0
    hip.call("br_hip_alibi_table", vp(alibi), heads, T, st)
    hip.call("br_hip_xmask_table", vp(mask), vp(xmask), B, T, st)
    sec = timer.run(lambda i: hip.call("br_hip_alibi_masked_softmax_fwd", vp(ss[i % 4]), vp(alibi), vp(xmask), vp(pp[i % 4]),
                                       B, heads, T, T, st), 100, 10, blocker)
    rec("alibi_masked_softmax_fwd [4,32,512,512] f32", sec, 2 * B * heads * T * T * 4 + B * T * T * 4)
    dd = [torch.empty_like(x) for x in ss]
    sec = timer.run(lambda i: hip.call("br_hip_softmax_bwd", vp(ss[i % 4]), vp(pp[i % 4]), vp(dd[i % 4]),
                                       B * heads * T, T, st), 100, 10, blocker)
    rec("softmax_bwd [65536,512] f32", sec, 3 * B * heads * T * T * 4)
    del ss, pp, dd, block_buf

    rows, vocab = 2048, V
    logits = torch.randn((rows, vocab), device="cuda") * 2.0
    dl = torch.empty_like(logits)
    target = torch.randint(0, vocab, (rows,), device="cuda", dtype=torch.int32)
    keep = (torch.rand(rows, device="cuda") < 0.9).to(torch.int32)
    lse, rl, res = (torch.empty(rows, device="cuda"), torch.empty(rows, device="cuda"), torch.empty(2, device="cuda"))
    sec = timer.run(lambda i: hip.call("br_hip_logsoftmax_nll_fwd", vp(logits), vp(target), vp(keep), vp(lse), vp(rl),
                                       vp(res), rows, vocab, st), 20, 3)
    rec("logsoftmax_nll_fwd [2048,250880] f32", sec, rows * vocab * 4)
    sec = timer.run(lambda i: hip.call("br_hip_logsoftmax_nll_bwd", vp(logits), vp(target), vp(keep), vp(lse), vp(dl),
                                       hip.F32, 1.0 / rows, rows, vocab, st), 20, 3)
    rec("logsoftmax_nll_bwd [2048,250880] f32", sec, 2 * rows * vocab * 4)
    del logits, dl

    # AdamW over one h -> 4h matrix (fp16 parameter with fp32 master copy):
    # reads grad, m, v, master (16 B), writes m, v, master (12 B) and the fp16 parameter (2 B)
    n = 4 * 4096 * 4096
    ps = [torch.zeros(n, device="cuda", dtype=torch.float16) for _ in range(2)]
    ms = [torch.randn(n, device="cuda") * 0.02 for _ in range(2)]
    gs = [torch.randn(n, device="cuda") for _ in range(2)]
    m1 = [torch.zeros(n, device="cuda") for _ in range(2)]
    m2 = [torch.zeros(n, device="cuda") for _ in range(2)]
    sec = timer.run(lambda i: hip.call("br_hip_adamw", vp(ps[i % 2]), hip.F16, vp(ms[i % 2]), vp(gs[i % 2]),
                                       vp(m1[i % 2]), vp(m2[i % 2]), n, 1e-4, 0.9, 0.95, 1e-8, 0.01, 1 + i // 2, st),
                    40, 4)
    rec("adamw [16384,4096] f16 + f32 master", sec, 30 * n)
    return out


def copy_leg(hip, timer, torch):
    """A plain copy kernel of known size (256 MiB read, 256 MiB written per
    launch): the yardstick the FETCH_SIZE / WRITE_SIZE counters of the GEMM are
    scaled by."""
    n = 64 << 20
    src = torch.randn(n, device="cuda")
    dst = torch.empty(n, device="cuda")
    st = timer.stream

    def fn(i):
        hip.call("br_hip_cast", ctypes.c_void_p(src.data_ptr()), hip.F32, ctypes.c_void_p(dst.data_ptr()), hip.F32, n, st)
    sec = timer.run(fn, 10, 2)
    return {"kernel": "copy_x16_kernel", "bytes_read": 4 * n, "bytes_written": 4 * n,
            "us": sec * 1e6, "GB/s": 8 * n / sec / 1e9}


def cpu_baseline_leg():
    """The CPU oracle (a restatement of the reference's operators; the
    reference itself has no CPU math path) on a bounded sample: one step of
    the same block at the same batch 4 x 512 tokens, forward + backward, all
    host threads (about 13 s)."""
    import oracle as orc
    from oracle import bloom_block as blk
    rng = np.random.default_rng(3)
    b, t = B, T
    w = blk.make_weights(rng, H, std=0.02)
    x = rng.standard_normal((b, t, H)).astype(np.float32)
    dy = rng.standard_normal((b, t, H)).astype(np.float32)
    alibi, xmask = orc.alibi(NH, t), orc.xmask(np.ones((b, t), np.int32))
    t0 = time.perf_counter()
    s = blk.layer_forward(w, x, alibi, xmask, NH)
    blk.layer_backward(w, s, x, dy, NH)
    sec = time.perf_counter() - t0
    return {"value": b * t / sec, "unit": "tokens/s", "cores": orc.threads(), "kind": "port",
            "sample": "one step of the same block (H=4096, 32 heads, FFN 16384) fwd+bwd at batch %d x %d tokens, fp32 "
                      "storage with fp64 accumulation, %.1f s of CPU work" % (b, t, sec),
            "kernels": cpu_kernel_rows(orc)}


def cpu_kernel_rows(orc):
    """The memory-bound kernels of configurations C1-C3 and the masked softmax
    of C4 on the host cores (the oracle's restatements, all threads): wall time
    and the same algorithmic bytes per second the GPU rows quote.  C1 and C2 run
    at full size, the softmax on one of the four sequences, C3 on a 64-row
    sample of its 2048 rows (1 MB per row; the kernels are row-parallel, so the
    rate carries over).  A baseline to read the GPU rows against, never
    a target."""
    rng = np.random.default_rng(0)
    rows = {}

    def timed(fn, reps=3):
        fn()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        return (time.perf_counter() - t0) / reps

    def rec(name, sec, nbytes, note=""):
        rows[name] = {"us": round(sec * 1e6, 1), "GB/s": round(nbytes / sec / 1e9, 2), "algorithmic_MB": round(nbytes / 1e6, 2)}
        if note:
            rows[name]["sample"] = note

    r, c = 2048, 4096
    x = rng.standard_normal((1, r, c)).astype(np.float32)
    g = (1 + 0.02 * rng.standard_normal(c)).astype(np.float32)
    bt = (0.02 * rng.standard_normal(c)).astype(np.float32)
    dy = rng.standard_normal((1, r, c)).astype(np.float32)
    y, _, var = orc.layernorm_fwd(x, g, bt, 1e-5)
    rec("layernorm_fwd [2048,4096] f32", timed(lambda: orc.layernorm_fwd(x, g, bt, 1e-5)), 2 * r * c * 4)
    rec("layernorm_bwd [2048,4096] f32", timed(lambda: orc.layernorm_bwd(dy, y, g, bt, var, 1e-5)), 3 * r * c * 4)
    r, c = 2048, 16384
    x = (1.5 * rng.standard_normal((r, c))).astype(np.float32)
    bias = (0.02 * rng.standard_normal(c)).astype(np.float32)
    dy = rng.standard_normal((r, c)).astype(np.float32)
    # the CPU path stores fp32 (the reference has no 16-bit host type); bytes are counted as the GPU row counts
    # them (2 B per element), so the two GB/s columns compare like with like
    rec("bias_gelu_fwd [2048,16384]", timed(lambda: orc.bias_gelu_fwd(x, bias)), 2 * r * c * 2, "fp32 storage on the host")
    rec("bias_gelu_bwd [2048,16384] (+dbias)", timed(lambda: orc.bias_gelu_bwd(dy, x, bias)), 3 * r * c * 2,
        "fp32 storage on the host")
    # the scores of one sequence of config C4 (a quarter of its batch): the reference's three operators in a row
    # (two broadcast additions and the softmax), then the softmax backward
    b1, nh, t = 1, NH, T
    s = rng.standard_normal((b1, nh, t, t)).astype(np.float32)
    al = orc.alibi(nh, t).reshape(1, nh, 1, t)
    xm = orc.xmask(np.ones((b1, t), np.int32)).reshape(b1, 1, t, t)
    p = orc.softmax_fwd(orc.add_bcast(orc.add_bcast(s, al), xm))
    rec("alibi_masked_softmax_fwd [4,32,512,512] f32", timed(lambda: orc.softmax_fwd(orc.add_bcast(orc.add_bcast(s, al), xm))),
        2 * b1 * nh * t * t * 4 + b1 * t * t * 4, "one of the 4 sequences; three host operators in a row")
    rec("softmax_bwd [65536,512] f32", timed(lambda: orc.softmax_bwd(s, p)), 3 * b1 * nh * t * t * 4, "one of the 4 sequences")
    r, v = 64, V
    logits = (2.0 * rng.standard_normal((r, v))).astype(np.float32)
    target = rng.integers(0, v, r).astype(np.int32)
    keep = (rng.random(r) < 0.9).astype(np.int32)
    note = "64 of the 2048 rows"
    rec("logsoftmax_nll_fwd [2048,250880] f32", timed(lambda: orc.logsoftmax_nll(logits, target, keep, False)), r * v * 4, note)
    both = timed(lambda: orc.logsoftmax_nll(logits, target, keep, True))
    rec("logsoftmax_nll_fwd+bwd [2048,250880] f32", both, 3 * r * v * 4, note + "; the host routine computes the loss and "
        "the gradient in one call")
    return rows


def main():
    args = parse()
    world = int(os.environ.get("WORLD_SIZE", "1"))
    if args.gpus != 1 or world != 1:
        print("bench.py measures one GPU: every layer of a configuration lives on a single MI355X and there is no "
              "multi-GPU path in this build (--gpus %d, WORLD_SIZE %d)." % (args.gpus, world), file=sys.stderr)
        sys.exit(2)
    import torch
    from blackriver_amd import hip, host
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    torch.cuda.init()
    host.boot(0, 1 << 30)
    host.set_echo_loss(False)   # stdout carries the one JSON line
    stream = ctypes.c_void_p(host.stream())
    timer = Timer(hip, stream)
    timer.device_sync = torch.cuda.synchronize

    result = {"metric": "elementwise GB/s (% of 8 TB/s HBM) + BLOOM-7B1 block fwd+bwd tokens/sec",
              "value": None, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
              "ms_per_step": None, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
              "data": "synthetic",
              "config": {"workload": "one BLOOM-7B1 decoder block fwd+bwd (BASELINE configs[3]): hidden 4096, "
                                     "32 heads x 128, FFN 16384, ALiBi causal attention, batch 4 x seq 512, fp16 "
                                     "weights ~N(0,0.02), fp32 activations and accumulation, seed 3",
                         "tokens_per_step": N, "gemm_gflop_per_step": STEP_GEMM_FLOP / 1e9}}
    if args.leg in ("all", "block"):
        sec, sec_mixed, sec_plain = block_leg(args, host, hip, timer)
        if sec_mixed is not None:
            result["ms_per_step_operator_chain_fp16_buffers"] = sec_mixed * 1e3
            result["ms_per_step_fp32_arena_words"] = sec_plain * 1e3
        result["value"] = N / sec
        result["ms_per_step"] = sec * 1e3
        result["step_gemm_tflops"] = STEP_GEMM_FLOP / sec / 1e12
        result["step_frac_of_mfma_peak"] = STEP_GEMM_FLOP / sec / 1e12 / MFMA_F16_PEAK_TFLOPS
    if args.leg in ("all", "model"):
        result["model"] = model_leg(args, host, timer)
    if args.leg in ("all", "roofline"):
        roof, gemms = roofline_leg(hip, timer, torch, full=args.leg == "all")
        result["roofline"] = roof
        if gemms:
            result["gemms"] = gemms
    if args.leg in ("all", "elementwise"):
        result["elementwise"] = elementwise_leg(hip, timer, torch)
    if args.leg == "copy":
        result["copy"] = copy_leg(hip, timer, torch)
    if args.leg == "all" and not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline_leg()
    host.sync()
    print(json.dumps(result))
    host.shutdown()


if __name__ == "__main__":
    main()
