#!/usr/bin/env python3
"""Benchmark of the quantized-GEMM hot path on one MI355X.

One "step" is one pass over every (shape, M) case of the chosen workload with synthetic inputs already resident in
HBM.  The default workload is the AWQ W4A16 Llama-3-8B MLP sweep (gate/up N=14336,K=4096 and down N=4096,K=14336,
M in {1,8,32,128,512}, bf16).  Weight copies are rotated so that no launch finds its weights in the 256 MB
Infinity Cache.

Prints ONE JSON line.  `value` is the time-weighted fraction of the MI355X roofline over the step, in percent:
sum over cases of max(bytes / 8 TB/s, flops / MFMA peak) divided by the measured step time.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "quant GEMM TFLOPS + HBM GB/s (% of MI355X roofline) over M=1..4096"
HBM_PEAK = 8.0e12                                  # B/s
MFMA_PEAK = {"f16": 2.5e15, "bf16": 2.5e15, "fp8": 5.0e15}   # dense FLOP/s
CACHE_BYTES = 320 << 20                            # rotate through more than the Infinity Cache


# HBM bytes per launch of a kernel variant, averaged over the cases that run it: rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (KiB per dispatch), each scaled by the factor the same counter shows for a 256 MiB device copy
# (`--calibrate-copy`): FETCH_SIZE reads half the bytes moved (x2.0), WRITE_SIZE reads them exactly (x1.0).
# Keyed by (config, kernel variant); None where no counter run has been made for the current kernel.
MEASURED_TRAFFIC = {
    (1, "w4a16_splitk_kernel<16x16,w4>"): 9350000,
    (2, "w4a16_splitk_kernel<16x16,w4>"): 31050000,
    (2, "w4a16_splitk_kernel<16x64,w4>"): 31900000,
    (2, "w4a16_splitk_kernel<32x64,w4>"): 37040000,
    (2, "w4a16_tile_kernel<128x256,w8>"): 94830000,
    (3, "w4a16_tile_kernel<256x256,w8>"): 1592190000,
    (4, "fp8_group_quant"): 26940000,
    (4, "fp8_splitk_kernel<16x16,w4>"): 133530000,
    (4, "fp8_splitk_kernel<16x32,w4>"): 134280000,
    (4, "fp8_tile_kernel<128x256,w8>"): 176820000,
    (4, "fp8_tile_kernel<256x256,w8>"): 519390000,
    (7, "w4a8_quant"): 12690000,
    (7, "w4a8_splitk_kernel<16x32,w8>"): 14420000,
    (7, "w4a8_splitk_kernel<16x64,w4>"): 68990000,
    (7, "w4a8_tile_kernel<128x256,w8>"): 60220000,
    (7, "w4a8_tile_kernel<256x256,w8>"): 197070000,
}


def seeded(cfg, idx):
    g = torch.Generator(device="cpu")
    g.manual_seed(1000 * cfg + idx)
    return g


def awq_pack_cols(codes):
    """[R, N] uint8 codes -> [R, N/8] int32 in AWQ column order (nibble p holds column {0,2,4,6,1,3,5,7}[p])."""
    R, N = codes.shape
    c = codes.view(R, N // 8, 8).to(torch.int64)
    order = [0, 2, 4, 6, 1, 3, 5, 7]
    w = torch.zeros((R, N // 8), dtype=torch.int64)
    for p, col in enumerate(order):
        w |= c[:, :, col] << (4 * p)
    return (w & 0xFFFFFFFF).to(torch.int64).view(torch.int32).view(R, N // 8, 2)[:, :, 0].contiguous()


class Case:
    def __init__(self, name, launch, flops, nbytes, peak_key, kernel, copies=1):
        self.name, self.launch, self.flops, self.bytes, self.peak_key, self.kernel = name, launch, flops, nbytes, peak_key, kernel
        self.copies = copies
        t_hbm = nbytes / HBM_PEAK
        t_mfma = flops / MFMA_PEAK[peak_key]
        self.bound = "hbm" if t_hbm >= t_mfma else "mfma"
        self.t_bound = max(t_hbm, t_mfma)


def copies_needed(weight_bytes):
    return max(2, min(64, -(-CACHE_BYTES // weight_bytes) + 1))


# ------------------------------------------------------------------------------------------------ workloads
def w4a16_cases(ops, L, cfg, shapes, Ms, dtype, awq, x_std, s_lo, s_hi):
    dev = "cuda"
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    cases, keep = [], []
    for si, (tag, N, K) in enumerate(shapes):
        g = seeded(cfg, si)
        G = K // 128
        if awq:
            q = torch.randint(-2**31, 2**31 - 1, (K, N // 8), generator=g, dtype=torch.int32)
            layout = L.SRC_AWQ
        else:
            q = torch.randint(-2**31, 2**31 - 1, (K // 8, N), generator=g, dtype=torch.int32)
            layout = L.SRC_GPTQ
        scales = (torch.rand((G, N), generator=g) * (s_hi - s_lo) + s_lo).to(tdt)
        zeros = torch.randint(6, 10, (G, N), generator=g, dtype=torch.uint8) if awq else None
        wp1 = ops.repack_weight(q.to(dev), layout, 1, K, N)
        sp1 = ops.repack_scales(scales.to(dev), L.SCALE_GN, 1, K, N, 128)
        zp1 = ops.repack_zeros(awq_pack_cols(zeros).to(dev), L.ZERO_AWQ_PACKED, K, N, 128) if awq else None
        R = copies_needed(wp1.numel())
        wps = [wp1] + [wp1.clone() for _ in range(R - 1)]
        sps = [sp1] + [sp1.clone() for _ in range(R - 1)]
        zps = [zp1] + [zp1.clone() for _ in range(R - 1)] if awq else [None] * R
        state = {"i": 0}
        keep.append(dict(q=q, scales=scales, zeros=zeros, N=N, K=K, tag=tag, awq=awq))
        for mi, M in enumerate(Ms):
            x = (torch.randn((M, K), generator=seeded(cfg, 100 * si + mi + 10)) * x_std).to(tdt).to(dev)
            y = torch.empty((M, N), dtype=tdt, device=dev)
            keep[-1].setdefault("x", {})[M] = x
            need = L.load().ksq_w4a16_workspace_size(M, N, K, 128, L.F16 if dtype == "f16" else L.BF16)
            ws = torch.empty(need, dtype=torch.uint8, device=dev) if need else None

            def launch(x=x, y=y, N=N, K=K, wps=wps, sps=sps, zps=zps, state=state, R=R, ws=ws):
                i = state["i"] = (state["i"] + 1) % R
                ops.w4a16_gemm(x, wps[i], sps[i], zps[i], N, K, 128, out=y, workspace=ws)

            nbytes = K * N // 2 + G * N * 2 + (G * N // 2 if awq else 0) + 2 * M * K + 2 * M * N
            flops = 2 * M * N * K
            desc = L.select_tile(L.KIND_W4A16, M, N, K, L.F16 if dtype == "f16" else L.BF16)
            kern = "%s<%dx%d,w%d>" % ("w4a16_splitk_kernel" if desc["kernel"] == 0 else "w4a16_tile_kernel",
                                      desc["block_m"], desc["block_n"], desc["waves"])
            cases.append(Case("%s:M=%d" % (tag, M), launch, flops, nbytes, dtype, kern, R))
    return cases, keep


def fp8_cases(ops, L, cfg, shapes, Ms):
    dev = "cuda"
    cases, keep = [], []
    for si, (tag, N, K) in enumerate(shapes):
        g = seeded(cfg, si)
        # e4m3 codes of bf16 N(0,0.02^2) weights under a per-128x128 amax/448 scale: drawn directly as the codes of
        # w/s with w/s ~ N(0, (448/4.2)^2) clipped to +-448 (amax of 16384 normals is about 4.2 sigma)
        wn = (torch.randn((N, K), generator=g) * (448.0 / 4.2)).clamp_(-448, 448)
        b = wn.to(torch.float8_e4m3fn).view(torch.uint8)
        b_s = torch.full(((N + 127) // 128, K // 128), 0.02 * 4.2 / 448.0, dtype=torch.float32)
        R = copies_needed(b.numel())
        bs_ = [ops.fp8_repack_weight(b.to(dev))]   # the load-time repack into 2 KiB MFMA fragments
        bs_ += [bs_[0].clone() for _ in range(R - 1)]
        b_sd = b_s.to(dev)
        state = {"i": 0}
        keep.append(dict(b=b, b_s=b_s, N=N, K=K, tag=tag))
        for mi, M in enumerate(Ms):
            gx = seeded(cfg, 100 * si + mi + 10)
            x = torch.randn((M, K), generator=gx)
            x = torch.where(torch.rand((M, K), generator=gx) < 0.01, x * 20, x).to(torch.bfloat16).to(dev)
            a_q = torch.empty((M, K), dtype=torch.uint8, device=dev)
            a_s = torch.empty((K // 128, M), dtype=torch.float32, device=dev)
            y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)

            def quant(x=x, a_q=a_q, a_s=a_s, K=K):
                ops.per_token_group_quant_fp8(x, K, 128, True, False, q=a_q, s=a_s)

            need = L.load().ksq_fp8_blockwise_workspace_size(M, N, K)
            ws = torch.empty(need, dtype=torch.uint8, device=dev) if need else None

            def gemm(a_q=a_q, a_s=a_s, y=y, bs_=bs_, b_sd=b_sd, state=state, R=R, ws=ws):
                i = state["i"] = (state["i"] + 1) % R
                ops.fp8_blockwise_gemm(a_q, a_s, bs_[i], b_sd, out=y, workspace=ws)

            quant()
            cases.append(Case("%s:quant:M=%d" % (tag, M), quant, 0, 2 * M * K + M * K + 4 * M * K // 128, "fp8",
                              "fp8_group_quant"))
            nbytes = N * K + b_s.numel() * 4 + M * K + 4 * M * K // 128 + 2 * M * N
            desc = L.select_tile(L.KIND_FP8_BLOCKWISE, M, N, K, L.BF16)
            kern = "%s<%dx%d,w%d>" % ("fp8_splitk_kernel" if desc["kernel"] == 0 else "fp8_tile_kernel",
                                      desc["block_m"], desc["block_n"], desc["waves"])
            cases.append(Case("%s:gemm:M=%d" % (tag, M), gemm, 2 * M * N * K, nbytes, "fp8", kern, R))
    return cases, keep


def w4a8_cases(ops, L, cfg, shapes, Ms):
    """W4A8: static per-tensor e4m3 quantization of bf16 activations (with the group sums the GEMM needs), then int4
    weights x e4m3 activations on the fp8 matrix instruction."""
    dev = "cuda"
    cases, keep = [], []
    for si, (tag, N, K) in enumerate(shapes):
        g = seeded(cfg, si)
        w = torch.randint(0, 256, (K, N // 2), generator=g, dtype=torch.uint8)
        scales = (torch.rand((K // 128, N), generator=g) * 0.012 + 0.003).to(torch.float16)
        wp1 = ops.w4a8_repack_weight(w.to(dev))
        R = copies_needed(wp1.numel())
        wps = [wp1] + [wp1.clone() for _ in range(R - 1)]
        sc_d = scales.to(dev)
        in_scale = torch.tensor([0.05], dtype=torch.float32, device=dev)
        state = {"i": 0}
        for mi, M in enumerate(Ms):
            gx = seeded(cfg, 100 * si + mi + 10)
            x = torch.randn((M, K), generator=gx)
            x = torch.where(torch.rand((M, K), generator=gx) < 0.01, x * 20, x).to(torch.bfloat16).to(dev)
            a_q = torch.empty((M, K), dtype=torch.uint8, device=dev)
            xsum = torch.empty((K // 128, M), dtype=torch.float32, device=dev)
            y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)

            def quant(x=x, a_q=a_q, xsum=xsum, M=M, K=K):
                L.check(L.load().ksq_w4a8_static_quant(x.data_ptr(), in_scale.data_ptr(), a_q.data_ptr(), xsum.data_ptr(),
                                                       M, K, L.W4A8_PER_TENSOR, L.BF16,
                                                       torch.cuda.current_stream().cuda_stream))

            need = L.load().ksq_w4a8_workspace_size(M, N, K)
            ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)

            def gemm(a_q=a_q, xsum=xsum, y=y, wps=wps, sc_d=sc_d, state=state, R=R, ws=ws, N=N):
                i = state["i"] = (state["i"] + 1) % R
                ops.w4a8_gemm(a_q, xsum, wps[i], sc_d, 0.035, N, out=y, workspace=ws)

            quant()
            cases.append(Case("%s:quant:M=%d" % (tag, M), quant, 0, 2 * M * K + M * K + 4 * M * K // 128, "fp8",
                              "w4a8_quant"))
            nbytes = N * K // 2 + (K // 128) * N * 2 + M * K + 4 * M * K // 128 + 2 * M * N
            if M <= 32:
                nt = 4
                while nt > 1 and (N % (16 * nt) or N // (16 * nt) < 128):
                    nt //= 2
                kern = "w4a8_splitk_kernel<%dx%d,w%d>" % (16 if M <= 16 else 32, 16 * nt, 8 if N // (16 * nt) < 256 else 4)
            else:
                d = L.select_tile(L.KIND_FP8_BLOCKWISE, M, N, K, L.BF16)   # the W4A8 tile kernel runs on this plan
                kern = "w4a8_tile_kernel<%dx%d,w%d>" % (d["block_m"], d["block_n"], d["waves"])
            cases.append(Case("%s:gemm:M=%d" % (tag, M), gemm, 2 * M * N * K, nbytes, "fp8", kern, R))
    return cases, keep


def moe_cases(ops, L, cfg, Ts, E=256, hidden=7168, inter=2048, topk=8, distinct=32):
    dev = "cuda"
    g = seeded(cfg, 0)
    tdt = torch.bfloat16
    # `distinct` independent expert slabs tiled to E experts: 5.8 GB of device weights either way
    w13 = torch.randint(0, 256, (distinct, 2 * inter, hidden // 2), generator=g, dtype=torch.uint8)
    w2 = torch.randint(0, 256, (distinct, hidden, inter // 2), generator=g, dtype=torch.uint8)
    s13 = (torch.rand((distinct, 2 * inter, hidden // 128), generator=g) * 0.008 + 0.002).to(tdt)
    s2 = (torch.rand((distinct, hidden, inter // 128), generator=g) * 0.008 + 0.002).to(tdt)
    rep = E // distinct
    w13p = ops.repack_weight(w13.to(dev), L.SRC_MOE_NK, distinct, hidden, 2 * inter).repeat(rep)
    s13p = ops.repack_scales(s13.to(dev), L.SCALE_NG, distinct, hidden, 2 * inter, 128).repeat(rep)
    w2p = ops.repack_weight(w2.to(dev), L.SRC_MOE_NK, distinct, inter, hidden).repeat(rep)
    s2p = ops.repack_scales(s2.to(dev), L.SCALE_NG, distinct, inter, hidden, 128).repeat(rep)
    per_expert = (2 * inter * hidden // 2 + hidden * inter // 2) + (2 * inter * hidden // 128 + hidden * inter // 128) * 2
    cases = []
    for ti, T in enumerate(Ts):
        gx = seeded(cfg, 10 + ti)
        x = torch.randn((T, hidden), generator=gx).to(tdt).to(dev)
        logits = torch.randn((T, E), generator=gx)
        tw, ids = torch.topk(torch.softmax(logits, -1), topk, dim=-1)
        touched = int(torch.unique(ids).numel())
        ids_d, tw_d = ids.to(torch.int32).to(dev), tw.float().contiguous().to(dev)

        def launch(x=x, ids_d=ids_d, tw_d=tw_d):
            ops.fused_moe_w4a16(x, w13p, s13p, w2p, s2p, ids_d, tw_d, E, hidden, inter, 128)

        nbytes = per_expert * touched + 2 * T * hidden * 2 + 64 * T
        flops = 2 * T * topk * (2 * inter * hidden + hidden * inter)
        cases.append(Case("moe:T=%d" % T, launch, flops, nbytes, "bf16", "moe_w4a16"))
    return cases, []


def moe_fp8_cases(ops, L, cfg, Ts, E=256, hidden=7168, inter=2048, topk=8, distinct=32):
    """Block-fp8 experts (DeepSeek-V3's own expert format): weights e4m3 [E, N, K] + fp32 scales per 128 x 128 block."""
    dev = "cuda"
    g = seeded(cfg, 0)
    tdt = torch.bfloat16
    rep = E // distinct

    def experts(n, k):
        # random e4m3 codes without NaN (exponent-mantissa 0x7f) and scales of the size amax/448 gives for N(0, 0.02)
        q = torch.randint(0, 256, (distinct, n, k), generator=g, dtype=torch.uint8)
        q = torch.where((q & 0x7f) == 0x7f, q & 0xfe, q)
        s = torch.rand((distinct, n // 128, k // 128), generator=g) * 1e-4 + 1e-4
        return ops.fp8_repack_weight(q.to(dev)).repeat(rep, 1, 1), s.to(dev).repeat(rep, 1, 1)

    w13, s13 = experts(2 * inter, hidden)
    w2, s2 = experts(hidden, inter)
    per_expert = (2 * inter * hidden + hidden * inter) + (2 * inter * hidden + hidden * inter) // (128 * 128) * 4
    cases = []
    for ti, T in enumerate(Ts):
        gx = seeded(cfg, 10 + ti)
        x = torch.randn((T, hidden), generator=gx).to(tdt).to(dev)
        logits = torch.randn((T, E), generator=gx)
        tw, ids = torch.topk(torch.softmax(logits, -1), topk, dim=-1)
        touched = int(torch.unique(ids).numel())
        ids_d, tw_d = ids.to(torch.int32).to(dev), tw.float().contiguous().to(dev)

        def launch(x=x, ids_d=ids_d, tw_d=tw_d):
            ops.fused_moe_fp8_blockwise(x, w13, s13, w2, s2, ids_d, tw_d)

        nbytes = per_expert * touched + 2 * T * hidden * 2 + 64 * T
        flops = 2 * T * topk * (2 * inter * hidden + hidden * inter)
        cases.append(Case("moe_fp8:T=%d" % T, launch, flops, nbytes, "fp8", "moe_fp8_blockwise"))
    return cases, []


def build(cfg, ops, L):
    if cfg == 1:
        return ("GPTQ W4A16 fp16 N=K=4096 M in {1,16}",) + w4a16_cases(
            ops, L, 1, [("q_proj", 4096, 4096)], [1, 16], "f16", False, 1.0, 0.004, 0.02) + ("f16",)
    if cfg == 2:
        return ("AWQ W4A16 bf16 Llama-3-8B MLP gate/up(14336x4096)+down(4096x14336) M in {1,8,32,128,512}",) + \
            w4a16_cases(ops, L, 2, [("gate_up", 14336, 4096), ("down", 4096, 14336)], [1, 8, 32, 128, 512], "bf16", True,
                        1.0, 0.003, 0.015) + ("bf16",)
    if cfg == 3:
        return ("GPTQ W4A16 fp16 Qwen-32B-like (25600x5120)+(5120x25600) M in {2048,4096,8192}",) + w4a16_cases(
            ops, L, 3, [("up", 25600, 5120), ("down", 5120, 25600)], [2048, 4096, 8192], "f16", False, 0.5, 0.002,
            0.01) + ("f16",)
    if cfg == 4:
        return ("blockwise FP8 DeepSeek-V3 dense MLP (18432x7168)+(7168x18432) M in {1,16,128,1024,4096}",) + \
            fp8_cases(ops, L, 4, [("up", 18432, 7168), ("down", 7168, 18432)], [1, 16, 128, 1024, 4096]) + ("fp8",)
    if cfg == 5:
        return ("DeepSeek-V3 MoE int4 bf16 E=256 top-8 T in {1,64,512,4096}",) + moe_cases(
            ops, L, 5, [1, 64, 512, 4096]) + ("bf16",)
    if cfg == 6:  # not one of the reference's five benchmark configurations: the block-fp8 expert path, same shapes as 5
        return ("DeepSeek-V3 MoE block-fp8 bf16 E=256 top-8 T in {1,64,512,4096}",) + moe_fp8_cases(
            ops, L, 6, [1, 64, 512, 4096]) + ("fp8",)
    if cfg == 7:  # not one of the reference's five benchmark configurations: the W4A8 path on the shapes of the
        # reference's own performance test (finegrained_mixed_dtype_gemm_thop_test.cu:312-321) plus decode and prefill
        return ("W4A8 bf16 (5120x5120)+(25600x5120) M in {1,16,64,128,256,4096}",) + w4a8_cases(
            ops, L, 7, [("sq", 5120, 5120), ("up", 25600, 5120)], [1, 16, 64, 128, 256, 4096]) + ("fp8",)
    raise SystemExit("unknown --config %d" % cfg)


# ------------------------------------------------------------------------------------------------ timing
def capture(fns):
    """One HIP graph holding the launches of `fns` in order (captured on a side stream, replayed on the current one)."""
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for f in fns:
            f()
    return g


def time_case(c, use_graph):
    """Average duration of one launch of case c in ms: HIP events around `reps` back-to-back launches on the launch
    stream.  With graphs the launches are replayed from one captured graph, which takes the host's per-launch cost
    (several microseconds from Python) out of the measurement of kernels that run for less than that."""
    reps = 200 if c.t_bound < 2e-5 else (48 if c.t_bound < 2e-4 else 8)
    reps = -(-reps // c.copies) * c.copies          # whole turns of the weight-copy rotation
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    if use_graph:
        g = capture([c.launch] * reps)
        g.replay()
        torch.cuda.synchronize()
        start.record()
        g.replay()
        end.record()
    else:
        c.launch()
        torch.cuda.synchronize()
        start.record()
        for _ in range(reps):
            c.launch()
        end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / reps


def cpu_baseline(cfg, keep, ops):
    """The oracle's dequantize-to-fp32 + fp32 GEMM on the host cores: one pass over a bounded sample of the workload."""
    if cfg not in (1, 2) or not keep:
        return None
    import numpy as np
    from oracle import ksq_oracle as orc
    orc.build()
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    prepared = []
    for k in keep:
        tag = orc.BF16 if k["x"][min(k["x"])].dtype == torch.bfloat16 else orc.F16
        if k["awq"]:
            codes = orc.awq_unpack(k["q"].numpy().view(np.uint32))
            zeros = k["zeros"].numpy()
        else:
            codes = orc.gptq_unpack(k["q"].numpy().view(np.uint32))
            zeros = None
        sb = k["scales"].view(torch.int16).numpy().view(np.uint16)
        xs = {M: k["x"][M].cpu().view(torch.int16).numpy().view(np.uint16) for M in sorted(k["x"])}
        prepared.append((k, tag, codes, zeros, sb, xs))
    # whole passes over the workload until at least 10 s of wall time have been spent (30 s cap inside a pass)
    flops, t, passes = 0, 0.0, 0
    while t < 10.0:
        for k, tag, codes, zeros, sb, xs in prepared:
            for M, xb in xs.items():
                t0 = time.perf_counter()
                orc.w4a16_gemm(xb, codes, sb, zeros, 128, tag)
                t += time.perf_counter() - t0
                flops += 2 * M * k["N"] * k["K"]
                if t > 30.0:
                    break
        passes += 1
    names = ", ".join("%s(%dx%d) M in {%s}" % (k["tag"], k["N"], k["K"], ",".join(map(str, xs)))
                      for k, _, _, _, _, xs in prepared)
    return {"value": round(flops / t / 1e12, 6), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": "%d pass(es) of the oracle (dequantize to fp32, fp32 GEMM, OpenMP) over %s" % (passes, names),
            "seconds": round(t, 3)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=2, help="BASELINE.json config number 1..5 (default 2); 6 = block-fp8 MoE, same shapes as 5; 7 = W4A8")
    ap.add_argument("--only", default="", help="substring filter on case names (for profiling one case)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="launch every kernel from Python instead of replaying "
                    "captured HIP graphs (adds the host's per-launch cost to short kernels)")
    ap.add_argument("--calibrate-copy", action="store_true", help="run only a 256 MiB device-to-device copy a few "
                    "times (the known-size kernel hardware traffic counters are scaled by) and exit")
    ap.add_argument("--details", action="store_true", help="also print a per-case table to stderr")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU's throughput; --gpus %d is not supported (this path has no "
                         "multi-GPU leg, every case is already a per-GPU shape)" % args.gpus)
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")

    if args.calibrate_copy:
        n = 256 << 20
        src = torch.randint(0, 255, (n,), dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": n, "copy_bytes_written": n, "launches": 5}))
        return

    from ksanallm_amd import lib as L
    from ksanallm_amd import ops

    workload, cases, keep, dtype = build(args.config, ops, L)
    if args.only:
        cases = [c for c in cases if args.only in c.name]
        if not cases:
            raise SystemExit("--only matched no case")

    use_graph = not args.no_graph
    n_graphs = max(c.copies for c in cases)

    def eager_step(_i=0):
        for c in cases:
            c.launch()

    if use_graph:
        # one captured graph per turn of the weight-copy rotation; step i replays graph i % n_graphs
        eager_step()
        torch.cuda.synchronize()
        graphs = [capture([c.launch for c in cases]) for _ in range(n_graphs)]
        # and one graph that holds a whole turn of the rotation (n_graphs consecutive steps): starting a graph costs
        # 20-30 us, as much as a step of two decode kernels takes; a serving loop replays graphs of hundreds of kernels
        turn = capture([c.launch for c in cases] * n_graphs) if n_graphs > 1 else None

        def step(i):
            graphs[i % n_graphs].replay()
    else:
        step = eager_step
        turn = None

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    done = 0
    while done < args.steps:       # exactly args.steps steps: whole turns while they fit, single steps for the rest
        if turn is not None and args.steps - done >= n_graphs:
            turn.replay()
            done += n_graphs
        else:
            step(args.warmup + done)
            done += 1
    end.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ms_per_step = start.elapsed_time(end) / args.steps

    # per-case kernel timing, same stream, after the timed region
    per_case = []
    for c in cases:
        ms = time_case(c, use_graph)
        sec = ms * 1e-3
        per_case.append({
            "case": c.name, "kernel": c.kernel, "us": round(ms * 1e3, 2), "tflops": round(c.flops / sec / 1e12, 3),
            "gbps": round(c.bytes / sec / 1e9, 1), "bound": c.bound,
            "frac": round(c.t_bound / sec, 4),
        })
    total_bound = sum(c.t_bound for c in cases)
    total_flops = sum(c.flops for c in cases)
    total_bytes = sum(c.bytes for c in cases)
    step_s = ms_per_step * 1e-3

    # dominant kernel = the kernel variant with the largest share of the step; its launches average over the cases
    # that run it, which is also what a profiler's per-kernel average shows
    groups = {}
    for c, p in zip(cases, per_case):
        g = groups.setdefault(c.kernel, {"us": 0.0, "flops": 0, "bytes": 0, "t_hbm": 0.0, "t_mfma": 0.0, "n": 0,
                                         "peak_key": c.peak_key, "cases": []})
        g["us"] += p["us"]
        g["flops"] += c.flops
        g["bytes"] += c.bytes
        g["t_hbm"] += c.bytes / HBM_PEAK
        g["t_mfma"] += c.flops / MFMA_PEAK[c.peak_key]
        g["n"] += 1
        g["cases"].append(c.name)
    dk = max(groups, key=lambda k: groups[k]["us"])
    g = groups[dk]
    sec = g["us"] * 1e-6
    if g["t_hbm"] >= g["t_mfma"]:
        ach = g["bytes"] / sec / 1e9
        roof = {"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                "frac": round(ach * 1e9 / HBM_PEAK, 4)}
    else:
        ach = g["flops"] / sec / 1e12
        roof = {"bound": "mfma", "achieved": round(ach, 3), "peak": MFMA_PEAK[g["peak_key"]] / 1e12, "unit": "TFLOP/s",
                "frac": round(ach * 1e12 / MFMA_PEAK[g["peak_key"]], 4)}
    traffic = MEASURED_TRAFFIC.get((args.config, dk))
    roof["traffic"] = traffic
    roof["kernel"] = dk
    roof["cases"] = g["cases"]
    roof["avg_launch_us"] = round(g["us"] / g["n"], 2)
    roof["algorithmic_bytes_per_launch"] = g["bytes"] // g["n"]
    roof["algorithmic_flops_per_launch"] = g["flops"] // g["n"]

    out = {
        "metric": METRIC, "value": round(100.0 * total_bound / step_s, 3), "unit": "% of roofline",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": "synthetic",
        "config": {"workload": workload, "cases": len(cases), "config_index": args.config - 1},
        "tflops": round(total_flops / step_s / 1e12, 3), "hbm_gbps": round(total_bytes / step_s / 1e9, 1),
        "wall_ms_per_step": round(wall_ms, 5), "launch": "hip graph replay" if use_graph else "python launches",
        "steps_per_graph": (n_graphs if turn is not None and args.steps >= n_graphs else 1),
        "peaks": {"hbm_gbps": HBM_PEAK / 1e9, "mfma_tflops": {k: v / 1e12 for k, v in MFMA_PEAK.items()}},
        "roofline": roof, "per_case": per_case,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args.config, keep, ops)
    if args.details:
        for p in per_case:
            print("%-28s %-20s %10.2f us %9.3f TFLOP/s %9.1f GB/s  %s %.1f%%" % (
                p["case"], p["kernel"], p["us"], p["tflops"], p["gbps"], p["bound"], 100 * p["frac"]), file=sys.stderr)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
