#!/usr/bin/env python3
"""Benchmark of the quantized-GEMM hot path on one MI355X.

One "step" is one pass over every (shape, M) case of the chosen workload with synthetic inputs already resident in
HBM.  The default workload is the whole metric: the five benchmark configurations (GPTQ fp16 4096^2 decode, AWQ bf16
Llama-3-8B MLP M = 1..512, GPTQ fp16 Qwen-32B-like prefill M = 2048..8192, blockwise-FP8 DeepSeek-V3 MLP M = 1..4096,
DeepSeek-V3 int4 MoE block T = 1..4096) in one process and one JSON line; `--config N` runs one of them (6 and 7 are
the block-fp8 MoE block and W4A8, which are not among the five).  Weight copies are rotated so that no launch finds
its weights in the 256 MB Infinity Cache.

Prints ONE JSON line.  `value` is the time-weighted fraction of the MI355X roofline over the step, in percent:
sum over cases of max(bytes / 8 TB/s, flops / MFMA peak) divided by the measured step time.

Side measurements, none a benchmark figure: `--library-gemm` times the vendor library's plain GEMMs at the
prefill shapes, `--constant-data` gives every operand of the dense cases one value (the same kernels and cycle
counts at the clock that operands which never toggle allow), and `--mfma-stream` times bare streams of the matrix
instructions on operands held in registers (what the matrix pipes sustain under the part's power limit with no kernel
around them).
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


def measured_traffic(kernel):
    """HBM bytes per launch of a kernel variant (fetched + written), from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
    runs whose totals are kept in profiles/traffic.json (each counter scaled by what it reads for a 256 MiB device copy,
    `--calibrate-copy`); None when no counter run covers the variant."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        table = json.load(f)
    row = table.get("kernels", {}).get(kernel)
    return None if row is None else int(row["fetch_bytes"] + row["write_bytes"])


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
    def __init__(self, name, launch, flops, nbytes, peak_key, kernel, copies=1, kind="", m=0):
        self.name, self.launch, self.flops, self.bytes, self.peak_key, self.kernel = name, launch, flops, nbytes, peak_key, kernel
        self.copies = copies
        self.kind, self.m = kind, m        # kind: "int4" | "fp8" | "fp8_quant" | "moe_int4" | ...; m: rows / tokens
        t_hbm = nbytes / HBM_PEAK
        t_mfma = flops / MFMA_PEAK[peak_key]
        self.bound = "hbm" if t_hbm >= t_mfma else "mfma"
        self.t_bound = max(t_hbm, t_mfma)


def copies_needed(weight_bytes):
    return max(2, min(64, -(-CACHE_BYTES // weight_bytes) + 1))


def kernel_label(L, kind, prefix, M, N, K, dt):
    d = L.select_tile(kind, M, N, K, dt)
    return "%s<%dx%d,w%d>" % (prefix + ("_splitk_kernel" if d["kernel"] == 0 else "_tile_kernel"),
                              d["block_m"], d["block_n"], d["waves"])


# ------------------------------------------------------------------------------------------------ workloads
CONSTANT_DATA = ""   # --constant-data: "all", "weights" or "activations" hold one value each (configs 1-4)
FP8_SHAPE = None     # --fp8-shape M,N,K: config 4 becomes one GEMM of that shape


def w4a16_cases(ops, L, cfg, shapes, Ms, dtype, awq, x_std, s_lo, s_hi):
    dev = "cuda"
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    ldt = L.F16 if dtype == "f16" else L.BF16
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
        if CONSTANT_DATA in ("all", "weights"):   # the same instructions on operands that never toggle
            q = torch.full_like(q, 0x11111111 * 9 - 2**32)   # every code 9
            scales = torch.full_like(scales, (s_lo + s_hi) / 2)
        wp1 = ops.repack_weight(q.to(dev), layout, 1, K, N)
        sp1 = ops.repack_scales(scales.to(dev), L.SCALE_GN, 1, K, N, 128)
        zp1 = ops.repack_zeros(awq_pack_cols(zeros).to(dev), L.ZERO_AWQ_PACKED, K, N, 128) if awq else None
        R = max(copies_needed(wp1.numel()), len(Ms))
        wps = [wp1] + [wp1.clone() for _ in range(R - 1)]
        sps = [sp1] + [sp1.clone() for _ in range(R - 1)]
        zps = [zp1] + [zp1.clone() for _ in range(R - 1)] if awq else [None] * R
        state = {"i": 0}
        rec = dict(kind="w4a16", q=q, scales=scales, zeros=zeros, N=N, K=K, tag=tag, awq=awq, x={}, y={},
                   packed=(wps[0], sps[0], zps[0]))
        keep.append(rec)
        for mi, M in enumerate(Ms):
            x = (torch.randn((M, K), generator=seeded(cfg, 100 * si + mi + 10)) * x_std).to(tdt).to(dev)
            if CONSTANT_DATA in ("all", "activations"):
                x = torch.full_like(x, x_std)
            y = torch.empty((M, N), dtype=tdt, device=dev)
            rec["x"][M], rec["y"][M] = x, y
            need = L.load().ksq_w4a16_workspace_size(M, N, K, 128, ldt)
            ws = torch.empty(need, dtype=torch.uint8, device=dev) if need else None

            def launch(x=x, y=y, N=N, K=K, wps=wps, sps=sps, zps=zps, state=state, R=R, ws=ws):
                i = state["i"] = (state["i"] + 1) % R
                ops.w4a16_gemm(x, wps[i], sps[i], zps[i], N, K, 128, out=y, workspace=ws)

            nbytes = K * N // 2 + G * N * 2 + (G * N // 2 if awq else 0) + 2 * M * K + 2 * M * N
            cases.append(Case("%s:M=%d" % (tag, M), launch, 2 * M * N * K, nbytes, dtype,
                              kernel_label(L, L.KIND_W4A16, "w4a16", M, N, K, ldt), R, "int4", M))
    return cases, keep


def fp8_cases(ops, L, cfg, shapes, Ms):
    dev = "cuda"
    cases, keep = [], []
    for si, (tag, N, K) in enumerate(shapes):
        g = seeded(cfg, si)
        # e4m3 codes of bf16 N(0,0.02^2) weights under a per-128x128 amax/448 scale: drawn directly as the codes of
        # w/s with w/s ~ N(0, (448/4.2)^2) clipped to +-448 (amax of 16384 normals is about 4.2 sigma)
        wn = (torch.randn((N, K), generator=g) * (448.0 / 4.2)).clamp_(-448, 448)
        if CONSTANT_DATA in ("all", "weights"):
            wn.fill_(112.0)
        b = wn.to(torch.float8_e4m3fn).view(torch.uint8)
        del wn
        b_s = torch.full(((N + 127) // 128, K // 128), 0.02 * 4.2 / 448.0, dtype=torch.float32)
        R = max(copies_needed(b.numel()), len(Ms))
        bs_ = [ops.fp8_repack_weight(b.to(dev))]   # the load-time repack into 2 KiB MFMA fragments
        bs_ += [bs_[0].clone() for _ in range(R - 1)]
        b_sd = b_s.to(dev)
        state = {"i": 0}
        rec = dict(kind="fp8", b=b, b_s=b_s, N=N, K=K, tag=tag, x={}, y={}, a_q={}, a_s={}, packed=(bs_[0], b_sd))
        keep.append(rec)
        for mi, M in enumerate(Ms):
            gx = seeded(cfg, 100 * si + mi + 10)
            x = torch.randn((M, K), generator=gx)
            x = torch.where(torch.rand((M, K), generator=gx) < 0.01, x * 20, x).to(torch.bfloat16).to(dev)
            if CONSTANT_DATA in ("all", "activations"):
                x = torch.full_like(x, 1.0)
            a_q = torch.empty((M, K), dtype=torch.uint8, device=dev)
            a_s = torch.empty((K // 128, M), dtype=torch.float32, device=dev)
            y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
            rec["x"][M], rec["y"][M], rec["a_q"][M], rec["a_s"][M] = x, y, a_q, a_s

            def quant(x=x, a_q=a_q, a_s=a_s, K=K):
                ops.per_token_group_quant_fp8(x, K, 128, True, False, q=a_q, s=a_s)

            need = L.load().ksq_fp8_blockwise_workspace_size(M, N, K)
            ws = torch.empty(need, dtype=torch.uint8, device=dev) if need else None

            def gemm(a_q=a_q, a_s=a_s, y=y, bs_=bs_, b_sd=b_sd, state=state, R=R, ws=ws):
                i = state["i"] = (state["i"] + 1) % R
                ops.fp8_blockwise_gemm(a_q, a_s, bs_[i], b_sd, out=y, workspace=ws)

            quant()
            cases.append(Case("%s:quant:M=%d" % (tag, M), quant, 0, 2 * M * K + M * K + 4 * M * K // 128, "fp8",
                              "fp8_group_quant", 1, "fp8_quant", M))
            nbytes = N * K + b_s.numel() * 4 + M * K + 4 * M * K // 128 + 2 * M * N
            cases.append(Case("%s:gemm:M=%d" % (tag, M), gemm, 2 * M * N * K, nbytes, "fp8",
                              kernel_label(L, L.KIND_FP8_BLOCKWISE, "fp8", M, N, K, L.BF16), R, "fp8", M))
    return cases, keep


def w4a8_cases(ops, L, cfg, shapes, Ms):
    """W4A8: static per-tensor e4m3 quantization of bf16 activations (with the group sums the GEMM needs), then int4
    weights x e4m3 activations on the fp8 matrix instruction."""
    dev = "cuda"
    cases = []
    for si, (tag, N, K) in enumerate(shapes):
        g = seeded(cfg, si)
        w = torch.randint(0, 256, (K, N // 2), generator=g, dtype=torch.uint8)
        scales = (torch.rand((K // 128, N), generator=g) * 0.012 + 0.003).to(torch.float16)
        wp1 = ops.w4a8_repack_weight(w.to(dev))
        R = max(copies_needed(wp1.numel()), len(Ms))
        wps = [wp1] + [wp1.clone() for _ in range(R - 1)]
        sc_d = scales.to(dev)
        in_scale = torch.tensor([0.05], dtype=torch.float32, device=dev)
        state = {"i": 0}
        for mi, M in enumerate(Ms):
            gx = seeded(cfg, 100 * si + mi + 10)
            x = torch.randn((M, K), generator=gx)
            x = torch.where(torch.rand((M, K), generator=gx) < 0.01, x * 20, x).to(torch.bfloat16).to(dev)
            if CONSTANT_DATA in ("all", "activations"):
                x = torch.full_like(x, 1.0)
            a_q = torch.empty((M, K), dtype=torch.uint8, device=dev)
            xsum = torch.empty((K // 128, M), dtype=torch.float32, device=dev)
            y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)

            def quant(x=x, a_q=a_q, xsum=xsum, M=M, K=K, in_scale=in_scale):
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
                              "w4a8_quant", 1, "w4a8_quant", M))
            nbytes = N * K // 2 + (K // 128) * N * 2 + M * K + 4 * M * K // 128 + 2 * M * N
            cases.append(Case("%s:gemm:M=%d" % (tag, M), gemm, 2 * M * N * K, nbytes, "fp8",
                              kernel_label(L, L.KIND_W4A8, "w4a8", M, N, K, L.BF16), R, "w4a8", M))
    return cases, []


def routing_variants(ids, E, touched_bytes):
    """Expert-id sets a MoE case alternates between.  With few tokens the touched experts fit into the 256 MB Infinity
    Cache, and replaying the same ids would time the cache, not HBM: such a case rotates through shifted copies of its
    ids (expert e -> (e + j*E/R) mod E) so that more than the cache holds passes before a set comes round again."""
    R = 1 if touched_bytes > CACHE_BYTES else min(8, -(-CACHE_BYTES // touched_bytes) + 1)
    return [((ids + j * (E // R)) % E).contiguous() for j in range(R)]


def moe_cases(ops, L, cfg, Ts, E=256, hidden=7168, inter=2048, topk=8, distinct=32):
    dev = "cuda"
    g = seeded(cfg, 0)
    tdt = torch.bfloat16
    # `distinct` independent expert slabs tiled to E experts (expert e holds slab e % distinct): 5.8 GB of device
    # weights either way
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
    rec = dict(kind="moe", w13=w13, w2=w2, s13=s13, s2=s2, distinct=distinct, E=E, hidden=hidden, inter=inter, topk=topk,
               x={}, ids={}, tw={}, out={})
    cases = []
    for ti, T in enumerate(Ts):
        gx = seeded(cfg, 10 + ti)
        x = torch.randn((T, hidden), generator=gx).to(tdt)
        logits = torch.randn((T, E), generator=gx)
        tw, ids = torch.topk(torch.softmax(logits, -1), topk, dim=-1)
        touched = int(torch.unique(ids).numel())
        ids = ids.to(torch.int32)
        rec["x"][T], rec["ids"][T], rec["tw"][T] = x, ids, tw.float().contiguous()
        x_d, tw_d = x.to(dev), tw.float().contiguous().to(dev)
        variants = [v.to(dev) for v in routing_variants(ids, E, per_expert * touched)]
        state = {"i": -1}
        holder = rec["out"]

        def launch(x_d=x_d, variants=variants, tw_d=tw_d, state=state, holder=holder, T=T):
            i = state["i"] = (state["i"] + 1) % len(variants)
            out = ops.fused_moe_w4a16(x_d, w13p, s13p, w2p, s2p, variants[i], tw_d, E, hidden, inter, 128)
            if i == 0:
                holder[T] = out

        nbytes = per_expert * touched + 2 * T * hidden * 2 + 64 * T
        flops = 2 * T * topk * (2 * inter * hidden + hidden * inter)
        cases.append(Case("moe:T=%d" % T, launch, flops, nbytes, "bf16", "moe_w4a16 block (align + 2 grouped GEMMs + sum)",
                          len(variants), "moe_int4", T))
    return cases, [rec]


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
        tw_d = tw.float().contiguous().to(dev)
        variants = [v.to(dev) for v in routing_variants(ids.to(torch.int32), E, per_expert * touched)]
        state = {"i": -1}

        def launch(x=x, variants=variants, tw_d=tw_d, state=state):
            i = state["i"] = (state["i"] + 1) % len(variants)
            ops.fused_moe_fp8_blockwise(x, w13, s13, w2, s2, variants[i], tw_d)

        nbytes = per_expert * touched + 2 * T * hidden * 2 + 64 * T
        flops = 2 * T * topk * (2 * inter * hidden + hidden * inter)
        cases.append(Case("moe_fp8:T=%d" % T, launch, flops, nbytes, "fp8",
                          "moe_fp8_blockwise block (quant + align + 2 grouped GEMMs + sum)", len(variants), "moe_fp8", T))
    return cases, []


WORKLOADS = {
    1: "GPTQ W4A16 fp16 N=K=4096 M in {1,16}",
    2: "AWQ W4A16 bf16 Llama-3-8B MLP gate/up(14336x4096)+down(4096x14336) M in {1,8,32,128,512}",
    3: "GPTQ W4A16 fp16 Qwen-32B-like (25600x5120)+(5120x25600) M in {2048,4096,8192}",
    4: "blockwise FP8 DeepSeek-V3 dense MLP (18432x7168)+(7168x18432) M in {1,16,128,1024,4096}",
    5: "DeepSeek-V3 MoE int4 bf16 E=256 top-8 T in {1,64,512,4096}",
    6: "DeepSeek-V3 MoE block-fp8 bf16 E=256 top-8 T in {1,64,512,4096}",
    7: "W4A8 bf16 (5120x5120)+(25600x5120) M in {1,16,64,128,256,4096}",
    8: "W4A16 decode on large weights: GPTQ bf16 (57344x8192), AWQ bf16 (28672x8192), GPTQ fp16 (25600x5120) M in {1,8,16}",
    9: "small problems of 64..512 rows: W4A16 fp16 (4096x4096)+(5120x5120), blockwise FP8 (4096x4096)+(2048x7168), "
       "W4A8 (4096x4096)+(5120x5120), M in {64,128,256,512}",
}
DTYPES = {1: "f16", 2: "bf16", 3: "f16", 4: "fp8", 5: "bf16", 6: "fp8", 7: "fp8", 8: "bf16", 9: "f16"}


def build(cfg, ops, L):
    """(cases, keep) of one configuration."""
    if cfg == 1:
        return w4a16_cases(ops, L, 1, [("q_proj", 4096, 4096)], [1, 16], "f16", False, 1.0, 0.004, 0.02)
    if cfg == 2:
        return w4a16_cases(ops, L, 2, [("gate_up", 14336, 4096), ("down", 4096, 14336)], [1, 8, 32, 128, 512], "bf16", True,
                           1.0, 0.003, 0.015)
    if cfg == 3:
        return w4a16_cases(ops, L, 3, [("up", 25600, 5120), ("down", 5120, 25600)], [2048, 4096, 8192], "f16", False, 0.5,
                           0.002, 0.01)
    if cfg == 4:
        if FP8_SHAPE:   # --fp8-shape: one GEMM of a shape of the caller's choice (clock and tile-count experiments)
            m, n, k = FP8_SHAPE
            return fp8_cases(ops, L, 4, [("shape", n, k)], [m])
        return fp8_cases(ops, L, 4, [("up", 18432, 7168), ("down", 7168, 18432)], [1, 16, 128, 1024, 4096])
    if cfg == 5:
        return moe_cases(ops, L, 5, [1, 64, 512, 4096])
    if cfg == 6:  # not one of the five benchmark configurations: the block-fp8 expert path, same shapes as 5
        return moe_fp8_cases(ops, L, 6, [1, 64, 512, 4096])
    if cfg == 7:  # not one of the five benchmark configurations: the W4A8 path on the shapes of the reference's own
        # performance test (finegrained_mixed_dtype_gemm_thop_test.cu:312-321) plus decode and prefill
        return w4a8_cases(ops, L, 7, [("sq", 5120, 5120), ("up", 25600, 5120)], [1, 16, 64, 128, 256, 4096])
    if cfg == 8:  # not one of the five benchmark configurations: the decode kernel where a launch moves 64 MB and more
        a, ka = w4a16_cases(ops, L, 8, [("wide", 57344, 8192)], [1, 8, 16], "bf16", False, 1.0, 0.004, 0.02)
        b, kb = w4a16_cases(ops, L, 8, [("awq", 28672, 8192)], [1, 8, 16], "bf16", True, 1.0, 0.003, 0.015)
        c, kc = w4a16_cases(ops, L, 8, [("up", 25600, 5120)], [1, 8, 16], "f16", False, 1.0, 0.004, 0.02)
        for x in c:
            x.peak_key = "f16"
        return a + b + c, ka + kb + kc
    if cfg == 9:  # not one of the five benchmark configurations: projections of smaller models at 64..512 rows, where the
        # decode-form kernels over 32-row blocks run instead of the tile kernels (--tile-kernels: the tile kernels)
        Ms = [64, 128, 256, 512]
        a, ka = w4a16_cases(ops, L, 9, [("w4a16_4096", 4096, 4096), ("w4a16_5120", 5120, 5120)], Ms, "f16", False, 1.0, 0.004, 0.02)
        b, kb = fp8_cases(ops, L, 9, [("fp8_4096", 4096, 4096), ("fp8_2048x7168", 2048, 7168)], Ms)
        c, kc = w4a8_cases(ops, L, 9, [("w4a8_4096", 4096, 4096), ("w4a8_5120", 5120, 5120)], Ms)
        return a + b + c, ka + kb + kc
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


def sample_clock(c, seconds):
    """Launches case c back to back for `seconds` while a thread reads the shader clock from rocm-smi every 50 ms:
    the clock the power management grants this kernel on this data, and the launch time at that clock."""
    import re
    import subprocess
    import threading
    samples, stop = [], []

    def reader():
        while not stop:
            try:
                out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=5).stdout
                samples.extend(int(m) for m in re.findall(r"sclk clock level: \d+: \((\d+)Mhz\)", out))
            except Exception:
                pass
            time.sleep(0.05)

    for _ in range(3):
        c.launch()
    torch.cuda.synchronize()
    th = threading.Thread(target=reader)
    th.start()
    beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    n, t0 = 0, time.time()
    beg.record()
    while time.time() - t0 < seconds:
        for _ in range(10):
            c.launch()
        torch.cuda.synchronize()
        n += 10
    end.record()
    torch.cuda.synchronize()
    stop.append(1)
    th.join()
    row = {"case": c.name, "kernel": c.kernel, "us": round(beg.elapsed_time(end) / n * 1e3, 2), "launches": n,
           "sclk_samples": len(samples)}
    if samples:
        row.update(sclk_mhz_mean=round(sum(samples) / len(samples), 1), sclk_mhz_min=min(samples), sclk_mhz_max=max(samples))
    return row


# ------------------------------------------------------------------------------------------------ CPU baseline
def _bits(t):
    import numpy as np
    return t.contiguous().cpu().view(torch.int16).numpy().view(np.uint16)


def _err(y_gpu, ref, limit=None, y32=None):
    """Raw rel-L2 and max-abs of a GPU result against the oracle's fp32 values; `ok` is the rel-L2 bar plus a finite
    result.  y32: the same call's sums before they were rounded to the output type (the fp32 entry points), whose
    max-abs is the figure the 2e-2 of the parity bar can be held against (half a unit in the last place of bf16 is
    0.031 from |y| = 8 on)."""
    import numpy as np
    limit = REL_L2_MAX if limit is None else limit
    y = y_gpu.float().cpu().numpy()
    assert y.shape == ref.shape, (y.shape, ref.shape)
    d = y - ref
    rel = float(np.linalg.norm(d) / max(np.linalg.norm(ref), 1e-30))
    out = {"rel_l2": rel, "max_abs": float(np.abs(d).max()), "max_ref": float(np.abs(ref).max()),
           "rel_l2_limit": round(limit, 6), "ok": bool(np.all(np.isfinite(y)) and rel <= limit)}
    if y32 is not None:
        out["max_abs_before_rounding"] = float(np.abs(y32.cpu().numpy() - ref).max())
    return out


REL_L2_MAX = 5e-3          # the parity bar of a GEMM against the fp32-accumulated dequantize-then-GEMM reference


def cpu_baseline(keeps, L, ops):
    """The oracle's dequantize-to-fp32 + fp32 GEMM on the host cores over a bounded sample of every case (all rows of a
    decode case, the first 128 rows of a prefill case, the first 4 tokens of a MoE block: about ten seconds of host
    work in all), timed, and held against what the GPU left in its output buffers for the same inputs: the raw figures
    of the parity bar (rel-L2, max-abs against the fp32 reference) appear beside the timing, every row with the limit
    it is held to (`ok`)."""
    import numpy as np
    from oracle import ksq_oracle as orc
    orc.build()
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    per_config, accuracy = [], []
    tot_flops, tot_t = 0, 0.0
    for cfg in sorted(keeps):
        flops, t, sample = 0, 0.0, []
        for k in keeps[cfg]:
            if k["kind"] == "w4a16":
                tdt = k["x"][min(k["x"])].dtype
                tag = orc.BF16 if tdt == torch.bfloat16 else orc.F16
                codes = orc.awq_unpack(k["q"].numpy().view(np.uint32)) if k["awq"] else orc.gptq_unpack(k["q"].numpy().view(np.uint32))
                zeros = k["zeros"].numpy() if k["awq"] else None
                sb = _bits(k["scales"])
                for M in sorted(k["x"]):
                    rows = min(M, 128)          # prefill cases: the first 128 rows of x
                    xb = _bits(k["x"][M][:rows])
                    t0 = time.perf_counter()
                    ref = orc.w4a16_gemm(xb, codes, sb, zeros, 128, tag)
                    t += time.perf_counter() - t0
                    flops += 2 * rows * k["N"] * k["K"]
                    sample.append("%s:M=%d%s" % (k["tag"], M, "" if rows == M else "[rows 0..%d]" % (rows - 1)))
                    wp, sp, zp = k["packed"]
                    y32 = ops.w4a16_gemm_f32(k["x"][M], wp, sp, zp, k["N"], k["K"], 128)[:rows]
                    accuracy.append(dict(case="c%d/%s:M=%d" % (cfg, k["tag"], M), rows=rows, **_err(k["y"][M][:rows], ref, y32=y32)))
            elif k["kind"] == "fp8":
                bq, b_s = k["b"].numpy(), k["b_s"].numpy()
                for M in sorted(k["x"]):
                    rows = min(M, 128)          # prefill cases: the first 128 rows (the quantizer works row by row)
                    xb = _bits(k["x"][M][:rows])
                    t0 = time.perf_counter()
                    qo, so = orc.fp8_group_quant(xb, k["K"], 128, True, False, orc.BF16)
                    ref = orc.fp8_blockwise_gemm(qo, so, bq, b_s, True)
                    t += time.perf_counter() - t0
                    flops += 2 * rows * k["N"] * k["K"]
                    sample.append("%s:M=%d%s" % (k["tag"], M, "" if rows == M else "[rows 0..%d]" % (rows - 1)))
                    e = _err(k["y"][M][:rows], ref, y32=ops.fp8_blockwise_gemm_f32(k["a_q"][M], k["a_s"][M], *k["packed"])[:rows])
                    e["quantizer_bits_equal"] = bool(np.array_equal(k["a_q"][M][:rows].cpu().numpy(), qo) and
                                                     np.array_equal(k["a_s"][M][:, :rows].cpu().numpy(), so))
                    accuracy.append(dict(case="c%d/%s:gemm:M=%d" % (cfg, k["tag"], M), rows=rows, **e))
            elif k["kind"] == "moe":
                d = k["distinct"]
                w13, w2 = k["w13"].numpy(), k["w2"].numpy()
                s13, s2 = _bits(k["s13"]), _bits(k["s2"])
                for T in sorted(k["x"]):
                    rows = min(T, 4)            # per-expert dequantization dominates: a few tokens already touch 30 experts
                    ids = (k["ids"][T][:rows] % d).contiguous().numpy().astype(np.int32)   # expert e holds slab e % distinct
                    # a few tokens run the second GEMM with the sum over top-k in it (fp32, rounded once): held against
                    # the same sum in fp32; otherwise every expert's share is rounded to T and summed in T, as the
                    # reference's kernels do
                    few = T <= ops.FEW_TOKENS
                    t0 = time.perf_counter()
                    ref = orc.moe_forward(_bits(k["x"][T][:rows]), w13, s13, w2, s2, ids, k["tw"][T][:rows].numpy(), 128, orc.BF16,
                                          sum_fp32=few)
                    t += time.perf_counter() - t0
                    flops += 2 * rows * k["topk"] * 3 * k["hidden"] * k["inter"]
                    sample.append("moe:T=%d%s" % (T, "" if rows == T else "[tokens 0..%d]" % (rows - 1)))
                    if T in k["out"]:
                        # the oracle hands back the block's output as bit patterns of T, like the kernel's buffer
                        ref_f = ref if few else orc.from_bits(np.asarray(ref).reshape(rows, -1), orc.BF16)
                        # two GEMMs in a row: where both run on the tile kernel, which rounds every dequantized weight
                        # to T, two independent rounding errors compound
                        tiled = L.load().ksq_moe_block_m(T * k["topk"], k["E"]) >= 128
                        accuracy.append(dict(case="c%d/moe:T=%d" % (cfg, T), rows=rows,
                                             **_err(k["out"][T][:rows], ref_f, REL_L2_MAX * (2 ** 0.5 if tiled else 1))))
        if t > 0:
            per_config.append({"config": cfg, "tflops": round(flops / t / 1e12, 6), "seconds": round(t, 3), "sample": ", ".join(sample)})
            tot_flops += flops
            tot_t += t
    if tot_t == 0:
        return None, accuracy
    return ({"value": round(tot_flops / tot_t / 1e12, 6), "unit": "TFLOP/s", "cores": threads, "kind": "port",
             "sample": "the oracle (dequantize to fp32, fp32 GEMM; fp8: quantize + block-scaled GEMM; MoE: per-expert dequantization, "
                       "both GEMMs, silu*mul, weighted sum; OpenMP) on: " +
                       "; ".join("config %d: %s" % (p["config"], p["sample"]) for p in per_config),
             "seconds": round(tot_t, 3), "per_config": per_config}, accuracy)


def library_gemm(steps, warmup):
    """Plain GEMMs of the vendor library at the prefill shapes (context for the roofline fractions, not a product path)."""
    def timed(f):
        for _ in range(warmup):
            f()
        beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        beg.record()
        for _ in range(steps):
            f()
        end.record()
        torch.cuda.synchronize()
        return beg.elapsed_time(end) / steps * 1e3
    rows = []
    for dt, name in ((torch.float16, "fp16"), (torch.bfloat16, "bf16")):
        for n, k in ((25600, 5120), (5120, 25600)):
            for m in (2048, 4096, 8192):
                x = torch.randn(m, k, device="cuda", dtype=dt) * 0.5
                w = torch.randn(n, k, device="cuda", dtype=dt) * 0.01
                if CONSTANT_DATA:
                    x, w = torch.full_like(x, 0.5), torch.full_like(w, 0.005)
                us = timed(lambda: torch.matmul(x, w.t()))
                tf = 2.0 * m * n * k / us / 1e6
                rows.append({"m": m, "n": n, "k": k, "dtype": name, "us": round(us, 1), "tflops": round(tf, 1),
                             "frac": round(tf * 1e12 / MFMA_PEAK["f16"], 3)})
    for n, k in ((18432, 7168), (7168, 18432)):
        for m in (1024, 4096):
            x = torch.randn(m, k, device="cuda").to(torch.float8_e4m3fn)
            w = torch.randn(n, k, device="cuda").to(torch.float8_e4m3fn)
            if CONSTANT_DATA:
                x = torch.full((m, k), 0.5, device="cuda").to(torch.float8_e4m3fn)
                w = torch.full((n, k), 0.5, device="cuda").to(torch.float8_e4m3fn)
            for scaling, sa, sb in (("per tensor", torch.ones((), device="cuda"), torch.ones((), device="cuda")),
                                    ("per row", torch.ones(m, 1, device="cuda"), torch.ones(1, n, device="cuda"))):
                us = timed(lambda: torch._scaled_mm(x, w.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16))
                tf = 2.0 * m * n * k / us / 1e6
                rows.append({"m": m, "n": n, "k": k, "dtype": "e4m3, scales " + scaling, "us": round(us, 1),
                             "tflops": round(tf, 1), "frac": round(tf * 1e12 / MFMA_PEAK["fp8"], 3)})
    for r in rows:
        print("%5d x %5d x %5d  %-22s %9.1f us %8.1f TFLOP/s  %5.1f %% of peak" %
              (r["m"], r["n"], r["k"], r["dtype"], r["us"], r["tflops"], 100 * r["frac"]), file=sys.stderr)
    print(json.dumps({"library_gemm": rows}))


def mfma_stream(iters=6000, launches=200):
    """Bare MFMA streams (ksq_diag_mfma_stream), 2 wavefronts per SIMD on all 256 CUs, launches of about 3 ms timed
    back to back for about 0.6 s: TFLOP/s on operands with random bits and on operands that are all one value."""
    from ksanallm_amd import lib as L
    lib = L.load()
    kinds = [(0, "v_mfma_f32_16x16x32_f16", "f16"), (1, "v_mfma_f32_16x16x32_bf16", "bf16"),
             (2, "v_mfma_scale_f32_16x16x128_f8f6f4 (e4m3)", "fp8"), (3, "v_mfma_f32_32x32x16_f16", "f16"),
             (4, "v_mfma_f32_32x32x16_bf16", "bf16"), (5, "v_mfma_scale_f32_32x32x64_f8f6f4 (e4m3)", "fp8")]
    sink = torch.zeros(256 * 512, dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    rows = []
    for kind, name, dt in kinds:
        row = {"instruction": name, "peak_tflops": MFMA_PEAK[dt] / 1e12}
        for constant in (0, 1):
            L.check(lib.ksq_diag_mfma_stream(kind, constant, 200, sink.data_ptr(), stream))
            torch.cuda.synchronize()
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            for _ in range(launches):
                L.check(lib.ksq_diag_mfma_stream(kind, constant, iters, sink.data_ptr(), stream))
            e.record()
            torch.cuda.synchronize()
            ms = s.elapsed_time(e) / launches
            row["constant_tflops" if constant else "random_tflops"] = round(lib.ksq_diag_mfma_stream_flops(kind, iters) / ms / 1e9, 1)
            row["constant_ms" if constant else "random_ms"] = round(ms, 3)
        row["random_frac_of_peak"] = round(row["random_tflops"] / row["peak_tflops"], 4)
        rows.append(row)
        print("%-44s random operands %7.1f TFLOP/s (%.1f %% of %g)   constant operands %7.1f TFLOP/s" % (
            name, row["random_tflops"], 100 * row["random_frac_of_peak"], row["peak_tflops"], row["constant_tflops"]),
            file=sys.stderr)
    print(json.dumps({"mfma_stream": rows, "wavefronts_per_simd": 2, "launch_iters": iters, "launches": launches}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="all", help="'all' (default): the five benchmark configurations 1..5 in one "
                    "step; or one number: 1..5, 6 = block-fp8 MoE on the shapes of 5, 7 = W4A8, 8 = W4A16 decode on large weights, "
                    "9 = small problems of 64..512 rows in the three formats")
    ap.add_argument("--only", default="", help="substring filter on case names (for profiling one case)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="launch every kernel from Python instead of replaying "
                    "captured HIP graphs (adds the host's per-launch cost to short kernels)")
    ap.add_argument("--calibrate-copy", action="store_true", help="run only a 256 MiB device-to-device copy a few "
                    "times (the known-size kernel hardware traffic counters are scaled by) and exit")
    ap.add_argument("--details", action="store_true", help="also print a per-case table to stderr")
    ap.add_argument("--constant-data", nargs="?", const="all", default="", choices=["all", "weights", "activations"],
                    help="dense W4A16 and block-fp8 cases: every weight code and scale, every activation, or both (the "
                    "default) hold one value (a valid GEMM on operands that never toggle), to show how much of the "
                    "kernel's time is the clock the data allows; not a benchmark figure")
    ap.add_argument("--fp8-shape", default="", help="M,N,K: configuration 4 becomes one blockwise-FP8 GEMM of that shape "
                    "(a side measurement, e.g. tile counts that fill all CUs or three quarters of them)")
    ap.add_argument("--sample-clock", type=float, default=0.0, metavar="SECONDS", help="instead of the benchmark: loop "
                    "every selected case for that long while reading the shader clock from rocm-smi every 50 ms, and "
                    "print launch time and clock per case (what the power management grants the kernel on this data)")
    ap.add_argument("--tile-kernels", action="store_true", help="switch the library's small-problem rule off "
                    "(ksq_set_small_problem_rule(0)): every case of more than 32 rows runs the MFMA tile kernel, to time "
                    "it against the decode-form kernel the rule would choose; not a benchmark figure")
    ap.add_argument("--mfma-stream", action="store_true", help="run only streams of independent MFMAs on register "
                    "operands (the library's ksq_diag_mfma_stream: no memory traffic, no LDS, no other arithmetic), on "
                    "random and on constant operands, and exit: the rate the matrix pipes sustain under the power limit")
    ap.add_argument("--library-gemm", action="store_true", help="run only the vendor library's plain GEMMs (torch.matmul "
                    "fp16 / bf16, torch._scaled_mm e4m3; no dequantization, no block scales) at the prefill shapes of "
                    "configurations 3 and 4 and exit: what a dense GEMM reaches on this part, beside the MFMA peak")
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

    global CONSTANT_DATA, FP8_SHAPE
    CONSTANT_DATA = args.constant_data
    if args.fp8_shape:
        FP8_SHAPE = tuple(int(v) for v in args.fp8_shape.split(","))
    if args.library_gemm:
        library_gemm(args.steps, args.warmup)
        return
    if args.mfma_stream:
        mfma_stream()
        return

    from ksanallm_amd import lib as L
    from ksanallm_amd import ops

    if args.tile_kernels:
        L.set_small_problem_rule(False)
    cfgs = [1, 2, 3, 4, 5] if args.config == "all" else [int(args.config)]
    whole = len(cfgs) > 1
    cases, keeps = [], {}
    for cfg in cfgs:
        cs, keep = build(cfg, ops, L)
        for c in cs:
            c.cfg = cfg
            if whole:
                c.name = "c%d/%s" % (cfg, c.name)
        cases += cs
        keeps[cfg] = keep
    if args.only:
        cases = [c for c in cases if args.only in c.name]
        if not cases:
            raise SystemExit("--only matched no case")

    if args.sample_clock > 0:
        rows = [sample_clock(c, args.sample_clock) for c in cases if c.flops > 0 or not whole]
        for r in rows:
            print("%-28s %-30s %9.1f us  sclk %s MHz (min %s, max %s, %d samples)" % (
                r["case"], r["kernel"][:30], r["us"], r.get("sclk_mhz_mean"), r.get("sclk_mhz_min"), r.get("sclk_mhz_max"),
                r["sclk_samples"]), file=sys.stderr)
        print(json.dumps({"sample_clock_seconds": args.sample_clock, "data": "synthetic, constant %s" % CONSTANT_DATA if
                          CONSTANT_DATA else "synthetic", "rows": rows}))
        return

    use_graph = not args.no_graph
    # one captured graph per turn of the weight-copy rotation; step i replays graph i % n_graphs.  The whole metric
    # moves gigabytes per step, so no weight survives in the Infinity Cache from one step to the next and two graphs do.
    n_graphs = 2 if whole else max(c.copies for c in cases)

    def eager_step(_i=0):
        for c in cases:
            c.launch()

    if use_graph:
        eager_step()
        torch.cuda.synchronize()
        graphs = [capture([c.launch for c in cases]) for _ in range(n_graphs)]
        # and one graph that holds a whole turn of the rotation (n_graphs consecutive steps): starting a graph costs
        # 20-30 us, as much as a step of two decode kernels takes; a serving loop replays graphs of hundreds of kernels
        turn = capture([c.launch for c in cases] * n_graphs) if (n_graphs > 1 and not whole) else None

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
    # that run it, which is also what a profiler's per-kernel average shows.  A MoE block is several kernels, not one:
    # it is left out of this choice unless nothing else runs.
    groups = {}
    for c, p in zip(cases, per_case):
        g = groups.setdefault(c.kernel, {"us": 0.0, "flops": 0, "bytes": 0, "t_hbm": 0.0, "t_mfma": 0.0, "n": 0,
                                         "peak_key": c.peak_key, "cases": [], "block": c.kind.startswith("moe")})
        g["us"] += p["us"]
        g["flops"] += c.flops
        g["bytes"] += c.bytes
        g["t_hbm"] += c.bytes / HBM_PEAK
        g["t_mfma"] += c.flops / MFMA_PEAK[c.peak_key]
        g["n"] += 1
        g["cases"].append(c.name)
    single = [k for k in groups if not groups[k]["block"]] or list(groups)
    dk = max(single, key=lambda k: groups[k]["us"])
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
    roof["traffic"] = measured_traffic(dk)
    roof["kernel"] = dk
    roof["cases"] = g["cases"]
    roof["avg_launch_us"] = round(g["us"] / g["n"], 2)
    roof["algorithmic_bytes_per_launch"] = g["bytes"] // g["n"]
    roof["algorithmic_flops_per_launch"] = g["flops"] // g["n"]

    # the two throughput targets of the scope contract, from the per-case rows
    def frac_min(pred):
        rows = [(p["frac"], p["case"]) for c, p in zip(cases, per_case) if pred(c)]
        return (min(rows)[0], [r[1] for r in rows]) if rows else (None, [])

    dec, dec_cases = frac_min(lambda c: c.kind == "int4" and c.m <= 16)
    big = [p["frac"] for c, p in zip(cases, per_case) if c.kind == "int4" and c.m <= 16 and c.bytes >= 64e6]
    moe_dec, moe_dec_cases = frac_min(lambda c: c.kind == "moe_int4" and c.m <= 64)
    pre, pre_cases = frac_min(lambda c: c.kind == "fp8" and c.m >= 2048)
    targets = {
        "int4_decode_hbm_frac_min": dec, "int4_decode_cases": dec_cases, "int4_decode_goal": 0.70,
        "int4_decode_64MB_up_hbm_frac_min": min(big) if big else None,
        "int4_moe_decode_block_hbm_frac_min": moe_dec, "int4_moe_decode_cases": moe_dec_cases,
        "fp8_prefill_mfma_frac_min": pre, "fp8_prefill_cases": pre_cases, "fp8_prefill_goal": 0.60,
    }

    workload = "; ".join("config %d: %s" % (c, WORKLOADS[c]) for c in cfgs) if whole else WORKLOADS[cfgs[0]]
    out = {
        "metric": METRIC, "value": round(100.0 * total_bound / step_s, 3), "unit": "% of roofline",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 / bf16 / fp8-e4m3 by configuration, fp32 accumulation" if whole else DTYPES[cfgs[0]],
        "data": "synthetic, constant %s (--constant-data)" % CONSTANT_DATA if CONSTANT_DATA else "synthetic",
        "config": {"workload": workload, "cases": len(cases), "configs": cfgs,
                   **({"tile_kernels": True} if args.tile_kernels else {})},
        "tflops": round(total_flops / step_s / 1e12, 3), "hbm_gbps": round(total_bytes / step_s / 1e9, 1),
        "wall_ms_per_step": round(wall_ms, 5), "launch": "hip graph replay" if use_graph else "python launches",
        "steps_per_graph": (n_graphs if turn is not None and args.steps >= n_graphs else 1),
        "peaks": {"hbm_gbps": HBM_PEAK / 1e9, "mfma_tflops": {k: v / 1e12 for k, v in MFMA_PEAK.items()}},
        "roofline": roof, "targets": targets, "per_case": per_case,
    }
    if not args.no_cpu and not args.only:
        out["cpu_baseline"], out["accuracy_vs_fp32_reference"] = cpu_baseline(keeps, L, ops)
        out["accuracy_ok"] = bool(out["accuracy_vs_fp32_reference"]) and all(r["ok"] for r in out["accuracy_vs_fp32_reference"])
        if not out["accuracy_ok"]:
            print("ACCURACY: rows beyond their limit: %s" % [r["case"] for r in out["accuracy_vs_fp32_reference"] if not r["ok"]],
                  file=sys.stderr)
    if args.details:
        for p in per_case:
            print("%-30s %-32s %10.2f us %9.3f TFLOP/s %9.1f GB/s  %s %.1f%%" % (
                p["case"], p["kernel"][:32], p["us"], p["tflops"], p["gbps"], p["bound"], 100 * p["frac"]), file=sys.stderr)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
