#!/usr/bin/env python3
"""Benchmark of the MX low-precision linear path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input: for both
grouped linears of an MoE expert layer (fc1 and fc2), forward + backward
through ``ops.grouped_gemm_fp8`` -- i.e. MX quantisation of activations,
weights (2-D blocks, every step, as the reference does when there is a single
microbatch: primus_turbo.py:1094-1103) and output gradients, the forward
grouped GEMM, the dgrad grouped GEMM and the variable-K wgrad grouped GEMM.

Default workload: the Mixtral-8x7B-shape MoE layer (8 experts, top-2, 16384
tokens -> 32768 routed rows, hidden 4096, ffn 14336, gate+up fused 28672),
routing from softmax of Gaussian logits plus a per-expert bias (skewed, ragged
tokens-per-expert).  Inputs are generated with the CPU generator from fixed
seeds (fp32, cast to bf16), uploaded, and resident in HBM before the timed
region; the CPU baseline runs on a row sample of the same tensors.

Prints ONE JSON line:  metric = grouped-GEMM algorithmic TFLOP/s of the whole
step (2*M*N*K per GEMM over all six GEMMs, divided by the wall time of the
step including every quantiser), plus a roofline object for the dominant
kernel and a CPU baseline (the C restatement of the oracle, timed on the host
cores on a 1/16 row sample).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

FP8_PEAK_TFLOPS = 5000.0  # MI355X dense FP8 MFMA
FP4_PEAK_TFLOPS = 10100.0  # MI355X dense FP4 MFMA
BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
HBM_PEAK_GBS = 8000.0  # MI355X HBM3E

WORKLOADS = {
    # name: (experts, top_k, tokens, hidden, fc1_out, fc2_in, routing, seed, fp4)
    "mixtral_8x7b_moe_mxfp8": dict(G=8, topk=2, tokens=16384, hidden=4096, fc1_out=28672, fc2_in=14336, routing="gauss_bias", seed=1003, fp4=False),
    "deepseek_v3_shard_mxfp8": dict(G=32, topk=8, tokens=8192, hidden=7168, fc1_out=4096, fc2_in=2048, routing="zipf", seed=1004, fp4=False),
    "gpt_oss_120b_mxfp4": dict(G=128, topk=4, tokens=16384, hidden=2880, fc1_out=5760, fc2_in=2880, routing="uniform", seed=1005, fp4=True, wgrad=False),
    # the same shapes under the Mixtral workload's routing recipe (Gaussian logits plus a per-expert bias): 16 experts
    # without tokens, 49 with fewer than 16, 11 with more than four times the mean
    "gpt_oss_120b_mxfp4_skewed": dict(G=128, topk=4, tokens=16384, hidden=2880, fc1_out=5760, fc2_in=2880, routing="gauss_bias", seed=1005, fp4=True, wgrad=False),
    # activations with 0.1 % of the entries multiplied by 50 (what moves E8M0 scales and saturates codes)
    "llama3_8b_mlp_mxfp8": dict(G=1, topk=1, tokens=8192, hidden=4096, fc1_out=14336, fc2_in=14336, routing="dense", seed=1002, fp4=False, outliers=True),
    # the pure MXFP4 recipe (E2M1 activations, weights and gradients) on the headline shapes
    "mixtral_8x7b_moe_mxfp4": dict(G=8, topk=2, tokens=16384, hidden=4096, fc1_out=28672, fc2_in=14336, routing="gauss_bias", seed=1003, fp4=True, act_fp4=True),
    # the non-MX "current scaling" recipe on the headline shapes (HYBRID: E4M3 forward, E5M2 gradients)
    "mixtral_8x7b_moe_fp8_tensorwise": dict(G=8, topk=2, tokens=16384, hidden=4096, fc1_out=28672, fc2_in=14336, routing="gauss_bias", seed=1003, fp4=False, tensorwise=True),
    # the 128-blockwise FP8 recipe (1 x 128 activation blocks, 128 x 128 weight blocks, fp32 scales; HYBRID formats) on the Llama MLP
    "llama3_8b_mlp_fp8_blockwise": dict(G=1, topk=1, tokens=8192, hidden=4096, fc1_out=14336, fc2_in=14336, routing="dense", seed=1002, fp4=False, blockwise=True, outliers=True),
    # the same recipe on the headline shapes: grouped forward / dgrad (a row tile per group) and the grouped weight gradient
    "mixtral_8x7b_moe_fp8_blockwise": dict(G=8, topk=2, tokens=16384, hidden=4096, fc1_out=28672, fc2_in=14336, routing="gauss_bias", seed=1003, fp4=False, blockwise=True),
    # the unquantised bf16 grouped GEMM (ops.grouped_gemm: what a layer outside the low-precision autocast runs) on the headline shapes
    "mixtral_8x7b_moe_bf16": dict(G=8, topk=2, tokens=16384, hidden=4096, fc1_out=28672, fc2_in=14336, routing="gauss_bias", seed=1003, fp4=False, bf16=True),
    # the same MLP with the RMSNorm that precedes fc1 in the layer (LayerNormColumnParallelLinear), folded into fc1's quantiser
    "llama3_8b_norm_mlp_mxfp8": dict(G=1, topk=1, tokens=8192, hidden=4096, fc1_out=14336, fc2_in=14336, routing="dense", seed=1002, fp4=False, norm=True, outliers=True),
}


# Bytes per launch that cross between the L2s and the memory side (memory-side cache or HBM) for the forward/dgrad
# grouped GEMM, measured with hardware counters (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE; KiB per dispatch
# averaged over the four launches of a step, each scaled by what the same counter reads for a 1 GiB -> 1 GiB
# elementwise kernel: 2.000 and 1.000).  The counter summary is committed as
# profiles/bench_mixtral_mxfp8_hbm_traffic.txt.
TRAFFIC_BYTES_PER_LAUNCH = {
    "mixtral_8x7b_moe_mxfp8": (3099696.1 * 2.000 + 821230.5 * 1.000) * 1024,
}


def route(spec):
    """tokens-per-expert (python list) from seeded synthetic router logits."""
    import torch

    G, topk, tokens = spec["G"], spec["topk"], spec["tokens"]
    if spec["routing"] == "dense":
        return [tokens]
    g = torch.Generator().manual_seed(spec["seed"])
    logits = torch.randn(tokens, G, generator=g)
    if spec["routing"] == "gauss_bias":
        logits = logits + torch.randn(G, generator=g)
    elif spec["routing"] == "zipf":
        ranks = torch.randperm(G, generator=g).float() + 1.0
        logits = logits + torch.log(ranks ** -1.2) * 3.0
    probs = torch.softmax(logits, dim=-1)
    idx = probs.topk(topk, dim=-1).indices.reshape(-1)
    return torch.bincount(idx, minlength=G).tolist()


def synth(shape, gen, device, scale=1.0, outliers=False, chunk=1 << 26):
    """Seeded synthetic bf16 tensor ~ N(0, scale^2) on ``device``: drawn in fp32 from ``gen`` (a CPU generator in the
    benchmark; tests may pass a device generator) in pieces of ``chunk`` elements of the flattened tensor, cast to
    bf16 and uploaded.  ``outliers``: 0.1 % of the entries, chosen by a uniform draw from the same generator right
    after each piece, are multiplied by 50 before the cast."""
    import torch

    n = 1
    for d in shape:
        n *= int(d)
    out = torch.empty(n, dtype=torch.bfloat16, device=device)
    for i in range(0, n, chunk):
        c = torch.randn(min(chunk, n - i), generator=gen, device=gen.device)
        if scale != 1.0:
            c *= scale
        if outliers:
            hit = torch.rand(c.numel(), generator=gen, device=gen.device) < 1e-3
            c = torch.where(hit, c * 50.0, c)
        out[i:i + c.numel()] = c.bfloat16().to(device)
    return out.view(*shape)


def synth_layer(spec, layer, rows, gen, device):
    """(x, w, dy, k, n) of linear ``layer`` (0: fc1, 1: fc2) of a workload, without autograd flags."""
    k, n = ((spec["hidden"], spec["fc1_out"]), (spec["fc2_in"], spec["hidden"]))[layer]
    grouped = spec["routing"] != "dense"
    x = synth((rows, k), gen, device, outliers=bool(spec.get("outliers")))
    w = synth((spec["G"], n, k) if grouped else (n, k), gen, device, scale=0.02)
    dy = synth((rows, n), gen, device)
    return x, w, dy, k, n


class LaunchTimer:
    """Brackets every C-ABI launch with events on the launch stream."""

    def __init__(self):
        self.records = []
        self.enabled = False

    def __call__(self, name, info):
        return _Bracket(self, name, info)


class _Bracket:
    def __init__(self, owner, name, info):
        self.o, self.name, self.info = owner, name, info

    def __enter__(self):
        if self.o.enabled:
            import torch

            self.e0 = torch.cuda.Event(enable_timing=True)
            self.e1 = torch.cuda.Event(enable_timing=True)
            self.e0.record(torch.cuda.current_stream())
        return self

    def __exit__(self, *exc):
        if self.o.enabled:
            import torch

            self.e1.record(torch.cuda.current_stream())
            self.o.records.append((self.name, self.info, self.e0, self.e1))
        return False


def norm_bytes(name, info):
    """Algorithmic bytes of one RMSNorm launch: bf16 read (+ bf16 write); backward reads x, dy and writes dx."""
    el = info["rows"] * info["k"]
    if name == "rmsnorm_bwd":
        return el * 6.0
    return el * (4.0 if info.get("want_y", True) else 2.0)


def quant_bytes(info):
    """Algorithmic bytes of one quantiser launch: bf16 read + codes + 1 scale byte / 32."""
    el = info["rows"] * info["cols"]
    code = 0.5 if info["fmt"] == 1 else 1.0
    copies = int(bool(info["rowwise"])) + int(bool(info["colwise"]))
    return el * (2.0 + copies * (code + 1.0 / 32.0))


def cpu_baseline(spec, lens, layers, sample_div=16):
    """The oracle's C restatement on the host cores, on 1/sample_div of the rows of the SAME tensors the GPU leg
    ran on (the first rows of every expert, the full-size weights): quantise -> dequantise -> fp32 matmul
    (torch CPU) -> bf16, forward + dgrad + wgrad of both linears.  ``layers``: (x, w, dy, k, n) device tensors."""
    import numpy as np
    import torch

    from oracle import c_oracle as C
    from oracle import mx_oracle as o

    C.load()
    threads = len(os.sched_getaffinity(0))
    threads = min(threads, int(os.environ.get("OMP_NUM_THREADS", threads)))
    torch.set_num_threads(threads)
    fmt_w = o.FMT_E2M1 if spec["fp4"] else o.FMT_E4M3
    fmt_a = o.FMT_E2M1 if spec.get("act_fp4") else o.FMT_E4M3
    G = spec["G"]
    slens = [max(1, ln // sample_div) if ln else 0 for ln in lens]
    m = sum(slens)
    starts = np.concatenate([[0], np.cumsum(lens)])[:-1]
    pick = torch.from_numpy(np.concatenate([np.arange(s0, s0 + ln) for s0, ln in zip(starts, slens)]).astype(np.int64))
    host = []
    for (x, w, dy, k, n) in layers:     # device -> host copies are outside the timed region
        idx = pick.to(x.device)
        host.append((x.detach()[idx].cpu(), w.detach().reshape(G, n, k).cpu(), dy.detach()[idx].cpu(), k, n))
    flops = 0.0
    t0 = time.perf_counter()
    for (xs_, ws_, dys_, k, n) in host:
        x = o.to_bf16_bits(xs_)
        dy = o.to_bf16_bits(dys_)
        w = o.to_bf16_bits(ws_)
        xq, xs = C.quantize_rowwise(x, fmt_a)
        xt, xts = C.quantize_colwise_segmented(x, slens, fmt_a)
        dq, ds = C.quantize_rowwise(dy, fmt_a)
        dt, dts = C.quantize_colwise_segmented(dy, slens, fmt_a)
        wq, ws, wqt, wst = C.quantize_2d(w, fmt_w)
        xf = torch.from_numpy(C.dequantize(xq, xs, fmt_a))
        df = torch.from_numpy(C.dequantize(dq, ds, fmt_a))
        xtf = torch.from_numpy(C.dequantize(xt, xts, fmt_a))
        dtf = torch.from_numpy(C.dequantize(dt, dts, fmt_a))
        offs = np.concatenate([[0], np.cumsum(slens)])
        _, poffs = o.segment_layout(slens)
        for e in range(G):
            if slens[e] == 0:
                continue
            wf = torch.from_numpy(C.dequantize(wq[e], ws[e], fmt_w))
            wtf = torch.from_numpy(C.dequantize(wqt[e], wst[e], fmt_w))
            sl = slice(int(offs[e]), int(offs[e + 1]))
            ps = slice(int(poffs[e]), int(poffs[e + 1]))
            y = (xf[sl] @ wf.t()).bfloat16()
            dx = (df[sl] @ wtf.t()).bfloat16()
            dw = (dtf[:, ps] @ xtf[:, ps].t()).bfloat16()
            del y, dx, dw
            flops += 6.0 * slens[e] * n * k
    dt_s = time.perf_counter() - t0
    # the reference's own CPU-runnable case at full size: X [4096, 4096] ~ N(0, 1), W [4096, 4096] ~ N(0, 0.02),
    # MXFP8 quantise both, dequantise, fp32 matmul, bf16 output (forward only)
    g1 = torch.Generator().manual_seed(1001)
    x1 = o.to_bf16_bits(torch.randn(4096, 4096, generator=g1).bfloat16())
    w1 = o.to_bf16_bits((torch.randn(4096, 4096, generator=g1) * 0.02).bfloat16())
    t1 = time.perf_counter()
    xq1, xs1 = C.quantize_rowwise(x1, o.FMT_E4M3)
    wq1, ws1, _, _ = C.quantize_2d(w1[None], o.FMT_E4M3)
    y1 = (torch.from_numpy(C.dequantize(xq1, xs1, o.FMT_E4M3)) @ torch.from_numpy(C.dequantize(wq1[0], ws1[0], o.FMT_E4M3)).t()).bfloat16()
    cfg1_s = time.perf_counter() - t1
    del y1
    return {
        "cfg1_dense_4096": {"value": round(2.0 * 4096 ** 3 / cfg1_s / 1e12, 6), "unit": "TFLOP/s", "seconds": round(cfg1_s, 3),
                            "sample": "full size: quantise X and W (C oracle), dequantise, torch CPU fp32 matmul, bf16 output"},
        "value": round(flops / dt_s / 1e12, 6),
        "unit": "TFLOP/s",
        "cores": threads,
        "kind": "port",
        "sample": f"the GPU leg's own tensors: the first 1/{sample_div} of every expert's rows ({m} routed rows), full-size weights; "
        f"C oracle quantise/dequantise + torch CPU fp32 matmul; {dt_s:.1f} s",
    }


def gemm_calibration(fp4_weights, dev, fp4_acts=False, bf16=False):
    """What this board's matrix cores deliver, measured in the same process, to read the GEMM figures against
    (the published peak assumes the 2.4 GHz boost clock; under load the board sits at its power limit):
    the library's register-only loop of the GEMM's own scaled MFMA (no memory traffic: the ceiling of any GEMM here),
    then one dense problem of the benchmark's size (M 32768, N 28672, K 4096) through this library's MX GEMM and through
    torch's vendor-library GEMMs: FP8 with one scale per tensor (no block scales) and, where torch supports it, MXFP8
    with E8M0 block scales.  About 4 s."""
    import torch

    from primus_amd import _lib

    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    out = {}

    def rate(fn, flops, seconds=0.6):
        fn()
        torch.cuda.synchronize()
        t_end = time.perf_counter() + 0.2
        while time.perf_counter() < t_end:      # bring the board to its steady clocks first
            fn()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        n, t_end = 0, time.perf_counter() + seconds
        e0.record()
        while time.perf_counter() < t_end:
            fn()
            n += 1
            torch.cuda.synchronize()
        e1.record()
        torch.cuda.synchronize()
        return round(n * flops / (e0.elapsed_time(e1) * 1e-3) / 1e12, 1)

    if bf16:
        # the unquantised workload: the register-only loop of the bf16 MFMA and torch's vendor dense bf16 GEMM
        iters = 8192
        flops = float(lib.mxl_calibrate_mfma_bf16_flops(iters))
        out["mfma_only_loop_bf16_TFLOP/s"] = rate(lambda: _lib.check(lib.mxl_calibrate_mfma_bf16(iters, st), "mxl_calibrate_mfma_bf16"), flops)
        out["mfma_only_loop"] = "mxl_calibrate_mfma_bf16: 256 workgroups x 4 waves, 32 MFMAs 32x32x16 bf16 per K slot on register operands, no memory traffic"
        M, N, Kd = 32768, 28672, 4096
        out["dense_gemm_shape_mnk"] = [M, N, Kd]
        x = torch.randn(M, Kd, device=dev).bfloat16()
        w = (torch.randn(N, Kd, device=dev) * 0.02).bfloat16()
        from primus_amd.pytorch import kernels as K
        out["this_library_bf16_one_group_TFLOP/s"] = rate(lambda: K.grouped_gemm_bf16_impl(x, w, None), 2.0 * M * N * Kd)
        out["torch_matmul_bf16_TFLOP/s"] = rate(lambda: torch.matmul(x, w.t()), 2.0 * M * N * Kd)
        return out
    iters = 4096
    flops = float(lib.mxl_calibrate_mfma_flops(iters))
    for name, (fa, fb) in (("fp8_x_fp8", (_lib.FMT_E4M3, _lib.FMT_E4M3)),) + ((("fp8_x_fp4", (_lib.FMT_E4M3, _lib.FMT_E2M1)),) if fp4_weights and not fp4_acts else ()) \
            + ((("fp4_x_fp4", (_lib.FMT_E2M1, _lib.FMT_E2M1)),) if fp4_acts else ()):
        def loop(fa=fa, fb=fb):
            _lib.check(lib.mxl_calibrate_mfma(fa, fb, iters, st), "mxl_calibrate_mfma")
        out["mfma_only_loop_%s_TFLOP/s" % name] = rate(loop, flops)
    out["mfma_only_loop"] = "mxl_calibrate_mfma: 256 workgroups x 4 waves, 16 scaled MFMAs 32x32x64 per K step on register operands, no memory traffic"
    M, N, Kd = 32768, 28672, 4096
    out["dense_gemm_shape_mnk"] = [M, N, Kd]
    # this library's MX GEMM on the same dense problem (one group), for a like-for-like figure beside torch's
    from primus_amd.pytorch import kernels as K
    x = torch.randn(M, Kd, device=dev).bfloat16()
    w = (torch.randn(N, Kd, device=dev) * 0.02).bfloat16()
    lay = K.pick_layout(1, N, Kd, M, fp8=True)
    xq, xs, _, _ = K.quantize_mx_impl(x, _lib.FMT_E4M3, rowwise=True, colwise=False, pad_to=K.GEMM_K_ALIGN, kchunk=lay)
    wq, ws, _, _ = K.quantize_mx_weight_2d_impl(w, _lib.FMT_E4M3, rowwise=True, colwise=False, pad_to=K.GEMM_K_ALIGN, kchunk=lay)
    del x, w
    out["this_library_mxfp8_block_scales_TFLOP/s"] = rate(lambda: K.gemm_mx_nt_impl(xq, xs, wq, ws, kchunk=lay), 2.0 * M * N * Kd)
    del xq, xs, wq, ws
    try:
        a8 = (torch.randn(M, Kd, device=dev) * 100).to(torch.float8_e4m3fn)
        b8 = (torch.randn(N, Kd, device=dev) * 100).to(torch.float8_e4m3fn)
        one = torch.ones((), device=dev)
        out["torch_scaled_mm_fp8_per_tensor_scale_TFLOP/s"] = rate(
            lambda: torch._scaled_mm(a8, b8.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16), 2.0 * M * N * Kd)
        try:
            sa = torch.full((M, Kd // 32), 127, dtype=torch.uint8, device=dev).view(torch.float8_e8m0fnu)
            sb = torch.full((N, Kd // 32), 127, dtype=torch.uint8, device=dev).view(torch.float8_e8m0fnu)
            out["torch_scaled_mm_mxfp8_block_scales_TFLOP/s"] = rate(
                lambda: torch._scaled_mm(a8, b8.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16), 2.0 * M * N * Kd)
        except Exception as ex:   # this torch build may not carry the MX path
            out["torch_scaled_mm_mxfp8_block_scales_TFLOP/s"] = None
            out["torch_scaled_mm_mxfp8_error"] = type(ex).__name__
    except Exception as ex:
        out["torch_scaled_mm_error"] = type(ex).__name__
    return out


def quantizer_twin(dev):
    """The dual MXFP8 quantiser's traffic without its arithmetic (mxl_calibrate_tile_copy: the same tiles in the same
    order, 2 bytes read and 1 + 1 written per element, streaming loads and stores) against the quantiser itself on
    the same tensor: how much of the distance to the stream calibration is the access pattern (a transposed copy
    written in 128-byte pieces a row pitch apart) and how much the kernel."""
    import torch

    from primus_amd import _lib
    from primus_amd.pytorch import kernels as K

    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    res = {"kernel": "mxl_calibrate_tile_copy: 128x128 bf16 tiles read, 1 byte/element to a row-major and 1 to a transposed array"}
    for rows, cols in ((32768, 4096), (32768, 28672)):
        x = torch.randn(rows, cols, device=dev, dtype=torch.bfloat16)
        o1 = torch.empty(rows, cols, dtype=torch.uint8, device=dev)
        o2 = torch.empty(cols, rows, dtype=torch.uint8, device=dev)

        def timed(fn, nbytes):
            for _ in range(3):
                fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(10):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return round(10 * nbytes / (e0.elapsed_time(e1) * 1e-3) / 1e9, 1)

        def twin(a, b):
            return lambda: _lib.check(lib.mxl_calibrate_tile_copy(x.data_ptr(), rows, cols, a, b, st), "mxl_calibrate_tile_copy")

        n = rows * cols
        entry = {
            "read+row+transposed_GB/s": timed(twin(o1.data_ptr(), o2.data_ptr()), 4.0 * n),
            "read+row_GB/s": timed(twin(o1.data_ptr(), None), 3.0 * n),
            "read+transposed_GB/s": timed(twin(None, o2.data_ptr()), 3.0 * n),
            "read_only_GB/s": timed(twin(None, None), 2.0 * n),
        }
        del o1, o2
        lay = K.pick_layout(1, 4096, cols, rows, fp8=True)
        entry["quantizer_GB/s"] = timed(
            lambda: K.quantize_mx_impl(x, _lib.FMT_E4M3, rowwise=True, colwise=True, pad_to=K.GEMM_K_ALIGN, kchunk=lay),
            (4.0 + 2.0 / 32) * n)
        res["%dx%d" % (rows, cols)] = entry
        del x
    return res


def board_sample(run_step, seconds):
    """Socket power and shader clocks (``amd-smi metric --power --clock``) sampled while ``run_step`` loops for
    ``seconds``: says how far below the 2.4 GHz that the MFMA peak is quoted at the chip clocks under this load.
    None when the tool is missing or prints something else."""
    import subprocess
    import threading

    import torch

    rows, stop = [], threading.Event()

    def sampler():
        while not stop.is_set():
            try:
                r = subprocess.run(["amd-smi", "metric", "--power", "--clock", "--csv"], capture_output=True, text=True, timeout=10)
                lines = [ln for ln in r.stdout.strip().splitlines() if ln.strip()]
                head, vals = lines[0].split(","), lines[1].split(",")
                rows.append(dict(zip(head, vals)))
            except Exception:
                return
            time.sleep(0.05)

    th = threading.Thread(target=sampler, daemon=True)
    t_end = time.perf_counter() + seconds
    run_step()
    torch.cuda.synchronize()
    th.start()
    while time.perf_counter() < t_end:
        run_step()
        torch.cuda.synchronize()
    stop.set()
    th.join(timeout=15)
    try:
        # the first and the last sample may straddle the loop's ends
        use = rows[1:-1] if len(rows) > 3 else rows
        power = [float(r["socket_power"]) for r in use]
        clocks = [float(v) for r in use for k, v in r.items() if k.startswith("gfx_") and k.endswith("_clk") and k.count("_") == 2]
        if not power or not clocks:
            return None
        return {"socket_power_w": round(sum(power) / len(power), 1), "gfx_clk_mhz_mean": round(sum(clocks) / len(clocks), 1),
                "gfx_clk_mhz_min": min(clocks), "gfx_clk_mhz_max": max(clocks), "gfx_clk_mhz_peak": 2400.0,
                "samples": len(use), "seconds": seconds, "source": "amd-smi metric --power --clock, sampled while the step loops"}
    except Exception:
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="mixtral_8x7b_moe_mxfp8", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gemm-calibration", action="store_true",
                    help="skip the matrix-core calibration (register-only MFMA loop, torch's vendor GEMMs)")
    ap.add_argument("--calibration-only", action="store_true",
                    help="run the matrix-core calibration alone and print its JSON (the command of the hardware-counter "
                         "comparison between torch's FP8 GEMM and this library's on one dense problem)")
    ap.add_argument("--no-wgrad-overlap", action="store_true",
                    help="keep wgrad on the launch stream behind dgrad (per-kernel durations are then undisturbed)")
    ap.add_argument("--board-seconds", type=float, default=2.0,
                    help="after the timed region, loop the step for this long while sampling socket power and shader "
                         "clocks with amd-smi (0: skip)")
    ap.add_argument("--no-graph-replay", action="store_true",
                    help="skip the measurement of the same step captured in a HIP graph and replayed")
    ap.add_argument("--calibrate-traffic", action="store_true",
                    help="launch one plain 1 GiB-in / 1 GiB-out elementwise kernel first, so that a hardware-counter "
                         "run of this command also reads the counters for a kernel of known HBM traffic")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no expert all-to-all); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    import primus_amd.pytorch as pt
    from primus_amd.pytorch import kernels as K
    from primus_amd.pytorch.core import Float4QuantConfig, Float8QuantConfig, Format, ScaleDtype, ScalingGranularity

    assert torch.cuda.is_available(), "bench.py needs a GPU: the MX linear path has no CPU fallback"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    spec = WORKLOADS[args.workload]
    if args.calibration_only:
        print(json.dumps({"mfma_calibration": gemm_calibration(spec["fp4"], dev, bool(spec.get("act_fp4")), bool(spec.get("bf16"))), "quantizer_traffic_twin": quantizer_twin(dev)}))
        return
    lens = route(spec)
    G, M = spec["G"], sum(lens)
    grouped = spec["routing"] != "dense"
    if spec["fp4"]:
        cfg = Float4QuantConfig(activation_format=Format.E2M1_X2 if spec.get("act_fp4") else Format.E4M3)
        op = pt.ops.grouped_gemm_fp4
    elif spec.get("tensorwise"):
        cfg = Float8QuantConfig(format=Format.HYBRID, granularity=ScalingGranularity.TENSORWISE)
        op = pt.ops.grouped_gemm_fp8 if grouped else None
    elif spec.get("blockwise"):
        cfg = Float8QuantConfig(format=Format.HYBRID, granularity=ScalingGranularity.BLOCKWISE, block_size=128)
        op = pt.ops.grouped_gemm_fp8 if grouped else None
    elif spec.get("bf16"):
        cfg = None
        op = lambda x, w, gl, trans_b=True, config=None: pt.ops.grouped_gemm(x, w, gl, trans_b=trans_b)  # noqa: E731
    else:
        cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE, scale_dtype=ScaleDtype.E8M0, block_size=32)
        op = pt.ops.grouped_gemm_fp8 if grouped else None

    # inputs from the CPU generator (fp32 -> bf16 -> upload), one seed per workload; `raw` keeps the plain tensors
    # for the CPU baseline
    gen = torch.Generator().manual_seed(spec["seed"])
    raw = [synth_layer(spec, i, M, gen, dev) for i in range(2)]

    def with_grad(layer, copy):
        x, w, dy, k, n = layer
        if copy:
            # detached copies: a clone of a tensor that already requires grad would be a non-leaf hanging on the first
            # set's leaves (their gradient-accumulation nodes, made on the default stream, would then outlive every
            # step, and a captured step would have to wait on that stream)
            x, w, dy = x.detach().clone(), w.detach().clone(), dy.detach().clone()
        return (x.requires_grad_(), w.requires_grad_(spec.get("wgrad", True)), dy, k, n)

    # Rotating buffer sets: a workload whose tensors would sit in the 256 MiB memory-side cache from one step to the
    # next runs over enough distinct copies to exceed 2 GB (the reference's own GEMM benchmark does the same,
    # primus/tools/benchmark/gemm_bench.py:60-123); the Mixtral workload's single set is 12 GB already.
    set_bytes = sum(t.numel() * 2 for (x, w, dy, _, _) in raw for t in (x, w, dy))
    n_sets = max(1, min(8, -(-(2 << 30) // set_bytes)))
    sets = [[with_grad(layer, i > 0) for layer in raw] for i in range(n_sets)]
    layers = sets[0]
    gl = torch.tensor(lens, dtype=torch.int64, device=dev)
    norm_w = torch.ones(spec["hidden"], device=dev).bfloat16().requires_grad_() if spec.get("norm") else None
    if not spec.get("wgrad", True):
        # Without a weight gradient the weights cannot change between steps: they are quantised once, before
        # the timed region, and the steps run on the cached copies (the reference's multi-microbatch path,
        # primus/backends/megatron/core/extensions/primus_turbo.py:1105-1115).
        from primus_amd.pytorch.core import QuantizedTensorPair, create_quantized_weight, float4_e2m1fn_x2, float8_e4m3

        dest = float4_e2m1fn_x2 if spec["fp4"] else float8_e4m3
        sets = [[(x, QuantizedTensorPair(*create_quantized_weight(w, dest, cfg)), dy, k, n) for (x, w, dy, k, n) in layer_set]
                for layer_set in sets]
        layers = sets[0]
    # forward + dgrad (+ wgrad unless the workload is defined without it): 2 M N K flops each
    passes = 3.0 if spec.get("wgrad", True) else 2.0
    flops_step = sum(2.0 * passes * M * n * k for (_, _, _, k, n) in layers)

    step_no = [0]

    def step():
        cur = sets[step_no[0] % n_sets]
        step_no[0] += 1
        for i, (x, w, dy, k, n) in enumerate(cur):
            if grouped:
                y = op(x, w, gl, trans_b=True, config=cfg)
            elif norm_w is not None and i == 0:
                y = pt.ops.rmsnorm_gemm_fp8(x, norm_w, 1e-5, w, config=cfg)
            else:
                y = pt.ops.gemm_fp8(x, w, trans_a=False, trans_b=True, out_dtype=None, config=cfg)
            # the gradients are returned and dropped, not accumulated into .grad
            wanted = [x] + ([w] if torch.is_tensor(w) and w.requires_grad else []) + ([norm_w] if norm_w is not None and i == 0 else [])
            torch.autograd.grad(y, wanted, dy)

    if args.calibrate_traffic:
        src = torch.zeros(1 << 28, dtype=torch.int32, device=dev)   # 1 GiB
        dst = torch.empty_like(src)
        torch.add(src, 1, out=dst)
        torch.cuda.synchronize()
        del src, dst

    pt.ops.set_wgrad_overlap(not args.no_wgrad_overlap)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    # Per-kernel accounting in a pass of its own, every launch bracketed with events on its stream and
    # wgrad kept behind dgrad: two kernels sharing the chip would inflate each other's duration.
    timer = LaunchTimer()
    K.set_launch_hook(timer)
    pt.ops.set_wgrad_overlap(False)
    timer.enabled = True
    kernel_steps = min(args.steps, 5)
    for _ in range(kernel_steps):
        step()
    torch.cuda.synchronize()
    timer.enabled = False
    K.set_launch_hook(None)

    ms_per_step = (t1 - t0) * 1e3 / args.steps
    value = flops_step / (ms_per_step * 1e-3) / 1e12

    # per-kernel accounting from the bracketed launches
    acc = {}
    for name, info, e0, e1 in timer.records:
        d = e0.elapsed_time(e1) * 1e-3
        a = acc.setdefault(name, dict(sec=0.0, n=0, flops=0.0, bytes=0.0))
        a["sec"] += d
        a["n"] += 1
        if "gemm" in name:
            a["flops"] += 2.0 * info["m"] * info["n"] * info["k"]
        elif name in ("rmsnorm_fwd", "rmsnorm_bwd"):
            a["bytes"] += norm_bytes(name, info)
        elif name == "amax":
            a["bytes"] += 2.0 * info["n"]
        else:
            a["bytes"] += quant_bytes(info)
    fwd_name = ("grouped_gemm_bf16" if spec.get("bf16") else
                ("grouped_gemm_blockwise_nt" if grouped else "gemm_blockwise_nt") if spec.get("blockwise") else
                "grouped_gemm_nt" if grouped else "gemm_nt")
    gk = acc[fwd_name]
    gemm_tflops = gk["flops"] / gk["sec"] / 1e12
    act_fp4 = bool(spec.get("act_fp4"))
    # the MFMA peak of the slower operand format: FP8 rate unless both operands are E2M1 (or bf16)
    peak = BF16_PEAK_TFLOPS if spec.get("bf16") else FP4_PEAK_TFLOPS if act_fp4 else FP8_PEAK_TFLOPS
    roofline = {
        # the MX and tensor-wise workloads run on the 4-slot ring kernel
        "kernel": "bf16_gemm_kernel<fwd/dgrad> (grouped_gemm_bf16)" if spec.get("bf16") else
                  "bw_gemm256_kernel<e4m3|e5m2,weight factors> (%s)" % fwd_name if spec.get("blockwise") else
                  "%s<%s,%s,fwd/dgrad%s> (%s)" % ("mx_gemm_ring_kernel",
                                                   "e4m3|e5m2" if spec.get("tensorwise") else "e2m1" if act_fp4 else "e4m3",
                                                   "e2m1" if spec["fp4"] else "e4m3",
                                                   ",alpha" if spec.get("tensorwise") else "", fwd_name),
        "bound": "mfma",
        "achieved": round(gemm_tflops, 2),
        "peak": peak,
        "unit": "TFLOP/s",
        "frac": round(gemm_tflops / peak, 4),
        "avg_launch_ms": round(gk["sec"] / gk["n"] * 1e3, 4),
        "flops_per_launch": gk["flops"] / gk["n"],
        "traffic": TRAFFIC_BYTES_PER_LAUNCH.get(args.workload),
    }
    kernels = {}
    for name, a in acc.items():
        ent = {"launches_per_step": a["n"] // kernel_steps, "ms_per_step": round(a["sec"] * 1e3 / kernel_steps, 4)}
        if a["flops"]:
            ent["TFLOP/s"] = round(a["flops"] / a["sec"] / 1e12, 2)
            ent["frac_bf16_mfma_peak" if spec.get("bf16") else "frac_fp4_mfma_peak" if act_fp4 else "frac_fp8_mfma_peak"] = round(a["flops"] / a["sec"] / 1e12 / peak, 4)
        else:
            ent["GB/s"] = round(a["bytes"] / a["sec"] / 1e9, 1)
            ent["frac_hbm_peak"] = round(a["bytes"] / a["sec"] / 1e9 / HBM_PEAK_GBS, 4)
        kernels[name] = ent
    gemm_sec = sum(a["sec"] for nme, a in acc.items() if "gemm" in nme)
    gemm_flops = sum(a["flops"] for nme, a in acc.items() if "gemm" in nme)

    out = {
        "metric": "%s grouped-GEMM TFLOPS (%s, quantisers inside the timed step)"
                  % ("bf16 (unquantised)" if spec.get("bf16") else "FP8 128-blockwise" if spec.get("blockwise") else
                     "FP8 tensor-wise" if spec.get("tensorwise") else "MXFP4" if spec.get("act_fp4") else "MXFP8",
                     "fwd+dgrad+wgrad" if spec.get("wgrad", True) else "fwd+dgrad"),
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 operands, fp32 accumulate" if spec.get("bf16")
                 else "fp8 e4m3 forward / e5m2 gradients, fp32 scales per 1x128 / 128x128 block, fp32 accumulate" if spec.get("blockwise")
                 else "mxfp4_e2m1 (E8M0 block scales) for every operand, fp32 accumulate" if spec.get("act_fp4")
                 else "mxfp4_e2m1 weights x mxfp8_e4m3 activations, fp32 accumulate" if spec["fp4"]
                 else "fp8 e4m3 forward / e5m2 gradients, one fp32 scale per tensor, fp32 accumulate" if spec.get("tensorwise")
                 else "mxfp8_e4m3 (E8M0 block scales), fp32 accumulate",
        "data": "synthetic (seeded CPU generator, fp32 -> bf16, uploaded; activations and gradients N(0,1)%s, random-init weights N(0,0.02)); %d rotating buffer set%s"
                % (" with 0.1 % of the activation entries x50" if spec.get("outliers") else "", n_sets, "" if n_sets == 1 else "s"),
        "config": {
            "workload": args.workload,
            "experts": G,
            "routed_rows": M,
            "tokens_per_expert": lens if G <= 32 else {"min": min(lens), "max": max(lens), "zeros": lens.count(0)},
            "gemms_nk": [[n, k] for (_, _, _, k, n) in layers],
            "flops_per_step": flops_step,
        },
        ("frac_bf16_mfma_peak_whole_step" if spec.get("bf16") else "frac_fp4_mfma_peak_whole_step" if act_fp4 else "frac_fp8_mfma_peak_whole_step"): round(value / peak, 4),
        "gemm_only_TFLOP/s": round(gemm_flops / gemm_sec / 1e12, 2),
        ("gemm_only_frac_bf16_mfma_peak" if spec.get("bf16") else "gemm_only_frac_fp4_mfma_peak" if act_fp4 else "gemm_only_frac_fp8_mfma_peak"): round(gemm_flops / gemm_sec / 1e12 / peak, 4),
        "wgrad_overlaps_dgrad": not args.no_wgrad_overlap,
        "kernels_note": "per-kernel figures: separate pass of %d steps after the timed region, wgrad serialised behind dgrad" % kernel_steps,
        "kernels": kernels,
        "roofline": roofline,
    }
    # what a plain streaming kernel reaches on this board: 1 GiB read + 1 GiB written by torch's elementwise add,
    # the practical ceiling the quantisers' GB/s are to be read against (their HBM traffic is the algorithmic one)
    src = torch.zeros(1 << 28, dtype=torch.int32, device=dev)
    dst = torch.empty_like(src)
    for _ in range(3):
        torch.add(src, 1, out=dst)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        torch.add(src, 1, out=dst)
    e1.record()
    torch.cuda.synchronize()
    stream_gbs = 10 * 2.0 * src.numel() * 4 / (e0.elapsed_time(e1) * 1e-3) / 1e9
    del src, dst
    out["hbm_stream_calibration"] = {"kernel": "torch.add(int32[2^28], 1, out=...): 1 GiB read, 1 GiB written", "GB/s": round(stream_gbs, 1),
                                     "frac_hbm_peak": round(stream_gbs / HBM_PEAK_GBS, 4)}
    for name in ("quantize", "quantize_weight_2d"):
        if name in kernels and "GB/s" in kernels[name]:
            kernels[name]["frac_of_stream_calibration"] = round(kernels[name]["GB/s"] / stream_gbs, 4)
    if not args.no_gemm_calibration:
        out["hbm_stream_calibration"]["quantizer_traffic_twin"] = quantizer_twin(dev)
    if not args.no_gemm_calibration:
        out["mfma_calibration"] = cal = gemm_calibration(spec["fp4"], dev, act_fp4, bool(spec.get("bf16")))
        ceiling = cal.get("mfma_only_loop_bf16_TFLOP/s" if spec.get("bf16") else "mfma_only_loop_fp4_x_fp4_TFLOP/s" if act_fp4 else
                          "mfma_only_loop_fp8_x_fp4_TFLOP/s" if spec["fp4"] else "mfma_only_loop_fp8_x_fp8_TFLOP/s")
        for name, entry in kernels.items():
            if "gemm" in name and "TFLOP/s" in entry and ceiling:
                entry["frac_of_mfma_only_loop"] = round(entry["TFLOP/s"] / ceiling, 4)
    if args.board_seconds > 0:
        pt.ops.set_wgrad_overlap(not args.no_wgrad_overlap)
        out["board"] = board_sample(step, args.board_seconds)
    if not args.no_graph_replay:
        # The same step captured once in a HIP graph and replayed (nothing on the path allocates behind torch's back,
        # synchronises or reads tokens-per-expert on the host): what the launch gaps of the eager loop cost.
        # Reported beside `value`, which stays the eager figure.
        try:
            pt.ops.set_wgrad_overlap(not args.no_wgrad_overlap)
            step_no[0] = 0
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step_no[0] = 0
                step()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            step_no[0] = 0
            with torch.cuda.graph(graph):
                step()
            for _ in range(2):
                graph.replay()
            torch.cuda.synchronize()
            g0 = time.perf_counter()
            for _ in range(args.steps):
                graph.replay()
            torch.cuda.synchronize()
            g_ms = (time.perf_counter() - g0) * 1e3 / args.steps
            out["graph_replay"] = {"ms_per_step": round(g_ms, 4), "TFLOP/s": round(flops_step / (g_ms * 1e-3) / 1e12, 2),
                                   "note": "one captured step (buffer set 0) replayed %d times; `value` is the eager loop" % args.steps}
            del graph
        except Exception as ex:      # reported, never fatal: the eager figures above stand on their own
            out["graph_replay"] = {"error": "%s: %s" % (type(ex).__name__, str(ex)[:200])}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(spec, lens, raw)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
