#!/usr/bin/env python3
"""Headline benchmark: NVFP4 quantize+pack of all Llama-3-8B-shaped linear weights on one MI355X.

One "step" = one pass of the quantize+pack hot path over the 224 bf16 weight tensors of the
model (32 layers x {q, k, v, o, gate, up, down}), inputs and per-tensor global amax already
resident in HBM, all outputs (packed codes, E4M3 block scales, fp32 global scales) written.
Prints ONE JSON line.  Synthetic weights: bf16 N(0, 0.02), generated on the device.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers 32] [--no-cpu-baseline]
"""

import argparse
import contextlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "tensorrt-model-optimizer_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# Llama-3-8B linear shapes [out, in]
LAYER_SHAPES = [("q_proj", 4096, 4096), ("k_proj", 1024, 4096), ("v_proj", 1024, 4096),
                ("o_proj", 4096, 4096), ("gate_proj", 14336, 4096), ("up_proj", 14336, 4096),
                ("down_proj", 4096, 14336)]
QUANT_BYTES_PER_ELEM = 2.0 + 0.5 + 1.0 / 16.0   # bf16 read + codes + block scale
AMAX_BYTES_PER_ELEM = 2.0
DEQUANT_BYTES_PER_ELEM = 0.5 + 1.0 / 16.0 + 2.0
# HBM bytes per launch of nvfp4_quantize_multi_kernel on the default 32-layer workload, from
# rocprofv3 --pmc FETCH_SIZE (6,829,310 KiB x 2.000) and WRITE_SIZE (3,833,868 KiB x 1.000); the
# scale factors come from a 1 GiB device copy in the same runs
# (profiles/nvfp4_quantize_multi_kernel__llama3_8b_weights.txt).
MEASURED_TRAFFIC_BYTES_32_LAYERS = 17.912e9
# mean kernel-trace duration of the 30 timed dispatches of the default run in that profile
PROFILE_TIMED_LAUNCH_US = 2873.0
TRAFFIC_SOURCE = ("profiles/nvfp4_quantize_multi_kernel__llama3_8b_weights.txt (rocprofv3 --pmc FETCH_SIZE, "
                  "WRITE_SIZE of this command, scaled by a device copy of known size)")


def make_weights(torch, layers, device):
    g = torch.Generator(device=device).manual_seed(2)
    ws = []
    for _ in range(layers):
        for _, n, k in LAYER_SHAPES:
            ws.append(torch.randn(n, k, generator=g, device=device, dtype=torch.bfloat16).mul_(0.02))
    return ws


def verify_against_restatement(torch, weights, amax, qplan):
    """What the timed launch wrote against the C restatement of the reference arithmetic on the
    host (packed codes, block scales, global scale), for tensors spread over the whole launch:
    k, o and down of the first layer, gate of the middle layer, and the three largest tensors
    of the last layer (the launch's last tiles)."""
    from oracle import cref

    packed, wsf, wsf2 = qplan.packed, qplan.wsf, qplan.wsf2
    torch.cuda.synchronize()
    per, n = len(LAYER_SHAPES), len(weights)
    picks = sorted({1, 3, 6, (n // per // 2) * per + 4, n - 3, n - 2, n - 1} & set(range(n)))
    for i in picks:
        p_c, s_c, w2_c = cref.nvfp4_quantize(weights[i].cpu(), 16, float(amax[i]))
        assert torch.equal(packed[i].cpu(), p_c), f"tensor {i}: packed codes differ"
        assert torch.equal(wsf[i].cpu().view(torch.uint8), s_c.view(torch.uint8)), f"tensor {i}: scales differ"
        assert float(wsf2[i]) == float(w2_c), f"tensor {i}: global scale differs"
    return (f"outputs of the timed launch for tensors {picks} of {n} (first, middle and last layer) "
            "equal the CPU restatement bit for bit")


def timed(torch, fn, steps, warmup):
    """Wall time per step (ms) and mean per-launch device time (ms) from events on the stream
    the kernels are launched on (torch's current stream)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    dev_ms = sum(s.elapsed_time(e) for s, e in zip(starts, ends)) / steps
    return wall_ms, dev_ms


def cpu_baseline(torch, passes=3, c_passes=4):
    """The reference's CPU path for the benchmarked configuration -- NVFP4QTensor.quantize on torch CPU
    tensors, restated op for op in oracle/ -- on a bounded sample: the seven weights of one
    decoder layer (all four shapes), one warm-up pass, then `passes` timed passes from a given
    global amax; the whole model is 32 such layers.  The OpenMP C restatement of the same
    arithmetic is timed beside it and must give the same bytes."""
    from oracle import cref
    from oracle import export as oexport

    g = torch.Generator().manual_seed(2)
    weights = []
    for _, n, k in LAYER_SHAPES:
        w = (0.02 * torch.randn(n, k, generator=g)).to(torch.bfloat16)
        weights.append((w, w.abs().max()))
    elems = sum(w.numel() for w, _ in weights)
    for w, amax in weights:                      # warm-up pass (threads, allocator), and the check
        p_t, s_t, _ = oexport.nvfp4_export(w, amax, 16)
        p_c, s_c, _ = cref.nvfp4_quantize(w, 16, float(amax))
        assert torch.equal(p_c, p_t) and torch.equal(s_c.view(torch.uint8), s_t.view(torch.uint8))
    t0 = time.perf_counter()
    for _ in range(passes):
        for w, amax in weights:
            oexport.nvfp4_export(w, amax, 16)
    secs = time.perf_counter() - t0
    t0 = time.perf_counter()
    for _ in range(c_passes):
        for w, amax in weights:
            cref.nvfp4_quantize(w, 16, float(amax))
    c_secs = time.perf_counter() - t0
    rate = passes * elems * QUANT_BYTES_PER_ELEM / secs / 1e9
    return {
        "value": round(rate, 4),
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"torch CPU restatement of NVFP4QTensor.quantize on the 7 weights of one layer "
                  f"({elems} elements), {passes} timed passes after one warm-up pass, {secs:.2f} s; "
                  f"32 layers extrapolate to {32 * secs / passes:.1f} s per model pass; host has "
                  f"{os.cpu_count()} logical CPUs",
        "c_port_GBps": round(c_passes * elems * QUANT_BYTES_PER_ELEM / c_secs / 1e9, 3),
        "c_port_threads": cref.threads(),
    }


def cpu_reference_configs(torch):
    """The other benchmark configurations on the reference's CPU path (torch restatements in oracle/), each
    run once on the host cores: C1 and C4 in full, C3 in full (21 alphas), C5's quantizer work on one
    layer and one sequence, extrapolated.  Seconds of wall time; a reported baseline only."""
    import torch.nn.functional as F  # noqa: F401

    from oracle import awq as oawq
    from oracle import fake_quant, qtensor, reduce

    out = {"threads": torch.get_num_threads()}

    def clock(fn):
        t0 = time.perf_counter()
        fn()
        return time.perf_counter() - t0

    g = torch.Generator().manual_seed(1)
    w = 0.02 * torch.randn(4096, 4096, generator=g)
    w.view(-1)[torch.randperm(w.numel(), generator=g)[:16777]] *= 50
    w = w.to(torch.bfloat16)
    clock(lambda: fake_quant.fp8_eager(w[:256], reduce.reduce_amax(w[:256])))  # warm the threads
    out["c1_fp8_amax_plus_qdq_4096x4096_s"] = round(
        clock(lambda: fake_quant.fp8_eager(w, reduce.reduce_amax(w))), 4)

    g = torch.Generator().manual_seed(3)
    w3 = (0.02 * torch.randn(4096, 4096, generator=g)).to(torch.bfloat16)
    c = torch.exp(torch.randn(4096, generator=g))
    c[torch.randperm(4096, generator=g)[:41]] *= 20
    x3 = (torch.randn(512, 4096, generator=g) * c).to(torch.bfloat16)
    out["c3_awq_lite_21_alphas_4096x4096_s"] = round(
        clock(lambda: oawq.awq_lite_search(w3, [x3], alpha_step=0.05, block_size=128)), 3)

    g = torch.Generator().manual_seed(4)
    x = (torch.randn(8192, 8192, generator=g) * torch.exp(1.5 * torch.randn(8192, generator=g))[None, :]
         ).to(torch.bfloat16)

    def c4_nvfp4():  # the CPU has no fake-quant kernel: quantize + dequantize through the QTensor
        p, s, s2 = qtensor.nvfp4_quantize(x, 16)
        qtensor.nvfp4_dequantize(p, s, s2, 16, x.shape, x.dtype)
    out["c4_nvfp4_amax_plus_qdq_8192x8192_s"] = round(clock(c4_nvfp4), 3)
    g = torch.Generator().manual_seed(5)
    w8 = (0.02 * torch.randn(8192, 8192, generator=g)).to(torch.bfloat16)

    def c4_smoothquant():  # quantizer work only: the layer's own GEMM is not part of it
        act = reduce.reduce_amax(x, axis=[0]).reshape(-1)
        pqs, w_new, in_amax, w_amax = oawq.smoothquant_linear(w8, act, 0.5)
        fake_quant.tensor_quant(x * pqs, in_amax, 8, False, False)
        fake_quant.tensor_quant(w_new, w_amax, 8, False, False)
    out["c4_smoothquant_int8_8192x8192_quantizer_work_s"] = round(clock(c4_smoothquant), 3)
    del x, w8

    # C5: per layer and forward the reference reduces the 7 weights (every forward) and, per
    # sequence, the inputs of the 7 linears and K / V; timed on one layer and one 512-token sequence
    g = torch.Generator().manual_seed(6)
    ws = [(0.02 * torch.randn(n, k, generator=g)).to(torch.bfloat16) for _, n, k in LAYER_SHAPES]
    acts = [torch.randn(512, k, generator=g).to(torch.bfloat16) for _, _, k in LAYER_SHAPES]
    kv = [torch.randn(8, 512, 128, generator=g).to(torch.bfloat16) for _ in range(2)]
    t_w = clock(lambda: [reduce.reduce_amax(t) for t in ws])
    t_a = clock(lambda: [reduce.reduce_amax(t) for t in acts + kv])
    forwards = 8  # 128 sequences in batches of 16
    out["c5_quantizer_work_one_layer_s"] = {"weights_one_forward": round(t_w, 4),
                                            "activations_and_kv_one_sequence": round(t_a, 4)}
    out["c5_quantizer_work_extrapolated_s"] = round(32 * (forwards * t_w + 128 * t_a), 1)
    out["note"] = ("reduce_amax / fake quant / QTensor code of the reference restated in torch, default "
                   "thread count; C5 counts the quantizer reductions only (no decoder GEMMs) and is 32 "
                   "layers x (8 forwards x weights + 128 sequences x activations) of the one-layer timings")
    return out


def single_tensor_configs(torch, steps, warmup):
    """The three single-tensor benchmark configurations (one tensor / one linear each), device time per pass.

    C1: FP8 abs-max + fake quant of a 4096 x 4096 weight with 0.1 % outliers (6 B / element).
    C3: AWQ-lite search, 21 alphas, W 4096 x 4096, X 512 x 4096 (mtq.quantize end to end, and the
        flop rate of its 22 GEMMs over that time).
    C4: NVFP4 abs-max + dynamic-block fake quant of 8192 x 8192 activations (6 B / element), and
        SmoothQuant (alpha 0.5) + INT8 on an 8192 x 8192 linear end to end.
    """
    import copy

    from torch import nn

    import modelopt_amd.torch.quantization as mtq
    from modelopt_amd import _hip

    dev = torch.device("cuda:0")
    out = {}

    g = torch.Generator().manual_seed(1)
    w = 0.02 * torch.randn(4096, 4096, generator=g)
    w.view(-1)[torch.randperm(w.numel(), generator=g)[:16777]] *= 50
    w = w.to(torch.bfloat16).to(dev)
    acc = torch.zeros(1, dtype=torch.float32, device=dev)
    y = torch.empty_like(w)

    def train(fn, reps=200):
        # one event pair around a train of passes (after an untimed train of the same length): a
        # pass is 20 - 80 us, which an event pair per pass would inflate by several microseconds
        for _ in range(reps):
            fn()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / reps

    def c1():
        # the calibrator's running maximum (no fill per pass: the accumulator only ever grows,
        # and a second look at the same tensor leaves it as it is), then the fake quant with it
        _hip.absmax_into(w, acc, 1, 1, w.numel())
        _hip.fp8_qdq(w, acc, 1, 1, w.numel(), out=y)
    ms = train(c1)
    out["c1_fp8_amax_plus_qdq_4096x4096"] = {"ms": round(ms, 4), "GBps": round(w.numel() * 6 / ms / 1e6, 1)}
    # the same in one launch that reads the tensor once (4 B / element): every workgroup keeps its
    # share in registers while the workgroups agree on the abs-max
    # a dynamic quantizer: the abs-max of this very call, then the fake quant of the same tensor,
    # on 32 different tensors in turn (1 GiB: none of them is in a cache when its turn comes).
    # With the hint the reduction uses plain loads and leaves the tensor in the memory-side cache
    # for the fake quant; without it, streaming loads as in a calibration pass.
    many = [torch.randn(4096, 4096, device=dev).to(torch.bfloat16) for _ in range(32)]
    turn = [0]

    def c1_dynamic(reread):
        x = many[turn[0] % len(many)]
        turn[0] += 1
        _hip.absmax_into(x, acc, 1, 1, x.numel(), reread=reread)
        _hip.fp8_qdq(x, acc.reshape(()), 1, 1, x.numel(), out=y)
    ms_hint, ms_stream = train(lambda: c1_dynamic(True), reps=128), train(lambda: c1_dynamic(False), reps=128)
    out["c1_fp8_dynamic_amax_plus_qdq_4096x4096_cold_inputs"] = {
        "ms": round(ms_hint, 4), "GBps": round(w.numel() * 6 / ms_hint / 1e6, 1),
        "ms_with_streaming_loads_in_the_reduction": round(ms_stream, 4)}
    del many

    def c1_fused():
        assert _hip.fused_amax_qdq(w, "fp8", out=y) is not None
    ms = train(c1_fused)
    out["c1_fp8_fused_amax_qdq_4096x4096"] = {"ms": round(ms, 4), "GBps": round(w.numel() * 4 / ms / 1e6, 1),
                                              "bytes_per_element": 4}
    wq = (0.02 * torch.randn(4096, 4096, generator=torch.Generator().manual_seed(7))).to(torch.bfloat16).to(dev)

    def nvfp4_two():
        acc.zero_()
        _hip.absmax_into(wq, acc, 1, 1, wq.numel())
        _hip.nvfp4_quantize(wq, acc.reshape(()), 16)

    def nvfp4_fused():
        assert _hip.nvfp4_quantize_fused(wq) is not None
    ms2, ms1 = train(nvfp4_two), train(nvfp4_fused)
    out["nvfp4_amax_plus_quantize_one_weight_4096x4096"] = {
        "two_launches_ms": round(ms2, 4), "fused_one_launch_ms": round(ms1, 4),
        "fused_GBps": round(wq.numel() * QUANT_BYTES_PER_ELEM / ms1 / 1e6, 1)}
    assert not _hip.fused_gave_up(dev)

    g = torch.Generator().manual_seed(4)
    x = (torch.randn(8192, 8192, generator=g) * torch.exp(1.5 * torch.randn(8192, generator=g))[None, :]
         ).to(torch.bfloat16).to(dev)
    y = torch.empty_like(x)

    acc.zero_()

    def c4():
        _hip.absmax_into(x, acc, 1, 1, x.numel())
        _hip.nvfp4_qdq(x, acc, 16, 0, out=y)
    ms = train(c4)
    out["c4_nvfp4_amax_plus_qdq_8192x8192"] = {"ms": round(ms, 4), "GBps": round(x.numel() * 6 / ms / 1e6, 1)}

    class OneLinear(nn.Module):
        def __init__(self, weight):
            super().__init__()
            self.proj = nn.Linear(weight.shape[1], weight.shape[0], bias=False, device=dev,
                                  dtype=torch.bfloat16)
            self.proj.weight.data.copy_(weight)

        def forward(self, t):
            return self.proj(t)

    busy = torch.empty(4096, 4096, dtype=torch.bfloat16, device=dev).normal_()

    def end_to_end(weight, acts, cfg, reps=12):
        best = None
        for _ in range(reps):          # smallest of `reps`; the first also pays GEMM autotuning
            model = OneLinear(weight)
            # a few milliseconds of unrelated matrix work first, as the layers before this one
            # would be in a model-sized run.  (The clocks still fall back during the half
            # millisecond of host work before the first big kernel: the clip search kernel, 1.35 ms
            # in a train of launches, takes 1.85 ms inside this call.)
            for _ in range(12):
                busy @ busy
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            mtq.quantize(model, cfg, lambda m: m(acts))
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            best = dt if best is None else min(best, dt)
        return best

    g = torch.Generator().manual_seed(5)
    w8 = (0.02 * torch.randn(8192, 8192, generator=g)).to(torch.bfloat16).to(dev)
    cfg = copy.deepcopy(mtq.INT8_SMOOTHQUANT_CFG)
    cfg["algorithm"] = {"method": "smoothquant", "alpha": 0.5}
    out["c4_smoothquant_int8_8192x8192_end_to_end_ms"] = round(end_to_end(w8, x, cfg) * 1e3, 3)
    del w8, x, y

    g = torch.Generator().manual_seed(3)
    w3 = (0.02 * torch.randn(4096, 4096, generator=g)).to(torch.bfloat16).to(dev)
    c = torch.exp(torch.randn(4096, generator=g))
    c[torch.randperm(4096, generator=g)[:41]] *= 20
    x3 = (torch.randn(512, 4096, generator=g) * c).to(torch.bfloat16).to(dev)
    cfg = copy.deepcopy(mtq.INT4_AWQ_CFG)
    cfg["algorithm"] = {"method": "awq_lite", "alpha_step": 0.05}
    secs = end_to_end(w3, x3, cfg)
    flops = 2 * 512 * 4096 * 4096 * 22
    out["c3_awq_lite_21_alphas_4096x4096"] = {
        "end_to_end_ms": round(secs * 1e3, 3), "gemm_flops": flops,
        "gemm_TFLOPs_over_end_to_end": round(flops / secs / 1e12, 1)}

    # the search step of that configuration on its own: one launch scores all 21 alphas (weights
    # scaled and INT4 block-quantised on the fly, bf16 MFMA GEMM, loss in the epilogue); the
    # MFMA roofline is MI355X's dense bf16 peak
    import torch.nn.functional as F
    scales = torch.exp(0.5 * torch.randn(21, 4096, generator=g)).to(torch.bfloat16).to(dev)
    ref = F.linear(x3, w3).contiguous()
    xs = _hip.awq_scaled_activations(x3, (1 / scales.float()).to(torch.bfloat16))
    loss = torch.zeros(21, dtype=torch.float64, device=dev)

    def search():
        _hip.awq_search_losses_into(xs, w3, scales, ref, 128, 4, False, False, loss)
    ms = train(search, reps=50)   # 50 untimed launches (past the clock ramp), then 50 under one event pair
    kflops = 2 * 512 * 4096 * 4096 * 21
    out["c3_awq_search_kernel_21_alphas"] = {
        "ms": round(ms, 4), "TFLOPs": round(kflops / ms / 1e9, 1), "bound": "mfma",
        "peak_TFLOPs": 2500.0, "frac": round(kflops / ms / 1e9 / 2500.0, 4)}

    # AWQ clip search on the same weight: 11 clip ratios x every 128-wide block, 64 calibration
    # tokens, one launch.  Vector-ALU bound: two vector instructions per rounded product (one
    # fp32 multiply each; one conversion to bf16 and one v_dot2c_f32_bf16 add per pair), against
    # an issue peak of one instruction per lane and clock: 256 CUs x 64 lanes x 2.4 GHz
    ratios = [round(float(v), 2) for v in torch.arange(0.5, 1.0, 0.05)] + [1.0]
    x64 = x3[::8].contiguous()
    w_amax = w3.view(-1, 128).abs().amax(1, keepdim=True)
    clip_loss = torch.zeros(len(ratios), 4096, 32, device=dev)

    def clip():
        _hip.awq_clip_losses_into(x64, w3, w_amax, ratios, 128, 4, False, False, clip_loss)
    ms = train(clip, reps=20)
    products = 4096 * 4096 * 64 * (len(ratios) + 1)
    out["awq_clip_search_kernel_11_ratios_4096x4096_64_tokens"] = {
        "ms": round(ms, 4), "rounded_products_per_s": round(products / ms * 1e3, 0), "bound": "valu",
        "vector_instructions_per_product": 2.0, "peak_lane_instructions_per_s": 39.32e12,
        "frac": round(2.0 * products / ms * 1e3 / 39.32e12, 4)}
    cfg = copy.deepcopy(mtq.INT4_AWQ_CFG)
    cfg["algorithm"] = {"method": "awq_clip"}
    out["awq_clip_4096x4096_end_to_end_ms"] = round(end_to_end(w3, x3, cfg) * 1e3, 3)
    return out


def secondary_kernels(torch, steps, warmup):
    """The library's other streaming kernels on the largest weight of a Llama-3-8B layer
    (14336 x 4096 bf16) and on one calibration batch of activations (8192 x 4096 bf16): device
    microseconds per launch and algorithmic bytes per second against the 8 TB/s HBM peak."""
    from modelopt_amd import _hip

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(2)
    out = {}

    def rec(name, fn, nbytes):
        # one event pair around a train of launches: these kernels run for 5 - 50 us, which a
        # pair of events per launch would inflate.  An untimed train of the same length goes
        # first: the first milliseconds after other work run 5 - 10 % slower (clocks, caches)
        reps = max(steps, 200)
        for _ in range(max(warmup, reps)):
            fn()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            fn()
        end.record()
        torch.cuda.synchronize()
        ms = start.elapsed_time(end) / reps
        out[name] = {"us": round(ms * 1e3, 2), "GBps": round(nbytes / ms / 1e6, 1),
                     "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 3)}

    n_rows, k = 14336, 4096
    w = torch.randn(n_rows, k, device=dev, generator=g).mul_(0.02).to(torch.bfloat16)
    n = w.numel()
    y = torch.empty_like(w)
    blk = torch.zeros(n // 128, dtype=torch.float32, device=dev)
    _hip.absmax_into(w, blk, 1, n // 128, 128)
    ws = blk.reshape(n_rows, k // 128) / 7.0
    s = torch.rand(k, device=dev, generator=g).add_(0.5).to(torch.bfloat16)
    amax = w.abs().amax().float()
    rec("int4_pack_rows_14336x4096", lambda: _hip.int4_pack_rows(w, ws), n * 2.5)
    rec("int4_block_quantize_14336x4096", lambda: _hip.int4_block_quantize(w, 128), n * 2.5)
    packed4, sc4 = _hip.int4_block_quantize(w, 128)
    rec("int4_block_dequantize_14336x4096", lambda: _hip.int4_block_dequantize(packed4, sc4, 128), n * 2.5)
    rec("scale_block_int_qdq_14336x4096", lambda: _hip.scale_block_int_qdq(w, s, 128, out=y), n * 4)
    rec("mul_cols_14336x4096", lambda: _hip.mul_cols(w, s, out=y), n * 4)
    col = torch.zeros(k, dtype=torch.float32, device=dev)
    rec("weight_scale_colsum_14336x4096", lambda: _hip.weight_scale_colsum_into(w, col, 128), n * 2)
    rec("fp8_qdq_14336x4096", lambda: _hip.fp8_qdq(w, amax, 1, 1, n, out=y), n * 4)
    rec("int8_qdq_14336x4096", lambda: _hip.int_qdq(w, amax, 1, 1, n, 8, False, False, out=y), n * 4)
    rec("nvfp4_qdq_14336x4096", lambda: _hip.nvfp4_qdq(w, amax, out=y), n * 4)
    pk, wsf, wsf2 = _hip.nvfp4_quantize(w, amax, 16)
    rec("nvfp4_dequantize_14336x4096", lambda: _hip.nvfp4_dequantize(pk, wsf, wsf2, 16, torch.bfloat16),
        n * DEQUANT_BYTES_PER_ELEM)
    del y, pk, wsf, packed4

    for t in (512, 8192):
        x = torch.randn(t, k, device=dev, generator=g).to(torch.bfloat16)
        b = torch.randn(t, k, device=dev, generator=g).to(torch.bfloat16)
        m = x.numel()
        a1 = torch.zeros(1, dtype=torch.float32, device=dev)
        ak = torch.zeros(k, dtype=torch.float32, device=dev)
        a64 = torch.zeros(1, dtype=torch.float64, device=dev)
        rec(f"abs_colsum_{t}x4096", lambda: _hip.abs_colsum_into(x, ak), m * 2)
        rec(f"absmax_per_tensor_{t}x4096", lambda: _hip.absmax_into(x, a1, 1, 1, m), m * 2)
        rec(f"absmax_per_column_{t}x4096", lambda: _hip.absmax_into(x, ak, t, k, 1), m * 2)
        rec(f"sq_diff_sum_{t}x4096", lambda: _hip.sq_diff_sum_into(x, b, a64), m * 4)
    return out


def calib_sweep(torch, layers, n_seqs, batch, seq_len=512):
    """Calibration sweep configuration: mtq.quantize (NVFP4 weights + inputs, FP8 KV cache, max calibration) on
    a random-init Llama-3-8B-shaped decoder over n_seqs x 512 uniform-random token ids.  Reports
    end-to-end seconds (the reference's own stopwatch brackets mtq.quantize the same way,
    examples/llm_ptq/hf_ptq.py:214-232), the forward-only seconds of the same data with no
    quantizers attached, and their difference = time attributable to the quantizer kernels."""
    import dataclasses

    import modelopt_amd.torch.quantization as mtq
    from modelopt_amd.testing.llama_decoder import LLAMA3_8B, LlamaForCausalLM

    dev = torch.device("cuda:0")
    cfg = dataclasses.replace(LLAMA3_8B, num_hidden_layers=layers)
    model = LlamaForCausalLM(cfg, device=dev, seed=5)
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, cfg.vocab_size, (n_seqs, seq_len), generator=g).to(dev)

    @torch.no_grad()
    def forward_loop(m):
        for i in range(0, n_seqs, batch):
            m(ids[i:i + batch])

    forward_loop(model)  # warm-up (GEMM autotuning, allocator)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    forward_loop(model)
    torch.cuda.synchronize()
    plain_s = time.perf_counter() - t0

    qcfg = mtq.utils.update_quant_cfg_with_kv_cache_quant(mtq.NVFP4_DEFAULT_CFG,
                                                          mtq.FP8_KV_CFG["quant_cfg"])
    # warm-up of the quantize path as the forward loop above is the warm-up of the plain one:
    # the same call on a one-layer model and one sequence, so that the tensor library's kernels
    # that only this path uses (loaded on first use, 10 - 20 ms each) are resident before the clock
    # starts -- the timed call is the only one of its kind in the process
    small = LlamaForCausalLM(dataclasses.replace(LLAMA3_8B, num_hidden_layers=1), device=dev, seed=6)
    from modelopt_amd.torch.export.unified_export_hf import _export_hf_checkpoint
    with torch.no_grad():
        mtq.quantize(small, qcfg, lambda m: m(ids[:1]))
        small(ids[:1])
        _export_hf_checkpoint(small)   # the export below is warmed up the same way
    del small
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    mtq.quantize(model, qcfg, forward_loop)
    torch.cuda.synchronize()
    calib_s = time.perf_counter() - t0
    n_q = sum(1 for m in model.modules() if isinstance(m, mtq.nn.TensorQuantizer) and m.is_enabled)
    # the quantizer kernels on their own: the same calibration pass once more with an event pair
    # around every library call (sum of the per-call device times)
    from modelopt_amd import _hip
    for m in model.modules():
        if isinstance(m, mtq.nn.TensorQuantizer):
            m.reset_amax()
    with _hip.KernelTimer() as kt:
        mtq.calibrate(model, "max", forward_loop)
    # the same data once more through the calibrated model: every forward fake-quantises the
    # inputs and weights of all 224 linears and K / V (what evaluating a PTQ model costs)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    forward_loop(model)
    torch.cuda.synchronize()
    fake_s = time.perf_counter() - t0
    w_bytes = sum(m.weight.numel() * 2 for m in model.modules()
                  if hasattr(m, "weight_quantizer") and m.weight_quantizer.is_enabled)

    # the export of the calibrated model, in memory (the reference's export_hf_checkpoint minus the
    # safetensors write): fusion pre-pass with its two-token forward, one quantize+pack launch for
    # all NVFP4 linears, scale buffers, state-dict renaming
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    state, _ = _export_hf_checkpoint(model)
    torch.cuda.synchronize()
    export_s = time.perf_counter() - t0
    packed_bytes = sum(v.numel() * v.element_size() for k, v in state.items()
                       if k.endswith((".weight", ".weight_scale")) and v.dtype in (torch.uint8, torch.float8_e4m3fn))
    del state
    tokens = n_seqs * seq_len
    # algorithmic: every quantizer reads its own input (7 linears + K and V per layer); actually
    # read: q / k / v and gate / up share one reduction of their common input
    act_bytes = tokens * layers * (38912 * 2 + 2 * 1024 * 2)
    act_bytes_read = tokens * layers * ((3 * 4096 + 14336) * 2 + 2 * 1024 * 2)
    return {
        "end_to_end_calib_s": round(calib_s, 3),
        "forward_only_s": round(plain_s, 3),
        "quantizer_overhead_s": round(calib_s - plain_s, 3),
        "quantizer_kernel_s": round(kt.total_seconds, 4),
        "quantizer_kernel_calls": dict(kt.calls),
        "enabled_quantizers": n_q,
        "tokens": tokens,
        "amax_bytes_algorithmic": {"activations_and_kv": act_bytes, "weights_once": w_bytes},
        "amax_bytes_read_after_sharing": {"activations_and_kv": act_bytes_read, "weights_once": w_bytes},
        "fake_quant_forward_s": round(fake_s, 3),
        "export_in_memory_s": round(export_s, 3),
        "export_packed_bytes": packed_bytes,
        "config": f"{layers} layers, {n_seqs} seqs x {seq_len} tokens, batch {batch}, NVFP4 W+A, FP8 KV, max",
    }


def probe_l2(torch):
    """How fast the compute units pull L2-resident data through L1 misses (the path the A operand of
    the AWQ-lite search kernel takes: 3.93 GB per launch of the 21-alpha 4096 x 4096 case).  A
    kernel that only loads, from libmodelopt_probe.so: one workgroup of 8 wavefronts per compute
    unit as in the search kernel (or four, with no unused LDS), every workgroup of an XCD walking
    the same region in step ("shared", the search kernel's pattern) or its own slice of it
    ("distinct"), 4 / 8 / 16 loads of 16 bytes in flight per lane."""
    import ctypes

    lib = ctypes.CDLL(os.path.join(ROOT, "tensorrt-model-optimizer_amd", "libmodelopt_probe.so"))
    fn = lib.mo_probe_l2_read
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                   ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    dev = torch.device("cuda:0")
    units = torch.cuda.get_device_properties(dev).multi_processor_count
    buf = torch.zeros(8 * (4 << 20), dtype=torch.uint8, device=dev)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    rows = []
    for per_unit, ballast in ((1, 96 << 10), (4, 0)):
        wgs = units * per_unit
        for pattern in ("shared", "distinct"):
            for region in (2 << 20, 4 << 20):
                for depth in (4, 8, 16):
                    step = 512 * depth * 16
                    span = region if pattern == "shared" else region // (wgs // 8) // step * step
                    if span == 0:
                        continue
                    passes = max(1, (256 << 20) // span // per_unit)   # about 64 GB through L1 misses per launch

                    def launch():
                        rc = fn(buf.data_ptr(), buf.numel(), region, span, wgs, passes, int(pattern == "distinct"),
                                depth, ballast, sink.data_ptr(), stream)
                        assert rc == 0, rc

                    for _ in range(2):
                        launch()
                    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    e0.record()
                    for _ in range(5):
                        launch()
                    e1.record()
                    torch.cuda.synchronize()
                    ms = e0.elapsed_time(e1) / 5
                    nbytes = wgs * passes * span
                    rows.append({"workgroups_per_unit": per_unit, "pattern": pattern, "region_mb_per_xcd": region >> 20,
                                 "loads_in_flight_per_lane": depth, "ms": round(ms, 3),
                                 "tb_per_s": round(nbytes / ms / 1e9, 2),
                                 "gb_per_s_per_unit": round(nbytes / ms / 1e6 / units, 1)})
    assert int(sink.item()) == 0
    return {"probe": "l2_resident_reads_through_l1_misses", "compute_units": units, "rows": rows}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=15,
                    help="untimed launches first: the first ten or so run slower (first touch of the outputs, clocks)")
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip amax / dequant side measurements")
    ap.add_argument("--no-calib-sweep", action="store_true",
                    help="skip the mtq.quantize calibration sweep on the Llama-3-8B-shaped decoder")
    ap.add_argument("--calib-seqs", type=int, default=128)
    ap.add_argument("--calib-batch", type=int, default=16)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 1 GiB device copy (a kernel of known traffic for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--probe-l2", action="store_true",
                    help="only measure the L2 -> compute unit read rate with the load-only probe kernel and exit")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py measures one GPU only: this build has no multi-GPU path (got --gpus {a.gpus}); "
              "the path shards by tensor with no exchange", file=sys.stderr)
        sys.exit(2)

    import torch
    from modelopt_amd import _hip

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (torch.cuda.is_available() is False)", file=sys.stderr)
        sys.exit(1)
    _hip.load()  # fail loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    if a.probe_l2:
        print(json.dumps(probe_l2(torch)))
        return

    weights = make_weights(torch, a.layers, dev)
    elems = sum(w.numel() for w in weights)
    aplan = _hip.AbsmaxPlan(weights)
    amax = aplan.run().clone()                   # calibrated per-tensor amax, as export has it
    qplan = _hip.Nvfp4QuantizePlan(weights, amax)
    torch.cuda.synchronize()

    qplan.verify()   # the inputs still sit where the job table says; not repeated per timed step
    wall_ms, dev_ms = timed(torch, lambda: qplan.run(verify=False), a.steps, a.warmup)
    verified = verify_against_restatement(torch, weights, amax, qplan)
    quant_bytes = elems * QUANT_BYTES_PER_ELEM
    value = quant_bytes / (wall_ms * 1e-3) / 1e9
    achieved = quant_bytes / (dev_ms * 1e-3) / 1e9

    out = {
        "metric": "nvfp4_quantize_pack_throughput",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"NVFP4 quantize+pack of Llama-3-8B linear weights, {a.layers} layers x 7 "
                        f"tensors ({len(weights)} tensors, {elems} elements), bf16 N(0,0.02), "
                        "16-element blocks, E4M3 block scales, fp32 global scale from a given amax",
            "elements": elems,
            "algorithmic_bytes": int(quant_bytes),
            "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
            "verified": verified,
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "nvfp4_quantize_multi_kernel",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "launch_ms": round(dev_ms, 4),
            # the same fraction from the committed rocprofv3 kernel trace of the default run (another
            # session, profiler attached): algorithmic bytes / mean duration of its timed dispatches
            "frac_from_profile": (round(quant_bytes / (PROFILE_TIMED_LAUNCH_US * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)
                                  if a.layers == 32 else None),
            # frac = algorithmic bytes / launch_ms / peak; traffic is NOT measured by this run: it is
            # the counter reading of the committed profile of this same command
            "traffic": MEASURED_TRAFFIC_BYTES_32_LAYERS if a.layers == 32 else None,
            "traffic_source": TRAFFIC_SOURCE if a.layers == 32 else None,
        },
    }

    if a.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        big = torch.empty(1 << 30, dtype=torch.uint8, device=dev).zero_()  # push src out of the caches
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst, big

    if not a.no_extras:
        extras = {}
        w_ms, d_ms = timed(torch, aplan.run, a.steps, a.warmup)
        extras["amax_pass"] = {"ms": round(d_ms, 4),
                               "GBps": round(elems * AMAX_BYTES_PER_ELEM / d_ms / 1e6, 1)}

        # amax -> quantize back to back, the quantize launch reading the freshly reduced amax
        qplan_pipe = _hip.Nvfp4QuantizePlan(weights, aplan.acc)

        def pipeline2():
            aplan.run()
            qplan_pipe.run()
        w_ms, d_ms = timed(torch, pipeline2, a.steps, a.warmup)
        extras["amax_plus_quantize_pipeline"] = {
            "ms": round(w_ms, 4),
            "GBps": round(elems * (AMAX_BYTES_PER_ELEM + QUANT_BYTES_PER_ELEM) / w_ms / 1e6, 1)}
        # does a tensor that was just read come back faster (from the 256 MB memory-side cache)?
        # abs-max of one 117 MB weight over and over, against the same kernel walking through the
        # same-shaped weight of every layer (each last touched gigabytes ago)
        big = max(range(len(LAYER_SHAPES)), key=lambda j: weights[j].numel())
        same = [weights[big]] * a.layers
        each = [weights[l * len(LAYER_SHAPES) + big] for l in range(a.layers)]
        acc1 = torch.zeros(1, dtype=torch.float32, device=dev)

        def reread(ts):
            for t in ts:
                _hip.absmax_into(t, acc1, 1, 1, t.numel())
        _, warm_ms = timed(torch, lambda: reread(same), 5, 2)
        _, cold_ms = timed(torch, lambda: reread(each), 5, 2)
        extras["reread_of_one_weight"] = {
            "bytes": weights[big].numel() * 2,
            "just_read_us": round(warm_ms / a.layers * 1e3, 2),
            "read_long_ago_us": round(cold_ms / a.layers * 1e3, 2)}

        # dequant round trip on the first layer's tensors
        packed, wsf, wsf2 = qplan.run()
        n1 = len(LAYER_SHAPES)
        e1 = sum(w.numel() for w in weights[:n1])

        def dequant():
            for i in range(n1):
                _hip.nvfp4_dequantize(packed[i], wsf[i], wsf2[i], 16, torch.bfloat16)
        w_ms, d_ms = timed(torch, dequant, a.steps, a.warmup)
        extras["dequantize_one_layer"] = {
            "ms": round(d_ms, 4), "GBps": round(e1 * DEQUANT_BYTES_PER_ELEM / d_ms / 1e6, 1)}
        # what PyTorch-ROCm users get today: the reference's extensions refuse to build without
        # CUDA, so its NVFP4 weight packing is the eager multi-pass torch code of its QTensor class
        # run on the device; restated inline here on the first layer's seven weights
        def eager_pack():
            for i in range(n1):
                w = weights[i]
                wsf2 = amax[i] / (6.0 * 448.0)
                blocks = w.reshape(*w.shape[:-1], -1, 16)
                bs = blocks.abs().amax(dim=-1).float() / (6.0 * wsf2)
                bs = torch.where(bs == 0, torch.ones_like(bs), bs).to(torch.float8_e4m3fn)
                v = blocks.float() / (bs.float() * wsf2).unsqueeze(-1)
                a = v.abs()
                bounds = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], device=w.device)
                ordv = torch.searchsorted(bounds, a, out_int32=True)
                odd = (a == 0.75) | (a == 1.75) | (a == 3.5)
                codes = ((v < 0).to(torch.uint8) << 3) + (ordv + odd).to(torch.uint8)
                codes = codes.reshape(*w.shape)
                (codes[..., 1::2] << 4) | codes[..., 0::2]
        w_ms, d_ms = timed(torch, eager_pack, 3, 1)
        extras["eager_torch_pack_one_layer_on_gpu"] = {
            "ms": round(d_ms, 4), "GBps": round(e1 * QUANT_BYTES_PER_ELEM / d_ms / 1e6, 1)}

        # plain device copy of 4 GiB: the read + write rate the memory system sustains
        src = torch.empty(1 << 32, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        w_ms, d_ms = timed(torch, lambda: dst.copy_(src), 5, 2)
        extras["device_copy_4GiB"] = {"ms": round(d_ms, 4), "GBps": round(2 * src.numel() / d_ms / 1e6, 1)}
        del src, dst

        with contextlib.redirect_stdout(sys.stderr):   # the calibration algorithms print progress
            extras["single_tensor_configs"] = single_tensor_configs(torch, a.steps, a.warmup)
        extras["secondary_kernels"] = secondary_kernels(torch, a.steps, a.warmup)
        out["extras"] = extras

    if not a.no_calib_sweep:
        del weights, aplan, qplan
        torch.cuda.empty_cache()
        with contextlib.redirect_stdout(sys.stderr):
            out["calib_sweep"] = calib_sweep(torch, a.layers, a.calib_seqs, a.calib_batch)

    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch)
        if not a.no_extras:
            with contextlib.redirect_stdout(sys.stderr):
                out.setdefault("extras", {})["cpu_reference_path"] = cpu_reference_configs(torch)
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
