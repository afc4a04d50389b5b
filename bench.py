#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2] [--no-cpu-baseline]

A step is one pass of  OnlineHadamard -> Quantizer -> Linear4bit  (Hadamard + per-token int4
quantise + int4 GEMM + fp16 dequant) over one batch of seeded synthetic tokens already resident in
HBM.  Workloads (shapes of Llama-2; inputs as in the reference's qlinear benchmark but with the
outlier channels that motivate the Hadamard):
    c1  q_proj 7B      X [2048, 4096]   W int4 [4096, 4096]     no online Hadamard
    c1n the same with the RMSNorm in front of the quantiser (fused RMSNorm + Quantizer kernel)
    c1o o_proj 7B      attention output [2048, 32, 128] -> Hadamard across the 32 heads -> Quantizer
        (one fused kernel) -> W int4 [4096, 4096]
    c2  down_proj 7B   X [2048, 11008]  W int4 [4096, 11008]    Hadamard FWHT(64) (x) had_172   (default)
    c3d down_proj 7B, prefill 16 x 2048 tokens  X [32768, 11008]
    c3  the four linears of a 7B decoder layer at 32768 tokens as ONE step: fused qkv 4096->12288, o 4096->4096,
        gate_up 4096->22016 (Quantizer in front of each) and down 11008->4096 (Hadamard+Quantizer): 13.26 TOP
        (c3a, c3b, c3c: the first three on their own)
    c4  down_proj 70B decode  X [64, 28672]  W int4 [8192, 28672]  Hadamard FWHT(1024) (x) had_28
        (c4m1, c4m8: 1 / 8 tokens; c4g1, c4g8, c4g64: gate_up W int4 [57344, 8192])
    c5  KV-cache write path of one layer: K and V [32, 4096, 8, 128] fp16 -> asymmetric int4 per head
        vector (K through the head-dimension Hadamard first); metric GB/s of algorithmic bytes
Decode workloads (M <= 64) rotate among several copies of the weights so that they are streamed from
HBM rather than from the 256 MB last-level cache.
Prints ONE JSON line on stdout (metric = TOPS of the whole step, 2.M.N.K / t).
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

WORKLOADS = {
    #        M      K      N     hadamard
    "c1": (2048, 4096, 4096, False),
    "c1n": (2048, 4096, 4096, False),       # input_layernorm -> Quantizer -> q_proj
    "c1o": (2048, 4096, 4096, False),       # attention output -> Hadamard over heads -> Quantizer -> o_proj
    "c2": (2048, 11008, 4096, True),
    "c3d": (32768, 11008, 4096, True),
    "c3a": (32768, 4096, 12288, False),     # fused qkv
    "c3b": (32768, 4096, 4096, False),      # o_proj
    "c3c": (32768, 4096, 22016, False),     # gate_up
    "c3": (0, 0, 0, False),                 # the whole layer set (separate code path below)
    "c4m32": (32, 28672, 8192, True),
    "c4g32": (32, 8192, 57344, False),
    "c4": (64, 28672, 8192, True),          # decode, 70B down_proj
    "c4m1": (1, 28672, 8192, True),
    "c4m8": (8, 28672, 8192, True),
    "c4g1": (1, 8192, 57344, False),        # decode, 70B gate_up (input already quantised upstream: no Hadamard)
    "c4g8": (8, 8192, 57344, False),
    "c4g64": (64, 8192, 57344, False),
    "c5": (0, 0, 0, False),                 # KV-cache quantisation (separate code path below)
}
INT8_MFMA_PEAK_TOPS = 5000.0     # MI355X dense int8, published
HBM_PEAK_GBS = 8000.0

# HBM-side traffic of the GEMM kernel per launch, from two `rocprofv3 --pmc` runs of this script
# (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch, averaged over the run's dispatches of that kernel).
# The same counters read 131083.8 KiB / 262144.0 KiB for a plain 256 MiB device copy
# (--copy-calibration: 262144 KiB read and written), so reads are scaled by 2.0 and writes by 1.0.
FETCH_SCALE, WRITE_SCALE = 262144.0 / 131083.8, 262144.0 / 262144.0
TRAFFIC_KIB = {
    #        FETCH_SIZE   WRITE_SIZE
    "c1": (16551.0, 16384.0),
    "c1o": (16590.5, 16384.0),
    "c2": (44210.0, 16384.0),
    "c3d": (528791.7, 262144.0),
    "c4": (62375.6, 1024.0),
    "c4m1": (57494.0, 16.0),
    "c4g64": (124423.7, 7168.0),
    "c5": (131145.3, 69774.2),              # kv_had128_kernel (K cache), per launch
}


def synth_x(m, k, seed=0, outliers=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g)
    if outliers:
        idx = torch.randperm(k, generator=g)[: -(-k // 100)]
        x[:, idx] *= 20
    return x.half()


def synth_w(n, k, seed=1):
    """N(0, 0.02) weights ("already rotated"), per-row fp16 scale amax/7, RTN codes, packed."""
    from quarot_amd.functional import pack_i4
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(n, k, generator=g) * 0.02).half()
    s = (w.abs().amax(dim=1, keepdim=True).float() / 7).half()
    codes = torch.clamp(torch.round((w.float() / s.float()).half().float()), -8, 7).to(torch.int8)
    return pack_i4(codes), s


def cpu_baseline(x, w_packed, w_scales, hadamard, m, n, k, budget_rows, rmsnorm=False, heads=0):
    """The reference's CPU path (torch Hadamard + quant + integer matmul + dequant) on a bounded
    row sample of the same workload, all host threads; TOPS scaled to the sample's own work."""
    from oracle import cpu_baseline as cb
    rows = min(m, budget_rows)
    xs = x[:rows].clone()
    wc = cb.unpacked_codes(w_packed.numpy())
    ws = w_scales.view(-1)
    torch.set_num_threads(os.cpu_count() or 1)
    cb.linear4bit_path(xs[:2], wc[:64], ws[:64], hadamard, rmsnorm, heads)   # warm-up
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        cb.linear4bit_path(xs, wc, ws, hadamard, rmsnorm, heads)
        times.append(time.perf_counter() - t0)
    t = float(np.median(times))
    return {"value": round(2.0 * rows * n * k / t / 1e12, 5), "unit": "TOPS", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"first {rows} of {m} rows, full N and K, median of 3 ({t * 1e3:.0f} ms); torch "
                      + ("fp32 RMSNorm + " if rmsnorm else "fp32 matmul_hadU + " if hadamard
                         else "fp32 matmul_hadU over heads + " if heads else "")
                      + "fp16 sym quant + int32 torch matmul + fp16 dequant"}


def bench_kv(args, dev):
    """Workload c5: quantise K (Hadamard over the head dimension, then asymmetric int4) and V
    (asymmetric int4) of one layer, [32, 4096, 8, 128] fp16 each, resident in HBM."""
    from quarot_amd.transformers import kv_cache as kv
    shape = (32, 4096, 8, 128)

    def synth(seed):
        g = torch.Generator().manual_seed(seed)
        t = torch.randn(shape, generator=g)
        mask = torch.rand(shape, generator=torch.Generator().manual_seed(5)) < 0.005
        t[mask] *= 15
        return t.half()

    k_cpu, v_cpu = synth(4), synth(6)
    k, v = k_cpu.to(dev), v_cpu.to(dev)
    vectors = k.numel() // 128
    bytes_one = 2 * k.numel() + vectors * (64 + 4)          # fp16 in; codes + scale + zero out
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]

    def step(ev=None):
        if ev is not None:
            ev[0].record()
        kq = kv.asym_quantize_and_pack_i4(k, hadamard=True)
        if ev is not None:
            ev[1].record()
        vq = kv.asym_quantize_and_pack_i4(v, hadamard=False)
        kd = kv.unpack_i4_and_asym_dequantize(*kq)          # the round trip of the config
        vd = kv.unpack_i4_and_asym_dequantize(*vq)
        return kd, vd

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(evs[i])
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    k_ms = float(np.mean([a.elapsed_time(b) for a, b in evs]))
    traffic = None
    if TRAFFIC_KIB.get("c5"):
        f, w = TRAFFIC_KIB["c5"]
        traffic = round((f * FETCH_SCALE + w * WRITE_SCALE) * 1024)
    roof = {"bound": "hbm", "achieved": round(bytes_one / (k_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "traffic": traffic}
    roof["frac"] = round(roof["achieved"] / roof["peak"], 4)
    roof["kernel"] = "kv_had128_kernel (K cache: Hadamard on the matrix cores + asymmetric int4)"
    roof["kernel_ms"] = round(k_ms, 4)
    out = {
        "metric": "KV-cache int4 quantise + dequantise GB/s (K with Hadamard, V)", "value": round(4 * bytes_one / (ms * 1e-3) / 1e9, 1),
        "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16 -> u4 (fp32 Hadamard, fp16 quantiser)",
        "data": "synthetic",
        "config": {"workload": "c5: K and V [32,4096,8,128] fp16 (0.5% elements x15) -> asym int4 + fp16 scale/zero per head vector "
                               "-> fp16 again (four launches)",
                   "vectors_per_tensor": vectors, "head_dim": 128},
        "roofline": roof,
    }
    if not args.no_cpu_baseline:
        from oracle import quarot_oracle as o
        n = vectors // 256                                   # 4096 vectors of each tensor
        ks, vs = k_cpu.reshape(-1, 128)[:n].numpy(), v_cpu.reshape(-1, 128)[:n].numpy()
        t0 = time.perf_counter()
        o.kv_asym_quant(o.kv_hadamard(ks))
        o.kv_asym_quant(vs)
        t = time.perf_counter() - t0
        sample_bytes = 2 * (2 * ks.size + n * 68)
        out["cpu_baseline"] = {"value": round(sample_bytes / t / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"first {n} of {vectors} vectors of each tensor ({t * 1e3:.0f} ms); numpy oracle "
                                         f"(fp32 FWHT + fp16 asymmetric quantiser)"}
    print(json.dumps(out))


def bench_layer(args, dev):
    """Workload c3: the four W4A4 linears of a Llama-2-7B decoder layer at M = 32768 tokens (prefill,
    16 x 2048) as one step; inputs of each linear are separate seeded tensors resident in HBM."""
    import quarot_amd
    m = 32768
    parts = [("qkv", 4096, 12288, False, 0), ("o", 4096, 4096, False, 10), ("gate_up", 4096, 22016, False, 20),
             ("down", 11008, 4096, True, 30)]
    mods = []
    for name, k, n, had, seed in parts:
        x = synth_x(m, k, seed=seed, outliers=True).to(dev)
        w, sw = synth_w(n, k, seed=seed + 1)
        lin = quarot_amd.nn.Linear4bit(k, n).half().to(dev)
        lin.weight.copy_(w.to(dev))
        lin.weight_scales.copy_(sw.to(dev))
        front = (quarot_amd.nn.OnlineHadamardQuantizer(k) if had else quarot_amd.nn.Quantizer()).to(dev)
        mods.append((x, front, lin))
    ops = sum(2.0 * m * k * n for _, k, n, _, _ in parts)
    evs = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in parts]
           for _ in range(args.steps)]

    def step(ev=None):
        for j, (x, front, lin) in enumerate(mods):
            p = front(x)
            if ev is not None:
                ev[j][0].record()
            y = quarot_amd.linear_i4(p.quantized_x, p.scales_x, lin.weight, lin.weight_scales, None)
            if ev is not None:
                ev[j][1].record()
            del y                                           # 0.8 - 1.4 GB each: returned to the pool before the next one

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(evs[i])
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    gemm = [float(np.mean([evs[i][j][0].elapsed_time(evs[i][j][1]) for i in range(args.steps)])) for j in range(len(parts))]
    gemm_ms = sum(gemm)
    roof = {"bound": "mfma", "achieved": round(ops / (gemm_ms * 1e-3) / 1e12, 1), "peak": INT8_MFMA_PEAK_TOPS,
            "unit": "TFLOP/s", "traffic": None}
    roof["frac"] = round(roof["achieved"] / roof["peak"], 4)
    roof["kernel"] = "gemm_sp256_kernel (int4 GEMM + dequant epilogue), four launches"
    roof["kernel_ms"] = round(gemm_ms, 4)
    roof["per_linear"] = {name: {"ms": round(t, 4), "TOPS": round(2.0 * m * k * n / (t * 1e-3) / 1e12, 1)}
                          for (name, k, n, _, _), t in zip(parts, gemm)}
    out = {
        "metric": "Linear4bit TOPS (had+quant+GEMM)", "value": round(ops / (ms * 1e-3) / 1e12, 2), "unit": "TOPS", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int4 x int4 -> int32 (int8 MFMA), fp16 scales", "data": "synthetic",
        "config": {"workload": "c3: Llama-2-7B decoder-layer linear set at M=32768 (qkv 4096->12288, o 4096->4096, "
                               "gate_up 4096->22016, down 11008->4096 with online Hadamard), W4A4",
                   "M": m, "total_TOP": round(ops / 1e12, 2)},
        "roofline": roof,
    }
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--graph", action="store_true",
                    help="time replays of the step captured in a HIP graph (decode steps are host-launch-bound when "
                         "launched eagerly from Python); the first replay is checked against the eager result")
    ap.add_argument("--cpu-rows", type=int, default=64)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="instead of a workload, run a plain 256 MiB device copy 20 times (known traffic: 256 MiB read, "
                         "256 MiB written per launch) for scaling the profiler's FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path is data-parallel over tokens with no exchange; "
              "run one process per GPU and add the values (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    import quarot_amd
    from quarot_amd import _lib
    if not _lib.LIB_PATH.exists():
        from quarot_amd import build
        build.build(verbose=False)
    _lib.lib()
    dev = torch.device("cuda:0")
    if args.copy_calibration:
        src = torch.randint(0, 255, (256 * 1024 * 1024,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(20):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": {"launches": 20, "read_bytes": src.numel(), "written_bytes": src.numel()}}))
        return
    if args.workload == "c5":
        return bench_kv(args, dev)
    if args.workload == "c3":
        return bench_layer(args, dev)
    m, k, n, hadamard = WORKLOADS[args.workload]
    x_cpu = synth_x(m, k, seed=0, outliers=True)
    w_cpu, sw_cpu = synth_w(n, k, seed=1)
    x = x_cpu.to(dev)
    lin = quarot_amd.nn.Linear4bit(k, n).half().to(dev)
    lin.weight.copy_(w_cpu.to(dev))
    lin.weight_scales.copy_(sw_cpu.to(dev))
    rmsnorm = args.workload == "c1n"
    heads = 32 if args.workload == "c1o" else 0
    if heads:
        x = x.view(m, heads, k // heads)                    # as attention writes it: [tokens, heads, head_dim]
    front = (quarot_amd.nn.OnlineHadamardQuantizer(k) if hadamard else quarot_amd.nn.RMSNormQuantizer(k) if rmsnorm
             else quarot_amd.nn.HeadsHadamardQuantizer(heads) if heads else quarot_amd.nn.Quantizer()).to(dev)
    # decode: identical weight copies used round-robin, more bytes in total than the last-level cache
    copies = [lin.weight]
    if m <= 64:
        while sum(c.numel() for c in copies) < 640 * 1024 * 1024:
            copies.append(lin.weight.clone())
    state = {"i": 0}

    # decode steps are bound by the host: front kernel and GEMM go out in ONE call into the library
    # (same two launches; the per-kernel events of the prefill workloads need the two-call form)
    one_call = m <= 64 and not rmsnorm and not heads
    had_args = (front.had_rem_dim, front.rem_dim) if hadamard else (None, 0)

    def step(ev=None):
        if one_call and ev is None:
            w = copies[state["i"] % len(copies)]
            state["i"] += 1
            return quarot_amd.quantized_linear(x, w, lin.weight_scales, lin.bias, *had_args)
        p = front(x)
        if ev is not None:
            ev[0].record()
        w = copies[state["i"] % len(copies)]
        state["i"] += 1
        y = quarot_amd.linear_i4(p.quantized_x, p.scales_x, w, lin.weight_scales, lin.bias)
        if ev is not None:
            ev[1].record()
        return y

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    torch.cuda.synchronize()
    if args.graph:
        # one graph per weight copy would defeat the rotation: capture a run of len(copies) steps
        state["i"] = 0
        want = step().clone()
        state["i"] = 0
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            outs = [step() for _ in range(len(copies))]
        graph.replay()
        torch.cuda.synchronize()
        if not torch.equal(outs[0], want):
            raise RuntimeError("graph replay differs from the eager step")
        reps = max(1, args.steps // len(copies))
        t0 = time.perf_counter()
        for _ in range(reps):
            graph.replay()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / (reps * len(copies))
        for i in range(min(args.steps, 20)):                # GEMM time from eager launches (events cannot go into the graph)
            step(events[i])
        torch.cuda.synchronize()
        gemm_ms = float(np.mean([a.elapsed_time(b) for a, b in events[:min(args.steps, 20)]]))
    else:
        t0 = time.perf_counter()
        for i in range(args.steps):
            step(None if one_call else events[i])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        ms = (t1 - t0) * 1e3 / args.steps
        # (decode: the GEMM is timed further down from back-to-back launches)
        gemm_ms = 0.0 if one_call else float(np.mean([a.elapsed_time(b) for a, b in events]))
    ops = 2.0 * m * n * k
    value = ops / (ms * 1e-3) / 1e12

    # staged (reference-shaped) chain for comparison, untimed in `value`
    staged_front = (torch.nn.Sequential(quarot_amd.nn.OnlineHadamard(k), quarot_amd.nn.Quantizer()) if hadamard
                    else torch.nn.Sequential(quarot_amd.nn.RMSNorm(k), quarot_amd.nn.Quantizer()) if rmsnorm
                    else quarot_amd.nn.Quantizer()).to(dev)
    if heads:
        # the reference's sequence: transform on the transposed view, transpose back, reshape, quantise
        had_heads, quant = quarot_amd.nn.OnlineHadamard(heads).to(dev), quarot_amd.nn.Quantizer()
        staged_front = lambda t: quant(had_heads(t.transpose(-1, -2)).transpose(-1, -2).reshape(m, k).contiguous())
    for _ in range(3):
        lin(staged_front(x))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(max(10, args.steps // 4)):
        lin(staged_front(x))
    torch.cuda.synchronize()
    staged_ms = (time.perf_counter() - t0) * 1e3 / max(10, args.steps // 4)

    decode = m <= 64
    if decode:
        # a decode step is launch-bound on the host, so events around one launch would time an idle
        # GPU: time a back-to-back batch of the GEMM launch instead (weights still rotating)
        p = front(x)
        reps = 60
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for phase in range(2):
            if phase == 1:
                e0.record()
            for i in range(reps):
                quarot_amd.linear_i4(p.quantized_x, p.scales_x, copies[i % len(copies)], lin.weight_scales, lin.bias)
        e1.record()
        torch.cuda.synchronize()
        gemm_ms = e0.elapsed_time(e1) / reps
    traffic = None
    if args.workload in TRAFFIC_KIB:
        f, w = TRAFFIC_KIB[args.workload]
        traffic = round((f * FETCH_SCALE + w * WRITE_SCALE) * 1024)
    if decode:
        algo_bytes = n * k / 2 + m * k / 2 + 2 * m + 2 * n + 2 * m * n
        roof = {"bound": "hbm", "achieved": round(algo_bytes / (gemm_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "traffic": traffic}
    else:
        roof = {"bound": "mfma", "achieved": round(ops / (gemm_ms * 1e-3) / 1e12, 1), "peak": INT8_MFMA_PEAK_TOPS,
                "unit": "TFLOP/s", "traffic": traffic}
    roof["frac"] = round(roof["achieved"] / roof["peak"], 4)
    t256 = ((m + 255) // 256) * ((n + 255) // 256)
    t128 = ((m + 127) // 128) * ((n + 255) // 256)
    if m <= 4:
        kern = "gemv_i4_kernel"
    elif decode:
        kern = "gemm_ks_kernel<64,256>" if m > 16 and (n + 255) // 256 >= 128 else "decode_i4_kernel"
    elif t128 >= 128:       # the library's choice between its two pipelined kernels, by rounds of tiles
        kern = "gemm_sp256_kernel" if (t256 + 255) // 256 <= ((t128 + 255) // 256) * 0.61 else "gemm_spk_kernel"
    else:
        kern = "gemm_ks_kernel<64,256>"
    roof["kernel"] = kern
    roof["kernel"] += " (int4 GEMM + dequant epilogue)"
    roof["kernel_ms"] = round(gemm_ms, 4)

    out = {
        "metric": "Linear4bit TOPS (had+quant+GEMM)", "value": round(value, 2), "unit": "TOPS", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int4 x int4 -> int32 (int8 MFMA), fp16 scales",
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: Linear4bit X[{m},{k}] fp16 (1% outlier channels x20) . W int4[{n},{k}]"
                               + (" with online Hadamard" if hadamard else " behind RMSNorm" if rmsnorm
                                  else f" behind the Hadamard across {heads} heads" if heads else ""),
                   "M": m, "K": k, "N": n,
                   "path": ("fused Hadamard+quantise kernel" if hadamard else "fused RMSNorm+quantise kernel" if rmsnorm
                            else "fused heads-Hadamard+quantise kernel" if heads else "quantise kernel")
                           + ", fused GEMM+dequant kernel" + (" (one library call per step)" if one_call else ""),
                   "staged_reference_api_ms": round(staged_ms, 4), "launch": "hip graph replay" if args.graph else "eager"},
        "roofline": roof,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(x_cpu, w_cpu, sw_cpu, hadamard, m, n, k, args.cpu_rows, rmsnorm, heads)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
