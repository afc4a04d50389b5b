#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--repeats R] [--workload c2]
                    [--no-cpu-baseline] [--no-per-config] [--graph]

A step is one pass of  OnlineHadamard -> Quantizer -> Linear4bit  (Hadamard + per-token int4
quantise + int4 GEMM + fp16 dequant) over one batch of seeded synthetic tokens already resident in
HBM.  Workloads (shapes of Llama-2; inputs as in the reference's qlinear benchmark but with the
outlier channels that motivate the Hadamard):
    c1  q_proj 7B      X [2048, 4096]   W int4 [4096, 4096]     no online Hadamard
    c1n the same with the RMSNorm in front of the quantiser (fused RMSNorm + Quantizer kernel)
    c1o o_proj 7B      attention output [2048, 32, 128] -> Hadamard across the 32 heads -> Quantizer
        (one fused kernel) -> W int4 [4096, 4096]
    c2  down_proj 7B   X [2048, 11008]  W int4 [4096, 11008]    Hadamard FWHT(64) (x) had_172   (default)
    c2_fp32had  the same with OnlineHadamard(force_fp32=True): the reference benchmark's "+FP32had" column
    c3  the four linears of a 7B decoder layer at 32768 tokens as ONE step: fused qkv 4096->12288, o 4096->4096,
        gate_up 4096->22016 (Quantizer in front of each) and down 11008->4096 (Hadamard+Quantizer): 13.26 TOP
        (c3a, c3b, c3c, c3d: each of them on its own)
    c4mT  down_proj 70B decode  X [T, 28672]  W int4 [8192, 28672]  Hadamard FWHT(1024) (x) had_28, T in 1, 8, 32, 64
    c4gT  gate_up 70B decode    X [T, 8192]   W int4 [57344, 8192]
    c5  KV-cache write path of one layer: K and V [32, 4096, 8, 128] fp16 -> asymmetric int4 per head
        vector (K through the head-dimension Hadamard first) -> fp16 again; metric GB/s of algorithmic bytes
    c6  one decode step on the paged int4 cache that c5's tensors fill (32 sequences x 4096 tokens x 8 heads x 128,
        pages of 16): quantise-and-append of the new token's K / V, Hadamard of the query, attention over the
        cache; metric GB/s of the cache bytes read (c6b: 1 sequence x 2048 tokens x 32 heads, the default of
        benchmarks/qattention_benchmark.py:9-13,129-139)
    b13v, b70v, b13d, b70d  the other sizes of the reference's benchmarks/qlinear_benchmark.py:8-18 at 2048 tokens
        (5120->5120, 8192->8192 with the Hadamard in front; down_proj 13824->5120 and 28672->8192 with it)
Decode workloads (M <= 64) rotate among several copies of the weights so that they are streamed from
HBM rather than from the 256 MB last-level cache.

Timing follows benchmarks/qlinear_benchmark.py:20-40,88-113: warm-up, then a loop of K steps between two
synchronisations, repeated R times; the step time is the median of the R loops and the spread is
reported as mean +- 1.96 sigma.  Nothing but the step's own launches is inside a timed loop; the time
of each kernel comes from a separate pass: back-to-back launches of that kernel alone between one pair
of HIP events on the launch stream, queued behind a few milliseconds of device copies so that the
host's per-call cost (longer than the short kernels) does not show.

Prints ONE JSON line on stdout.  The default run measures the headline workload (c2) and, in
`per_config`, every other benchmark configuration with fewer repeats.
"""
import argparse
import json
import os
import re
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

WORKLOADS = {
    #        M      K      N     front
    "c1": (2048, 4096, 4096, "quant"),
    "c1n": (2048, 4096, 4096, "rmsnorm"),     # input_layernorm -> Quantizer -> q_proj
    "c1o": (2048, 4096, 4096, "heads"),       # attention output -> Hadamard over heads -> Quantizer -> o_proj
    "c2": (2048, 11008, 4096, "had"),
    "c2_fp32had": (2048, 11008, 4096, "had32"),   # the "+FP32had" chain of benchmarks/qlinear_benchmark.py:68-73 (force_fp32=True)
    "c3a": (32768, 4096, 12288, "quant"),     # fused qkv
    "c3b": (32768, 4096, 4096, "quant"),      # o_proj
    "c3c": (32768, 4096, 22016, "quant"),     # gate_up
    "c3d": (32768, 11008, 4096, "had"),       # down_proj
    "c3": None,                               # the whole layer set as one step
    "c5": None,                               # KV-cache quantisation
    "c6": None,                               # decode attention over the paged int4 cache of config 5's size
    "c6b": None,                              # the same at the reference benchmark's default: 1 sequence x 2048 tokens x 32 heads
    "b13v": (2048, 5120, 5120, "had"),        # qlinear_benchmark.py model_sizes / mlp_sizes at 13B and 70B
    "b70v": (2048, 8192, 8192, "had"),
    "b13d": (2048, 13824, 5120, "had"),
    "b70d": (2048, 28672, 8192, "had"),
}
for _t in (1, 8, 32, 64):
    WORKLOADS[f"c4m{_t}"] = (_t, 28672, 8192, "had")      # decode, 70B down_proj
    WORKLOADS[f"c4g{_t}"] = (_t, 8192, 57344, "quant")    # decode, 70B gate_up
PER_CONFIG = ["c1", "c2_fp32had", "c3", "c4g1", "c4g8", "c4g32", "c4g64", "c4m1", "c4m8", "c4m32", "c4m64", "c5", "c6", "b13v", "b70v", "b13d", "b70d",
              "c2_fp6", "c3_fp6"]
INT8_MFMA_PEAK_TOPS = 5000.0     # MI355X dense int8, published
FP6_MFMA_PEAK_TOPS = 10100.0     # MI355X dense fp6, published (the opt-in exact int4 GEMM on 6-bit operands)
HBM_PEAK_GBS = 8000.0

# Profile summaries that hold the FETCH_SIZE / WRITE_SIZE readings of a workload's dominant kernel
# ("traffic_kib: kernel=<substring> fetch=<KiB per dispatch> write=<KiB per dispatch>") and the copy
# calibration ("traffic_scale: fetch=<factor> write=<factor>").
PROFILE_OF = {
    "c1": "gemm_spk_c1_q_proj_7b.txt", "c1n": "rmsnorm_quant_rows_c1n_q_proj_7b.txt",
    "c1o": "heads_hadamard_quant_c1o_o_proj_7b.txt", "c2": "gemm_spk_and_hadamard_m64r_c2_down_proj_7b.txt",
    "c2_fp32had": "gemm_spk_and_hadamard_m64_fp32_c2_down_proj_7b.txt",
    "c3": "gemm_sp256_c3_prefill_layer_set_32768_tokens.txt",
    "c4g1": "quant_gemv_c4g1_decode_70b_gate_up.txt",
    "c4g8": "decode_xs_c4g8_decode_8_tokens_70b_gate_up.txt", "c4g32": "decode_xs_c4g32_decode_32_tokens_70b_gate_up.txt",
    "c4g64": "decode_xs_c4g64_decode_64_tokens_70b_gate_up.txt", "c4m1": "bm_gemv_c4m1_decode_70b_down_proj.txt",
    "c4m8": "decode_i4_c4m8_decode_8_tokens_70b_down_proj.txt", "c4m32": "decode_i4_c4m32_decode_32_tokens_70b_down_proj.txt",
    "c4m64": "decode_xs_sliced_c4m64_decode_64_tokens_70b_down_proj.txt", "c5": "kv_quant_c5_kv_cache_32x4096x8x128.txt",
    "c6": "paged_decode_i4_c6_decode_attention_32x4096x8x128.txt",
    "b13v": "gemm_sp256_b13v_2048x5120x5120.txt", "b70v": "gemm_sp256_b70v_2048x8192x8192.txt",
    "b13d": "gemm_sp256_b13d_2048x13824x5120.txt", "b70d": "gemm_sp256_b70d_2048x28672x8192.txt",
    "c2_fp6": "gemm_f6_c2_down_proj_7b.txt", "c3d_fp6": "gemm_f6_c3d_down_proj_32768_tokens.txt",
    "c3_fp6": "gemm_f6_c3_prefill_layer_set_32768_tokens.txt",
}


def traffic_from_profile(workload, kernel):
    """(bytes per launch, source file) from the committed rocprofv3 summary of this workload, scaled by
    the copy calibration; (None, None) when no summary carries the readings."""
    pdir = os.path.join(ROOT, "profiles")
    name = PROFILE_OF.get(workload)
    try:
        text = open(os.path.join(pdir, name)).read() if name else ""
        cal = open(os.path.join(pdir, "copy_calibration_256MiB.txt")).read()
    except OSError:
        return None, None
    sc = re.search(r"traffic_scale:\s*fetch=([\d.]+)\s+write=([\d.]+)", cal)
    if not sc:
        return None, None
    kib, seen = 0.0, set()                       # a dominant "kernel" of two launches (K-sliced decode) sums both
    for m in re.finditer(r"traffic_kib:\s*kernel=(\S+)\s+fetch=([\d.]+)\s+write=([\d.]+)", text):
        if m.group(1) in kernel and m.group(1) not in seen:
            seen.add(m.group(1))
            kib += float(m.group(2)) * float(sc.group(1)) + float(m.group(3)) * float(sc.group(2))
    if seen:
        return round(kib * 1024), f"profiles/{name}"
    return None, None


def synth_x(m, k, seed=0, outliers=True, device="cpu"):
    g = torch.Generator(device=device).manual_seed(seed)
    x = torch.randn(m, k, generator=g, device=device)
    if outliers:
        idx = torch.randperm(k, generator=g, device=device)[: -(-k // 100)]
        x[:, idx] *= 20
    return x.half()


def synth_w(n, k, seed=1, device="cpu"):
    """N(0, 0.02) weights ("already rotated"), per-row fp16 scale amax/7, RTN codes, packed."""
    from quarot_amd.functional import pack_i4
    g = torch.Generator(device=device).manual_seed(seed)
    w = (torch.randn(n, k, generator=g, device=device) * 0.02).half()
    s = (w.abs().amax(dim=1, keepdim=True).float() / 7).half()
    codes = torch.clamp(torch.round((w.float() / s.float()).half().float()), -8, 7).to(torch.int8)
    return pack_i4(codes), s


MIN_SPAN_MS = 150.0      # timed loops keep coming until they span this much GPU time (see timed_loops)
MAX_LOOPS = 600
_RAMP = {}


def timed_loops(step, steps, warmup, repeats, min_span_ms=MIN_SPAN_MS):
    """warm-up, then loops of exactly `steps` steps, each between two synchronisations and holding nothing but
    the step's own launches.  Returns per-step milliseconds of the LAST `repeats` loops.
    After an idle period this GPU needs about 30 ms of continuous work before its clocks settle (20-step loops
    of the default workload from a cold start: 92, 104, 98, 94, 91, 89, 87, 86, 84 ... 81 us per step, level from
    the twentieth loop on), so with short loops the first ones measure the ramp, not the kernels: loops are run
    until they span `min_span_ms` in all (at least `repeats`, at most MAX_LOOPS), and the last `repeats` are the
    measurement.  The first loop's time and the number of loops are reported next to it.  (The context columns,
    measured right behind the main loops on a GPU that is already at its clocks, pass min_span_ms = 0.)"""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    out, span = [], 0.0
    while len(out) < repeats or (span < min_span_ms and len(out) < MAX_LOOPS):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) * 1e3
        out.append(dt / steps)
        span += dt
    _RAMP.update(first_loop_ms=round(out[0], 5), loops_run=len(out))
    return out[-repeats:]


def spread(ms_list):
    a = np.asarray(ms_list, dtype=np.float64)
    return {"median_ms": round(float(np.median(a)), 5), "mean_ms": round(float(a.mean()), 5),
            "ci95_ms": round(float(1.96 * a.std()), 5), "min_ms": round(float(a.min()), 5), "repeats": int(a.size),
            "loops_run": _RAMP.get("loops_run", int(a.size)), "first_loop_ms": _RAMP.get("first_loop_ms")}


_BLOCKER = {}


def kernel_ms(fn, reps):
    """Average duration of one launch of fn(): `reps` back-to-back launches between one pair of HIP events
    on the launch stream.  The host needs longer to issue a launch than a short kernel runs, and an idle
    GPU would then time the host: a device copy is queued first, so that the events and every launch are
    already waiting in the stream when the GPU reaches them.  The copy is kept as short as that allows
    (~16 us of host time per launch to cover: 0.8 ms for 50 launches) and follows 20 ms of the function itself:
    the GPU's clocks follow what it has been doing for the last milliseconds, and behind 6-13 ms of copying --
    the blocker this pass used to queue -- the prefill GEMMs ran 8-11 % slower than in the loop of the step
    (68.8 against 63.3 us for the default workload's, whose step loop -- 83.1 us -- is the sum of 18.4, 63.3
    and two launch boundaries; behind a sleeping kernel likewise: 71 us)."""
    if "src" not in _BLOCKER:
        _BLOCKER["src"] = torch.empty(1 << 32, dtype=torch.uint8, device="cuda")
        _BLOCKER["dst"] = torch.empty(1 << 32, dtype=torch.uint8, device="cuda")
    fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.02:                   # (20 ms of GPU time: the host would queue far more unsynchronised)
        for _ in range(8):
            fn()
        torch.cuda.synchronize()
    nbytes = min(1 << 32, max(1 << 30, reps * (42 << 20)))      # the copy moves ~2.6 GB per millisecond
    _BLOCKER["dst"][:nbytes].copy_(_BLOCKER["src"][:nbytes])
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps


def mfma_i8_rate(pattern, launches=10, iters=4096, workgroups=1024):
    """TOP/s of the library's register-only loop of v_mfma_i32_32x32x32_i8 (qr_calib_mfma_i8: four waves per
    workgroup, four accumulator chains per wave, no memory access): what the matrix pipe sustains with nothing
    else going on.  pattern 0: zero operands, 1: random int4 codes as the GEMMs feed them, 2: random int8, 3: random int4 codes as
    sign-extended int8."""
    from quarot_amd import _lib
    L = _lib.lib()
    dev = torch.device("cuda:0")
    out = torch.empty(workgroups * 256, dtype=torch.int32, device=dev)
    st = _lib.stream_ptr(dev)
    ops = workgroups * 4 * iters * 16 * 65536.0
    return ops / (kernel_ms(lambda: _lib.check(L.qr_calib_mfma_i8(pattern, iters, workgroups, out.data_ptr(), st)), launches) * 1e-3) / 1e12


def gpu_clock_mhz():
    """Current shader clock from rocm-smi (None when the tool is missing or prints something else)."""
    import subprocess
    try:
        txt = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=20).stdout
    except (OSError, subprocess.SubprocessError):
        return None
    m = re.search(r"sclk clock level:?\s*\d*:?\s*\((\d+)Mhz\)", txt, flags=re.I)
    return int(m.group(1)) if m else None


def mfma_ceiling(seconds):
    """The int8 matrix instruction alone (no loads, no LDS, no unpacking): short bursts, then `seconds` of back-to-back
    launches per operand pattern with the shader clock sampled from rocm-smi while they run."""
    import threading
    from quarot_amd import _lib
    L = _lib.lib()
    dev = torch.device("cuda:0")
    res = {"instruction": "v_mfma_i32_32x32x32_i8", "published_peak_TOPS": INT8_MFMA_PEAK_TOPS, "patterns": {}}
    wg, iters = 1024, 8192
    out = torch.empty(wg * 256, dtype=torch.int32, device=dev)
    st = _lib.stream_ptr(dev)
    ops = wg * 4 * iters * 16 * 65536.0
    for pattern, label in ((0, "zero operands"), (1, "random int4 codes x16 (what the GEMMs feed)"), (2, "random int8 bytes"),
                           (3, "random int4 codes sign-extended to int8")):
        burst = mfma_i8_rate(pattern, launches=5, iters=iters, workgroups=wg)
        clocks, stop = [], threading.Event()

        def sample():
            while not stop.is_set():
                c = gpu_clock_mhz()
                if c:
                    clocks.append(c)
                time.sleep(0.25)

        th = threading.Thread(target=sample)
        torch.cuda.synchronize()
        th.start()
        t0 = time.perf_counter()
        n = 0
        while time.perf_counter() - t0 < seconds:
            for _ in range(20):
                _lib.check(L.qr_calib_mfma_i8(pattern, iters, wg, out.data_ptr(), st))
            torch.cuda.synchronize()
            n += 20
        t = time.perf_counter() - t0
        stop.set()
        th.join()
        tail = clocks[len(clocks) // 2:]
        res["patterns"][label] = {"burst_TOPS": round(burst, 1), "sustained_TOPS": round(n * ops / t / 1e12, 1),
                                  "sustained_seconds": round(t, 2), "frac_of_published_peak": round(n * ops / t / 1e12 / INT8_MFMA_PEAK_TOPS, 4),
                                  "sclk_mhz_second_half": [min(tail), max(tail)] if tail else None, "sclk_samples": len(clocks)}
    return res


def gemm_kernel_name(m, n, k=0):
    t256 = ((m + 255) // 256) * ((n + 255) // 256)
    t128 = ((m + 127) // 128) * ((n + 255) // 256)
    groups = (n + 31) // 32                # the library's choice: enough groups of 32 rows to give every CU a workgroup
    xs = any((groups + rg - 1) // rg >= 192 for rg in range(4, 9))
    if m == 1 or (m <= 4 and not xs):
        return "gemv_i4_kernel"
    if m <= 64:
        if not xs and m >= 40 and k >= 16384:   # narrow weight, many tokens, long K: K sliced across workgroups + slab sum
            return "decode_xs_kernel (K sliced) + dequant_slabs_kernel"
        return "decode_xs_kernel" if xs else "decode_i4_kernel"
    if t128 >= 128:         # the library's choice between its pipelined kernels, by rounds of tiles (256-, 192- or 128-row)
        t192 = ((m + 191) // 192) * ((n + 255) // 256)
        r256, r192, r128 = (t256 + 255) // 256, ((t192 + 255) // 256) * 0.80, ((t128 + 255) // 256) * 0.57
        return "gemm_sp256_kernel" if (r256 <= r128 and r256 <= r192) or r192 <= r128 else "gemm_spk_kernel"
    return "gemm_ks_kernel<64,256>"


FRONT_KERNEL = {"had": "hadamard kernel + quantiser (fused)", "had32": "hadamard kernel in fp32 precision + quantiser (fused)",
                "quant": "quant_rows_kernel",
                "rmsnorm": "rmsnorm_quant_rows_kernel", "heads": "heads_hadamard_quant_rows_kernel"}


class LinearWorkload:
    """One quantised linear layer: front (quantiser, optionally behind a Hadamard / RMSNorm / heads
    Hadamard) + Linear4bit, operands resident in HBM."""

    def __init__(self, name, dev, on_gpu_data=False, fp6=False):
        import quarot_amd
        self.q = quarot_amd
        self.name = name
        self.fp6 = fp6
        self.m, self.k, self.n, self.front_kind = WORKLOADS[name]
        m, k, n = self.m, self.k, self.n
        self.decode = m <= 64
        src = dev if on_gpu_data else "cpu"
        self.x_cpu = None
        x = synth_x(m, k, seed=0 if not self.decode else 3, outliers=not self.decode, device=src)
        w, sw = synth_w(n, k, seed=1, device=src)
        if not on_gpu_data:
            self.x_cpu, self.w_cpu, self.sw_cpu = x, w, sw
        self.x = x.to(dev)
        self.lin = quarot_amd.nn.Linear4bit(k, n).half().to(dev)
        self.lin.weight.copy_(w.to(dev))
        self.lin.weight_scales.copy_(sw.to(dev))
        self.heads = 32 if self.front_kind == "heads" else 0
        if self.heads:
            self.x = self.x.view(m, self.heads, k // self.heads)   # as attention writes it: [tokens, heads, head_dim]
        nn_ = quarot_amd.nn
        self.front = {"had": lambda: nn_.OnlineHadamardQuantizer(k), "had32": lambda: nn_.OnlineHadamardQuantizer(k, force_fp32=True),
                      "rmsnorm": lambda: nn_.RMSNormQuantizer(k),
                      "heads": lambda: nn_.HeadsHadamardQuantizer(self.heads), "quant": lambda: nn_.Quantizer()}[self.front_kind]().to(dev)
        # decode: identical weight copies used round-robin, more bytes in total than the last-level cache
        self.copies = [self.lin.weight]
        if self.decode:
            while sum(c.numel() for c in self.copies) < 640 * 1024 * 1024:
                self.copies.append(self.lin.weight.clone())
        self.i = 0
        # front kernel and GEMM go out in ONE call into the library (decode steps, and the shorter prefill
        # steps, are otherwise bound by the host's per-call cost)
        self.one_call = self.front_kind in ("had", "had32", "quant") and not fp6
        if fp6:
            # the opt-in FP6 matrix path: the step converts the activations' codes and runs the GEMM on 6-bit
            # operands (the weights' 6-bit copy is made once, at the first call)
            assert not self.decode and k % 64 == 0
            self.lin.prefill_fp6, self.lin.fp6_min_rows = True, 0
        self.had_args = (self.front.had_rem_dim, self.front.rem_dim) if self.front_kind in ("had", "had32") else (None, 0)
        # one token behind a 1024-point factor: the library runs front and dot products in ONE kernel
        self.single_launch = self.one_call and m == 1 and (
            (self.front_kind == "had" and k % 1024 == 0 and k // 1024 in (12, 20, 28)) or (self.front_kind == "quant" and k <= 32768))
        self.fp32_had = self.front_kind == "had32"
        self.ops = 2.0 * m * n * k

    def weight(self):
        w = self.copies[self.i % len(self.copies)]
        self.i += 1
        return w

    def step(self):
        if self.fp6:
            return self.lin(self.front(self.x))
        if self.one_call:
            return self.q.quantized_linear(self.x, self.weight(), self.lin.weight_scales, self.lin.bias, *self.had_args,
                                           force_fp32=self.fp32_had)
        p = self.front(self.x)
        return self.q.linear_i4(p.quantized_x, p.scales_x, self.weight(), self.lin.weight_scales, self.lin.bias)

    def gemm(self, p):
        if self.fp6:
            return self.q.linear_f6(self.p6, p.scales_x, self.lin._weight_f6(), self.lin.weight_scales, self.lin.bias)
        return self.q.linear_i4(p.quantized_x, p.scales_x, self.weight(), self.lin.weight_scales, self.lin.bias)

    def staged_step(self):
        """The reference-shaped chain of separate modules (untimed in `value`)."""
        nn_ = self.q.nn
        if not hasattr(self, "_staged"):
            dev = self.x.device
            if self.front_kind in ("had", "had32"):
                self._staged = torch.nn.Sequential(nn_.OnlineHadamard(self.k, force_fp32=self.fp32_had), nn_.Quantizer()).to(dev)
            elif self.front_kind == "rmsnorm":
                self._staged = torch.nn.Sequential(nn_.RMSNorm(self.k), nn_.Quantizer()).to(dev)
            elif self.front_kind == "heads":
                had_heads, quant = nn_.OnlineHadamard(self.heads).to(dev), nn_.Quantizer()
                self._staged = lambda t: quant(had_heads(t.transpose(-1, -2)).transpose(-1, -2).reshape(self.m, self.k).contiguous())
            else:
                self._staged = nn_.Quantizer()
        return self.lin(self._staged(self.x))

    def fp16_linear_ms(self, steps):
        """Context only, never a target: torch's fp16 linear layer on the same shape (the reference's benchmark
        prints its int4 chains beside it, benchmarks/qlinear_benchmark.py:60-66,102-106); random weights."""
        w = torch.randn(self.n, self.k, device=self.x.device, dtype=torch.float16) * 0.02
        x = self.x.reshape(self.m, self.k)
        return float(np.median(timed_loops(lambda: torch.nn.functional.linear(x, w), steps, 3, 3, min_span_ms=0)))

    def kernel_times(self, reps):
        """(front kernel ms, GEMM kernel ms), each from a pass of its own (decode: the weights still
        rotating among their copies)."""
        p = self.front(self.x)
        if self.fp6:
            self.p6 = self.q.convert_i4_f6(p.quantized_x)
            self.convert_ms = kernel_ms(lambda: self.q.convert_i4_f6(p.quantized_x), reps)
        if self.single_launch:      # the step IS the dominant kernel; the front kernel of the two-launch chain beside it
            return kernel_ms(lambda: self.front(self.x), reps), kernel_ms(self.step, reps)
        return kernel_ms(lambda: self.front(self.x), reps), kernel_ms(lambda: self.gemm(p), reps)

    def front_bytes(self):
        return 2.0 * self.m * self.k + self.m * self.k / 2 + 2 * self.m

    def gemm_bytes(self):
        m, k, n = self.m, self.k, self.n
        return n * k / 2 + m * k / 2 + 2 * m + 2 * n + 2 * m * n

    def fused_bytes(self):
        """Algorithmic bytes of the one-kernel step: the weights, the fp16 row, the table (if any), scales and outputs."""
        m, k, n = self.m, self.k, self.n
        return n * k / 2 + 2 * m * k + (2 * (k // 1024) ** 2 if self.front_kind == "had" else 0) + 2 * n + 2 * m * n

    def rooflines(self, front_ms, gemm_ms):
        kern = "gemm_f6_kernel" if self.fp6 else gemm_kernel_name(self.m, self.n, self.k)
        if self.fp6:
            g = {"bound": "mfma", "achieved": round(self.ops / (gemm_ms * 1e-3) / 1e12, 1), "peak": FP6_MFMA_PEAK_TOPS, "unit": "TOP/s",
                 "convert_kernel_ms": round(self.convert_ms, 5)}
        elif self.single_launch:
            kern = "bm_gemv_kernel" if self.front_kind == "had" else "quant_gemv_kernel"
            g = {"bound": "hbm", "achieved": round(self.fused_bytes() / (gemm_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s"}
        elif self.decode:
            g = {"bound": "hbm", "achieved": round(self.gemm_bytes() / (gemm_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s"}
        else:
            g = {"bound": "mfma", "achieved": round(self.ops / (gemm_ms * 1e-3) / 1e12, 1), "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOP/s"}
        g["frac"] = round(g["achieved"] / g["peak"], 4)
        g["kernel"] = kern + (" (exact int4 GEMM on FP6 operands + dequant epilogue)" if self.fp6 else
                              (" (Hadamard + quantiser" if self.front_kind == "had" else " (quantiser")
                              + " + int4 dot products + dequant epilogue in one launch)" if self.single_launch else
                              " (int4 GEMM + dequant epilogue)")
        g["kernel_ms"] = round(gemm_ms, 5)
        f = {"bound": "hbm", "achieved": round(self.front_bytes() / (front_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
             "kernel": FRONT_KERNEL[self.front_kind], "kernel_ms": round(front_ms, 5)}
        f["frac"] = round(f["achieved"] / f["peak"], 4)
        if self.single_launch:
            f["note"] = "the front kernel of the two-launch chain, for comparison: this step does not launch it"
        return g, f

    def describe(self):
        tail = {"had": " with online Hadamard", "had32": " with online Hadamard in fp32 (force_fp32=True)", "rmsnorm": " behind RMSNorm", "heads": f" behind the Hadamard across {self.heads} heads",
                "quant": ""}[self.front_kind]
        data = "1% outlier channels x20" if not self.decode else "N(0,1)"
        return f"{self.name}: Linear4bit X[{self.m},{self.k}] fp16 ({data}) . W int4[{self.n},{self.k}]" + tail


def run_linear(name, dev, steps, warmup, repeats, kernel_reps, on_gpu_data, graph=False, fp6=False):
    wl = LinearWorkload(name, dev, on_gpu_data, fp6=fp6)
    extra = {}
    if graph:
        # one graph per weight copy would defeat the rotation: capture a run of len(copies) steps
        wl.i = 0
        want = wl.step().clone()
        wl.i = 0
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            outs = [wl.step() for _ in range(len(wl.copies))]
        g.replay()
        torch.cuda.synchronize()
        if not torch.equal(outs[0], want):
            raise RuntimeError("graph replay differs from the eager step")
        per = len(wl.copies)
        loops = [t / per for t in timed_loops(g.replay, max(1, steps // per), max(1, warmup // per), repeats)]
        extra["launch"] = "hip graph replay"
    else:
        loops = timed_loops(wl.step, steps, warmup, repeats)
        extra["launch"] = "eager" + (" (one library call per step)" if wl.one_call else "") + (
            " (front, conversion to 6-bit operands, GEMM)" if wl.fp6 else "")
    sp = spread(loops)
    ms = sp["median_ms"]
    front_ms, gemm_ms = wl.kernel_times(kernel_reps)
    groof, froof = wl.rooflines(front_ms, gemm_ms)
    staged = timed_loops(wl.staged_step, max(5, steps // 4), 3, min(repeats, 3), min_span_ms=0)
    if not wl.decode:
        extra["fp16_linear_ms"] = round(wl.fp16_linear_ms(max(5, steps // 10)), 5)
    # the whole step against the same roofline as its dominant kernel (algorithmic bytes of the GEMM for decode)
    extra["step_frac"] = round((wl.gemm_bytes() / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS) if wl.decode
                               else wl.ops / (ms * 1e-3) / 1e12 / (FP6_MFMA_PEAK_TOPS if wl.fp6 else INT8_MFMA_PEAK_TOPS), 4)
    res = {"ms": ms, "value": round(wl.ops / (ms * 1e-3) / 1e12, 2), "unit": "TOPS", "timing": sp, "roofline": groof,
           "front": froof, "kernels_ms_sum": round((0.0 if wl.single_launch else front_ms) + gemm_ms + (wl.convert_ms if wl.fp6 else 0.0), 5),
           "staged_reference_api_ms": round(float(np.median(staged)), 5), "workload": wl.describe(), **extra}
    return wl, res


def run_layer(dev, steps, warmup, repeats, kernel_reps, fp6=False):
    """Workload c3: the four W4A4 linears of a Llama-2-7B decoder layer at M = 32768 tokens (prefill,
    16 x 2048) as one step; operands generated on the GPU, resident in HBM.  fp6: the GEMMs on the opt-in
    FP6 matrix path (each step then also converts the activations' codes to 6-bit operands)."""
    import quarot_amd
    m = 32768
    parts = [("qkv", 4096, 12288, "quant", 10), ("o", 4096, 4096, "quant", 11), ("gate_up", 4096, 22016, "quant", 12),
             ("down", 11008, 4096, "had", 13)]
    xs = {4096: synth_x(m, 4096, seed=0, device=dev), 11008: synth_x(m, 11008, seed=0, device=dev)}
    mods = []
    for name, k, n, kind, seed in parts:
        w, sw = synth_w(n, k, seed=seed, device=dev)
        lin = quarot_amd.nn.Linear4bit(k, n).half().to(dev)
        lin.weight.copy_(w)
        lin.weight_scales.copy_(sw)
        if fp6:
            lin.prefill_fp6, lin.fp6_min_rows = True, 0
        front = (quarot_amd.nn.OnlineHadamardQuantizer(k) if kind == "had" else quarot_amd.nn.Quantizer()).to(dev)
        mods.append((xs[k], front, lin))
    ops = sum(2.0 * m * k * n for _, k, n, _, _ in parts)

    def step():
        for x, front, lin in mods:
            p = front(x)
            y = lin(p) if fp6 else quarot_amd.linear_i4(p.quantized_x, p.scales_x, lin.weight, lin.weight_scales, None)
            del y                                           # 0.3 - 1.4 GB each: returned to the pool before the next one

    sp = spread(timed_loops(step, steps, warmup, repeats))
    ms = sp["median_ms"]
    per, gemm_total, front_total = {}, 0.0, 0.0
    peak = FP6_MFMA_PEAK_TOPS if fp6 else INT8_MFMA_PEAK_TOPS
    for (name, k, n, kind, _), (x, front, lin) in zip(parts, mods):
        p = front(x)
        f_ms = kernel_ms(lambda: front(x), kernel_reps)
        if fp6:
            p6 = quarot_amd.convert_i4_f6(p.quantized_x)
            c_ms = kernel_ms(lambda: quarot_amd.convert_i4_f6(p.quantized_x), kernel_reps)
            g_ms = kernel_ms(lambda: quarot_amd.linear_f6(p6, p.scales_x, lin._weight_f6(), lin.weight_scales, None), kernel_reps)
            del p6
            front_total += c_ms
        else:
            g_ms = kernel_ms(lambda: quarot_amd.linear_i4(p.quantized_x, p.scales_x, lin.weight, lin.weight_scales, None), kernel_reps)
        del p
        gemm_total += g_ms
        front_total += f_ms
        per[name] = {"gemm_ms": round(g_ms, 4), "gemm_TOPS": round(2.0 * m * k * n / (g_ms * 1e-3) / 1e12, 1),
                     "gemm_frac": round(2.0 * m * k * n / (g_ms * 1e-3) / 1e12 / peak, 4),
                     "front_ms": round(f_ms, 4), "front_GBs": round((2.5 * m * k + 2 * m) / (f_ms * 1e-3) / 1e9, 1)}
        if fp6:
            per[name]["convert_ms"] = round(c_ms, 4)
    roof = {"bound": "mfma", "achieved": round(ops / (gemm_total * 1e-3) / 1e12, 1), "peak": peak, "unit": "TOP/s"}
    roof["frac"] = round(roof["achieved"] / roof["peak"], 4)
    roof["kernel"] = ("gemm_f6_kernel (exact int4 GEMM on FP6 operands + dequant epilogue), four launches" if fp6
                      else "gemm_sp256_kernel (int4 GEMM + dequant epilogue), four launches")
    roof["kernel_ms"] = round(gemm_total, 4)
    return {"ms": ms, "value": round(ops / (ms * 1e-3) / 1e12, 2), "unit": "TOPS", "timing": sp, "roofline": roof,
            "per_linear": per, "kernels_ms_sum": round(gemm_total + front_total, 4), "total_TOP": round(ops / 1e12, 2),
            "step_frac": round(ops / (ms * 1e-3) / 1e12 / peak, 4),
            "workload": "c3: Llama-2-7B decoder-layer linear set at M=32768 (qkv 4096->12288, o 4096->4096, gate_up 4096->22016, "
                        "down 11008->4096 with online Hadamard), W4A4, one step = " + ("12 launches (fronts, conversions to 6-bit operands, GEMMs)" if fp6 else "8 launches")}


def run_kv(dev, steps, warmup, repeats, kernel_reps, cpu_baseline):
    """Workload c5: quantise K (Hadamard over the head dimension, then asymmetric int4) and V
    (asymmetric int4) of one layer, [32, 4096, 8, 128] fp16 each, and dequantise both again."""
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

    def step():
        kq = kv.asym_quantize_and_pack_i4(k, hadamard=True)
        vq = kv.asym_quantize_and_pack_i4(v, hadamard=False)
        kd = kv.unpack_i4_and_asym_dequantize(*kq)          # the round trip of the config
        vd = kv.unpack_i4_and_asym_dequantize(*vq)
        return kd, vd

    sp = spread(timed_loops(step, steps, warmup, repeats))
    ms = sp["median_ms"]
    kq = kv.asym_quantize_and_pack_i4(k, hadamard=True)
    times = {
        "k_quant_hadamard": kernel_ms(lambda: kv.asym_quantize_and_pack_i4(k, hadamard=True), kernel_reps),
        "v_quant": kernel_ms(lambda: kv.asym_quantize_and_pack_i4(v, hadamard=False), kernel_reps),
        "dequant": kernel_ms(lambda: kv.unpack_i4_and_asym_dequantize(*kq), kernel_reps),
    }
    k_ms = times["k_quant_hadamard"]
    roof = {"bound": "hbm", "achieved": round(bytes_one / (k_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s"}
    roof["frac"] = round(roof["achieved"] / roof["peak"], 4)
    roof["kernel"] = "kv_had128_kernel (K cache: Hadamard on the matrix cores + asymmetric int4)"
    roof["kernel_ms"] = round(k_ms, 5)
    res = {"ms": ms, "value": round(4 * bytes_one / (ms * 1e-3) / 1e9, 1), "unit": "GB/s", "timing": sp, "roofline": roof,
           "step_frac": round(4 * bytes_one / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
           "kernels": {n: {"ms": round(t, 5), "GBs": round(bytes_one / (t * 1e-3) / 1e9, 1), "frac": round(bytes_one / (t * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
                       for n, t in times.items()},
           "workload": "c5: K and V [32,4096,8,128] fp16 (0.5% elements x15) -> asym int4 + fp16 scale/zero per head vector "
                       "-> fp16 again (four launches)", "vectors_per_tensor": vectors, "head_dim": 128}
    if cpu_baseline:
        from oracle import quarot_oracle as o
        n = vectors // 256                                   # 4096 vectors of each tensor
        ks, vs = k_cpu.reshape(-1, 128)[:n].numpy(), v_cpu.reshape(-1, 128)[:n].numpy()
        t0 = time.perf_counter()
        o.kv_asym_quant(o.kv_hadamard(ks))
        o.kv_asym_quant(vs)
        t = time.perf_counter() - t0
        sample_bytes = 2 * (2 * ks.size + n * 68)
        res["cpu_baseline"] = {"value": round(sample_bytes / t / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"first {n} of {vectors} vectors of each tensor ({t * 1e3:.0f} ms); numpy oracle "
                                         f"(fp32 FWHT + fp16 asymmetric quantiser)"}
    return res


def run_attention(name, dev, steps, warmup, repeats, kernel_reps, cpu_baseline):
    """Workloads c6 / c6b: one decode step on the paged int4 KV cache, driven as
    benchmarks/qattention_benchmark.py:53-57 drives it (length set by hand, update() with one new token per
    sequence, the returned callable on the query)."""
    from quarot_amd.transformers import kv_cache as kv
    B, S, H, P = (32, 4096, 8, 16) if name == "c6" else (1, 2048, 32, 2048)
    g = torch.Generator(device=dev).manual_seed(4)
    k = torch.randn(B, S, H, 128, generator=g, device=dev)
    mask = torch.rand(k.shape, generator=g, device=dev) < 0.005
    k[mask] *= 15
    v = torch.randn(B, S, H, 128, generator=g, device=dev)
    v[mask] *= 15
    cache = kv.MultiLayerPagedKVCache4Bit(B, P, S, dev, 1, H, 128)
    cache.update(k.half(), v.half(), 0, {})                  # the prompt: S tokens per sequence
    del k, v, mask
    k1 = torch.randn(B, 1, H, 128, generator=g, device=dev).half()
    v1 = torch.randn(B, 1, H, 128, generator=g, device=dev).half()
    q1 = torch.randn(B, 1, H, 128, generator=g, device=dev).half()

    def step():
        cache.length = S - 1                                 # the new token overwrites the last position every step
        return cache.update(k1, v1, 0, {})(q1)

    sp = spread(timed_loops(step, steps, warmup, repeats))
    ms = sp["median_ms"]
    specs = cache.get_cache_specs_for_flash_infer(None)
    qh = kv.matmul_had_cuda(q1.view(B, H, 128), torch.float16)
    out = torch.empty_like(qh)
    # the step's one launch by itself: the new token quantised and stored, the query transformed, attention over the cache
    k3, v3, q3 = k1.view(B, H, 128), v1.view(B, H, 128), q1.view(B, H, 128)
    a_ms = kernel_ms(lambda: kv.batch_decode_i4(out, q3, **specs, layer_idx=0, max_seq_len=S, q_hadamard=True,
                                                append=(k3, v3, True)), kernel_reps)
    cache_bytes = B * H * S * (2 * 64 + 2 * 4)               # codes and {scale, zero} of K and V
    roof = {"bound": "hbm", "achieved": round(cache_bytes / (a_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s"}
    roof["frac"] = round(roof["achieved"] / roof["peak"], 4)
    roof["kernel"] = "paged_decode_i4_kernel (quantise-and-append of the new token, query Hadamard and single-query attention with in-register dequantisation, one launch)"
    roof["kernel_ms"] = round(a_ms, 5)
    res = {"ms": ms, "value": round(cache_bytes / (ms * 1e-3) / 1e9, 1), "unit": "GB/s", "timing": sp, "roofline": roof,
           "step_frac": round(cache_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
           "workload": f"{name}: decode step on the paged int4 KV cache, {B} sequences x {S} tokens x {H} heads x 128, pages of {P}: "
                       "quantise-and-append of one token per sequence, query Hadamard, attention over the cache (one launch)"}
    if cpu_baseline:
        from oracle import quarot_oracle as o
        nb = 1                                               # one sequence, all heads
        tabs = [specs[n].cpu().numpy() for n in ("kv_indptr", "kv_indices", "last_page_offset")]
        one = (tabs[0][:2], tabs[1][:tabs[0][1]], tabs[2][:1])
        pages, scales = cache.pages.cpu().numpy(), cache.scales.cpu().numpy()
        t0 = time.perf_counter()
        o.paged_batch_decode(qh[:nb].cpu().numpy(), pages, scales, *one, 0)
        t = time.perf_counter() - t0
        res["cpu_baseline"] = {"value": round(nb * H * S * 136 / t / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                               "sample": f"sequence 0 of {B}, all heads ({t * 1e3:.0f} ms); numpy oracle (gather, fp32 dequantisation, "
                                         "float64 softmax attention)"}
    return res


def cpu_baseline(wl, budget_rows):
    """The reference's CPU path (torch Hadamard + quant + integer matmul + dequant) on a bounded
    row sample of the same workload, all host threads; TOPS scaled to the sample's own work."""
    from oracle import cpu_baseline as cb
    rows = min(wl.m, budget_rows)
    wc = cb.unpacked_codes(wl.w_cpu.numpy())
    ws = wl.sw_cpu.view(-1)
    hadamard, rmsnorm, heads = wl.front_kind in ("had", "had32"), wl.front_kind == "rmsnorm", wl.heads
    torch.set_num_threads(os.cpu_count() or 1)
    cb.linear4bit_path(wl.x_cpu[:2].clone(), wc[:64], ws[:64], hadamard, rmsnorm, heads)   # warm-up
    # size the sample for about 4 s per pass (three passes: 10-15 s of CPU work), starting from `budget_rows`
    t0 = time.perf_counter()
    cb.linear4bit_path(wl.x_cpu[:rows].clone(), wc, ws, hadamard, rmsnorm, heads)
    t_probe = time.perf_counter() - t0
    rows = min(wl.m, max(rows, int(rows * 4.0 / max(t_probe, 1e-3)) // 64 * 64))
    xs = wl.x_cpu[:rows].clone()
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        cb.linear4bit_path(xs, wc, ws, hadamard, rmsnorm, heads)
        times.append(time.perf_counter() - t0)
    t = float(np.median(times))
    return {"value": round(2.0 * rows * wl.n * wl.k / t / 1e12, 5), "unit": "TOPS", "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"first {rows} of {wl.m} rows, full N and K, median of 3 ({t * 1e3:.0f} ms); torch "
                      + ("fp32 RMSNorm + " if rmsnorm else "fp32 matmul_hadU + " if hadamard
                         else "fp32 matmul_hadU over heads + " if heads else "")
                      + "fp16 sym quant + int32 torch matmul + fp16 dequant"}


def brief(res):
    """The per-config view of a result: step time, value and the dominant kernel's roofline."""
    keep = ("ms", "value", "unit", "roofline", "front", "kernels", "per_linear", "kernels_ms_sum", "staged_reference_api_ms", "launch",
            "fp16_linear_ms", "step_frac")
    out = {k: res[k] for k in keep if k in res}
    out["ci95_ms"] = res["timing"]["ci95_ms"]
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500, help="steps per timed loop")
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--repeats", type=int, default=10, help="timed loops (median and mean +- 1.96 sigma are reported)")
    ap.add_argument("--kernel-reps", type=int, default=50, help="launches in the separate per-kernel event pass")
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-per-config", action="store_true", help="measure the chosen workload only")
    ap.add_argument("--graph", action="store_true",
                    help="time replays of the step captured in a HIP graph (decode steps are host-launch-bound when "
                         "launched eagerly from Python); the first replay is checked against the eager result")
    ap.add_argument("--fp6", action="store_true",
                    help="prefill linear workloads only: run the GEMM on the opt-in FP6 matrix path (Linear4bit.prefill_fp6); "
                         "the step then includes the conversion of the activations' codes to 6-bit operands")
    ap.add_argument("--cpu-rows", type=int, default=64,
                    help="rows of the first CPU-baseline pass; the timed sample is then sized for about 4 s per pass")
    ap.add_argument("--mfma-ceiling", type=float, default=0.0, metavar="SECONDS",
                    help="instead of a workload, run the register-only loop of the int8 matrix instruction (qr_calib_mfma_i8) for "
                         "SECONDS per operand pattern, with the shader clock sampled from rocm-smi beside it")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="instead of a workload, run a plain 256 MiB device copy 20 times (known traffic: 256 MiB read, "
                         "256 MiB written per launch) for scaling the profiler's FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this path is data-parallel over tokens with no exchange; "
              "run one process per GPU and add the values (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    if args.fp6 and args.workload != "c3" and (WORKLOADS[args.workload] is None or WORKLOADS[args.workload][0] <= 64):
        print("--fp6 applies to the prefill linear workloads (c1, c2, c3, c3a-c3d, b13*, b70*)", file=sys.stderr)
        sys.exit(2)
    from quarot_amd import _lib
    if not _lib.LIB_PATH.exists():
        from quarot_amd import build
        build.build(verbose=False)
    _lib.lib()
    dev = torch.device("cuda:0")
    if args.mfma_ceiling > 0:
        print(json.dumps({"mfma_i8_ceiling": mfma_ceiling(args.mfma_ceiling)}))
        return
    if args.copy_calibration:
        src = torch.randint(0, 255, (256 * 1024 * 1024,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(20):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": {"launches": 20, "read_bytes": src.numel(), "written_bytes": src.numel()}}))
        return

    def measure(name, headline):
        """headline: the protocol's full step / repeat counts; per-config: a fifth of the steps (at least 20 per
        loop, at most ~60 ms of GPU time per loop) and 5 loops."""
        fp6 = name.endswith("_fp6") or (args.fp6 and headline)      # per-config names "<workload>_fp6": the opt-in FP6 matrix path
        name = name[:-4] if name.endswith("_fp6") else name
        spec = WORKLOADS[name]
        big = name.startswith("c3") or name in ("c5", "c6")
        steps = args.steps if headline else max(20, args.steps // 5)
        if not headline and (name in ("c6", "c6b") or (spec is not None and spec[0] <= 64)):
            steps = max(steps, 100)                        # decode steps of 25-50 us: a loop's ~30 us of start and wake-up spread over 100
        if big:
            steps = max(5, steps // (25 if name == "c3" else 10))
        repeats = args.repeats if headline else max(3, args.repeats // 2)
        kreps = args.kernel_reps if not big else max(5, args.kernel_reps // 5)
        warm = args.warmup if not big else max(2, args.warmup // 5)
        if name == "c3":
            return None, run_layer(dev, steps, warm, repeats, kreps, fp6=fp6), steps, repeats
        if name == "c5":
            return None, run_kv(dev, steps, warm, repeats, kreps, headline and not args.no_cpu_baseline), steps, repeats
        if name in ("c6", "c6b"):
            return None, run_attention(name, dev, steps, warm, repeats, kreps, headline and not args.no_cpu_baseline), steps, repeats
        assert spec is not None
        wl, res = run_linear(name, dev, steps, warm, repeats, kreps, on_gpu_data=not headline, graph=args.graph and headline, fp6=fp6)
        return wl, res, steps, repeats

    wl, res, steps, repeats = measure(args.workload, True)
    roof = dict(res["roofline"])
    traffic, source = traffic_from_profile(args.workload + ("_fp6" if args.fp6 else ""), roof["kernel"])
    if traffic is not None and args.workload == "c3":
        traffic *= 4                                       # the step is four launches; the summary holds their average
    roof["traffic"] = traffic
    roof["traffic_source"] = source
    if roof.get("bound") == "mfma" and not args.fp6:
        # what the int8 matrix instruction alone sustains on this box right now (register-only loop, operands with the
        # GEMM's bit statistics, ~60 ms of launches): the part's own ceiling for ANY int8 kernel; `frac` stays against `peak`
        roof["attainable"] = round(mfma_i8_rate(1, launches=12), 1)
        roof["attainable_zero_operands"] = round(mfma_i8_rate(0, launches=12), 1)
        roof["frac_of_attainable"] = round(roof["achieved"] / roof["attainable"], 4)
    kv_line = args.workload in ("c5", "c6", "c6b")
    out = {
        "metric": ("KV-cache int4 quantise + dequantise GB/s (K with Hadamard, V)" if args.workload == "c5"
                   else "decode attention over the paged int4 KV cache, GB/s of cache bytes" if kv_line
                   else "Linear4bit TOPS (had+quant+GEMM)"),
        "value": res["value"], "unit": res["unit"], "n_gpus": 1, "steps": steps, "warmup": args.warmup, "repeats": repeats,
        "ms_per_step": res["ms"], "ms_per_step_mean": res["timing"]["mean_ms"], "ms_per_step_ci95": res["timing"]["ci95_ms"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": ("f16 -> u4 (fp32 Hadamard, fp16 quantiser)" if kv_line
                  else "int4 x int4 -> exact integers in fp32 (FP6 MFMA), fp16 scales" if args.fp6
                  else "int4 x int4 -> int32 (int8 MFMA), fp16 scales"),
        "data": "synthetic",
        "config": {"workload": res["workload"], "launch": res.get("launch", "eager"),
                   "timing": "median of the last `repeats` loops of `steps` steps, each loop between two synchronisations; loops run until "
                             f"they span {MIN_SPAN_MS:.0f} ms (`loops_run`), because the GPU's clocks take ~30 ms of work to settle after idling "
                             "(`first_loop_ms`: the first loop); kernel times from a separate pass of back-to-back launches of that kernel "
                             "alone between two HIP events on the launch stream",
                   "loops_run": res["timing"].get("loops_run"), "first_loop_ms": res["timing"].get("first_loop_ms")},
        "roofline": roof,
    }
    for key in ("front", "kernels", "per_linear", "kernels_ms_sum", "staged_reference_api_ms", "fp16_linear_ms", "step_frac"):
        if key in res:
            out[key] = res[key]
    if wl is not None:
        out["config"].update({"M": wl.m, "K": wl.k, "N": wl.n})
        if not args.no_cpu_baseline:
            out["cpu_baseline"] = cpu_baseline(wl, args.cpu_rows)
    elif "cpu_baseline" in res:
        out["cpu_baseline"] = res["cpu_baseline"]
    del wl
    if not args.no_per_config and args.workload == "c2":
        per = {}
        for name in PER_CONFIG:
            torch.cuda.empty_cache()
            _, r, _, _ = measure(name, False)
            per[name] = brief(r)
            t, s = traffic_from_profile(name, r["roofline"]["kernel"])
            if t is not None:
                per[name]["roofline"]["traffic"], per[name]["roofline"]["traffic_source"] = (4 * t if name in ("c3", "c3_fp6") else t), s
        out["per_config"] = per
        # the same table in a few numbers per workload: [step ms, dominant kernel ms, its roofline fraction, the step's]
        out["roofline"]["per_config"] = {name: [r["ms"], r["roofline"]["kernel_ms"], r["roofline"]["frac"], r.get("step_frac")]
                                         for name, r in per.items()}
        out["roofline"]["per_config_front"] = {name: [r["front"]["kernel_ms"], r["front"]["frac"]] for name, r in per.items() if "front" in r}
        out["per_config_note"] = ("same step definition as the headline; operands generated on the GPU, a fifth of the steps per loop "
                                  "(c3, c5: fewer still; decode and attention steps: at least 100) and half the repeats")
    print(json.dumps(out))


if __name__ == "__main__":
    main()
