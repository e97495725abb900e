#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only NAME] [--no-cpu]

NAME is one of prefill | ceiling | plumbing | module | long | decode | decode_b1 | kda | next | copy; "copy" runs a plain 1 GiB
device copy and nothing else (the known-size kernel against which the HBM
counters FETCH_SIZE / WRITE_SIZE are calibrated under rocprofv3 --pmc).

A "step" is one pass of the headline workload: windowed prefill attention with
fused RoPE on B=8, T=4096, H=8, D=128, window 1024 (bf16), inputs resident in
HBM.  One JSON line is printed.  `value` is the attention throughput of that
workload in TFLOP/s (algorithmic flops = 4*D*B*H*visible pairs); the `roofline`
object prices the dominant kernel against the 2.5 PFLOP/s dense bf16 MFMA peak;
`cpu_baseline` times the CPU oracle on a bounded sample of the same workload;
`extra` carries the other workloads (long-context prefill, KV-cache decode
against the 8 TB/s HBM peak, KDA), each with its own roofline fraction.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0
SCALE = 0.12


def prefill_flops(B, T, H, D, window):
    if window is None or window <= 0 or window >= T:
        pairs = T * (T + 1) // 2
    else:
        pairs = window * (window + 1) // 2 + (T - window) * window
    return 4.0 * D * B * H * pairs


def time_gpu(fn, steps, warmup, per_launch=False):
    """Milliseconds per call over `steps` calls after `warmup` untimed ones, HIP events on the current
    stream (the one the kernels are launched on).  Default: the mean, one event pair around all the
    calls.  per_launch: an event pair around every call; returns (median, mean) of the calls' own durations."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    if per_launch:
        marks = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for a, b in marks:
            a.record()
            fn()
            b.record()
        torch.cuda.synchronize()
        each = sorted(a.elapsed_time(b) for a, b in marks)
        return each[len(each) // 2], sum(each) / len(each)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / steps


def time_settled(fn, steps, warmup, seconds=0.4):
    """(ms per call settled, ms per call over the first `steps` calls from an idle GPU).  After a change of load the
    chip runs the first launches slower and settles over some hundred milliseconds (power management), so the timed
    steps follow `seconds` of the same call back to back."""
    fn()
    torch.cuda.synchronize()
    time.sleep(0.5)
    ms_first = time_gpu(fn, steps, 0)
    time_gpu(fn, max(int(seconds * 1e3 / ms_first), 1), 0)
    return time_gpu(fn, steps, warmup), ms_first


# ---- diagnostic kernels of the benchmark (their own library, not part of the product ABI) ----------
_probe_lib = None


def probe_lib():
    import ctypes
    global _probe_lib
    if _probe_lib is None:
        from daisy_amd import build as _build
        if not os.path.exists(_build.PROBE_LIB_PATH):
            raise RuntimeError(f"{_build.PROBE_LIB_PATH} is missing: build it with `python -m daisy_amd.build`")
        lib = ctypes.CDLL(_build.PROBE_LIB_PATH)
        lib.daisy_probe_matrix_rate.restype = ctypes.c_int
        lib.daisy_probe_matrix_rate.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                                ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
        lib.daisy_probe_matrix_rate_data.restype = ctypes.c_int
        lib.daisy_probe_matrix_rate_data.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                                     ctypes.c_void_p, ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
        lib.daisy_probe_read_rate.restype = ctypes.c_int
        lib.daisy_probe_read_rate.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        _probe_lib = lib
    return _probe_lib


def probe_matrix_rate(with_vector_mix, iters=50000, workgroups=256, device="cuda:0"):
    """Sustained rate of register-only bf16 MFMAs on every SIMD (optionally with the attention loop's vector
    mix), and the shader clock the chip ran at meanwhile.  Returns {"ms", "tflops", "clock_mhz"}."""
    import ctypes
    dev = torch.device(device)
    sink = torch.empty(4096, dtype=torch.float32, device=dev)
    ticks = torch.zeros(2 * workgroups, dtype=torch.int64, device=dev)
    lib = probe_lib()
    flop = ctypes.c_double(0.0)
    stream = torch.cuda.current_stream(dev).cuda_stream
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    rc = lib.daisy_probe_matrix_rate(int(with_vector_mix), workgroups, max(iters // 10, 1), sink.data_ptr(), ticks.data_ptr(),
                                     ctypes.byref(flop), stream)   # warm-up
    assert rc == 0, rc
    start.record()
    rc = lib.daisy_probe_matrix_rate(int(with_vector_mix), workgroups, iters, sink.data_ptr(), ticks.data_ptr(), ctypes.byref(flop), stream)
    end.record()
    assert rc == 0, rc
    torch.cuda.synchronize(dev)
    ms = start.elapsed_time(end)
    t = ticks.view(workgroups, 2).double().sum(0)
    return {"ms": ms, "tflops": flop.value / ms / 1e9, "clock_mhz": float(t[0] / t[1] * 100.0)}


def probe_matrix_rate_data(kind, seconds=1.0, iters=80000, workgroups=256, device="cuda:0", variant=0):
    """Sustained rate of register-only bf16 MFMAs whose operands change with every instruction and hold `kind` data
    ("zeros" or "normal": N(0,1) rounded to bf16), launches back to back for `seconds`; the rate and clock of the last
    quarter of the run.  The instruction stream is the same for both kinds: the difference is what the chip's power
    management takes for the toggling of the operand bits.  variant 3: the attention loop's mix (per MFMA 3 fma + 1 exp2,
    A operands read from LDS) instead of MFMAs alone, LDS tile and B operands filled with the data."""
    import ctypes
    dev = torch.device(device)
    n_el = 16 * 512 * 8
    data = (torch.zeros(n_el, device=dev) if kind == "zeros"
            else torch.randn(n_el, device=dev, generator=torch.Generator(device=dev).manual_seed(0))).bfloat16()
    sink = torch.empty(4096, dtype=torch.float32, device=dev)
    ticks = torch.zeros(2 * workgroups, dtype=torch.int64, device=dev)
    lib = probe_lib()
    flop = ctypes.c_double(0.0)
    stream = torch.cuda.current_stream(dev).cuda_stream

    def run():
        rc = lib.daisy_probe_matrix_rate_data(data.data_ptr(), n_el * 2, variant, workgroups, iters, sink.data_ptr(), ticks.data_ptr(),
                                              ctypes.byref(flop), stream)
        assert rc == 0, rc

    ms_one = time_gpu(run, 2, 1)
    n = max(int(seconds * 1e3 / ms_one), 4)
    time_gpu(run, 3 * n // 4, 0)
    ms = time_gpu(run, n - 3 * n // 4, 0)
    t = ticks.view(workgroups, 2).double().sum(0)
    return {"tflops": flop.value / ms / 1e9, "clock_mhz": float(t[0] / t[1] * 100.0), "seconds": n * ms_one / 1e3, "operands": kind}


def probe_read_rate(gib=2, workgroups=8192, repeats=5, device="cuda:0"):
    """Read-only streaming rate of the GPU over a `gib` GiB buffer: the practical ceiling of the decode kernel."""
    dev = torch.device(device)
    nbytes = gib << 30
    buf = torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(1)
    sink = torch.empty(4096, dtype=torch.int32, device=dev)
    lib = probe_lib()
    stream = torch.cuda.current_stream(dev).cuda_stream
    run = lambda: lib.daisy_probe_read_rate(buf.data_ptr(), nbytes, workgroups, sink.data_ptr(), stream)
    assert run() == 0
    ms = time_gpu(run, repeats, 0)
    return {"ms": ms, "bytes": nbytes, "gbs": nbytes / ms / 1e6}


def rope_table(D, T, base=10000.0, device="cuda:0"):
    freq = (1.0 / base) ** torch.linspace(0, 1, steps=D // 2, dtype=torch.float32)
    theta = torch.arange(T, dtype=torch.float32)[:, None] * freq[None, :]
    return theta.cos().to(device), theta.sin().to(device)


def rms(x):
    return torch.nn.functional.rms_norm(x, (x.size(-1),))


# ---------------------------------------------------------------------------------
def bench_prefill_c2(steps, warmup, cpu_baseline=True):
    """Config 2: B8 T4096 d1024 H8 D128 W1024, merged QKV, q/k/v RMS-normed, RoPE base 10000."""
    from daisy_amd import ops
    B, T, H, D, W, dim = 8, 4096, 8, 128, 1024, 1024
    g = torch.Generator().manual_seed(0)
    x = torch.randn(B, T, dim, generator=g).bfloat16()
    w = (torch.randn(3 * dim, dim, generator=g) * 0.02).bfloat16()
    dev = "cuda:0"
    qkv = torch.nn.functional.linear(x.to(dev), w.to(dev)).view(B, T, 3 * H, D)
    q, k, v = (rms(t) for t in qkv.chunk(3, dim=-2))
    cos, sin = rope_table(D, T)
    o = torch.empty(B, T, H, D, dtype=torch.bfloat16, device=dev)
    k_rot = torch.empty(B, T, H, D, dtype=torch.bfloat16, device=dev)

    def full():
        ops.prefill_attention(q, k, v, window=W, scale=SCALE, cos=cos, sin=sin, out=o, k_out=k_rot)

    o2 = torch.empty_like(o)

    def attn_only():
        ops.prefill_attention(q, k_rot, v, window=W, scale=SCALE, out=o2)

    # After a change of load the chip needs some hundred launches to settle (the power management moves the shader
    # clock when the HBM traffic of the pre-pass appears: ~200 us per step for the first steps from an idle GPU or
    # right after a run of the attention kernel alone, ~170 us from the third hundred on).  So the order is: (1) the
    # first steps from an idle GPU, for the record; (2) half a second of the headline step back to back (the sustained
    # figure); (3) the headline: `warmup` untimed and `steps` timed steps on the GPU as (2) left it; (4) the attention
    # kernel alone for at least a second; (5) its per-launch median.
    full()
    torch.cuda.synchronize()
    time.sleep(1.0)
    ms_full_from_idle = time_gpu(full, steps, 0)
    n_full_sustained = max(int(500.0 / ms_full_from_idle), steps)
    ms_full_sustained = time_gpu(full, n_full_sustained, 0)
    ms_full = time_gpu(full, steps, warmup)
    ms_estimate = time_gpu(attn_only, 10, 2)
    n_sustained = max(int(1100.0 / ms_estimate), steps)
    ms_sustained = time_gpu(attn_only, n_sustained, 0)
    # The dominant kernel alone: same launch, keys already rotated (k_rot from above).  Median of the
    # launches' own durations (an event pair around every launch), right behind the sustained run.
    ms_kernel, ms_kernel_mean = time_gpu(attn_only, steps, warmup, per_launch=True)
    clock_after = probe_matrix_rate(False, 4000)["clock_mhz"] if SUSTAINED_CLOCK else None

    flops = prefill_flops(B, T, H, D, W)
    res = {
        "workload": "prefill_c2_B8_T4096_H8_D128_W1024_rope",
        "ms_full": ms_full, "ms_full_first_steps_from_idle": ms_full_from_idle,
        "ms_full_sustained": ms_full_sustained, "full_sustained_launches": n_full_sustained,
        "tflops_full_sustained": flops / ms_full_sustained / 1e9,
        "ms_kernel": ms_kernel, "ms_kernel_mean": ms_kernel_mean,
        "flops": flops,
        "tflops_full": flops / ms_full / 1e9, "tflops_kernel": flops / ms_kernel / 1e9,
        "frac_of_peak_kernel": flops / ms_kernel / 1e9 / PEAK_BF16_TFLOPS,
        "sustained": {"launches": n_sustained, "seconds": n_sustained * ms_sustained / 1e3, "ms_kernel": ms_sustained,
                      "tflops_kernel": flops / ms_sustained / 1e9,
                      "frac_of_peak_kernel": flops / ms_sustained / 1e9 / PEAK_BF16_TFLOPS,
                      "shader_clock_mhz_right_after": clock_after},
        "min_hbm_bytes": 4 * B * T * H * D * 2,     # q, k, v read once, o written once
    }
    if cpu_baseline:
        res["cpu_baseline"] = cpu_prefill_baseline(q[:2].cpu(), k[:2].cpu(), v[:2].cpu(), cos.cpu(), sin.cpu(), W,
                                                   f"2 of {B} batch elements, all {H} heads, T={T}")
    return res


CPU_SECONDS = 10.0   # how long each CPU baseline keeps repeating its sample
SUSTAINED_CLOCK = True   # read the shader clock with the matrix probe right after the sustained run


def _repeat_for(fn, seconds):
    """Runs fn at least twice and until `seconds` have passed; returns (mean seconds per run, runs)."""
    fn()   # first run untimed: thread pools, allocator
    runs, t0 = 0, time.perf_counter()
    while True:
        fn()
        runs += 1
        dt = time.perf_counter() - t0
        if dt >= seconds:
            return dt / runs, runs


def cpu_prefill_baseline(q, k, v, cos, sin, W, sample):
    """The reference's CPU path (RoPE + dense additive mask + SDPA) restated by the oracle's pieces."""
    import oracle
    torch.set_num_threads(os.cpu_count() or 1)
    B, T, H, D = q.shape
    mask = oracle.window_mask(T, W)

    def one_pass():
        qr, kr = oracle.apply_rope(q, cos[:T], sin[:T]), oracle.apply_rope(k, cos[:T], sin[:T])
        torch.nn.functional.scaled_dot_product_attention(qr.transpose(1, 2), kr.transpose(1, 2), v.transpose(1, 2),
                                                         attn_mask=mask, scale=SCALE)

    dt, runs = _repeat_for(one_pass, CPU_SECONDS)
    return {"value": prefill_flops(B, T, H, D, W) / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "kind": "port", "sample": f"{sample}; {runs} passes in {dt * runs:.1f} s", "seconds": dt}


# HBM bytes per launch of the headline kernel: a recorded counter value, not something this run measures.  It is read
# from the committed rocprofv3 summary, whose line
#   bench.py reads: kernel=<name> FETCH_SIZE_KiB=<n> WRITE_SIZE_KiB=<n> fetch_factor=<f> write_factor=<f>
# names the kernel the counters were taken on (FETCH_SIZE / WRITE_SIZE per dispatch, each scaled by the factor the same
# counter shows for the 1 GiB copy of `--only copy`).  A summary taken on another kernel than the one this run launches
# is not used: the line then carries no traffic figure.
PREFILL_C2_KERNEL = "prefill_tile_kernel<128>"
PREFILL_C2_TRAFFIC_FILE = os.path.join("profiles", "prefill_tile_kernel_c2_hbm_traffic.txt")


def recorded_traffic(path, kernel):
    """(bytes per launch or None, a sentence on where the figure comes from)."""
    import re
    try:
        with open(os.path.join(ROOT, path)) as f:
            text = f.read()
    except OSError:
        return None, f"{path} is missing: no recorded counter value"
    m = re.search(r"bench\.py reads: kernel=(\S+) FETCH_SIZE_KiB=(\d+) WRITE_SIZE_KiB=(\d+) fetch_factor=([\d.]+) write_factor=([\d.]+)", text)
    if m is None:
        return None, f"{path} has no 'bench.py reads:' line"
    if m.group(1) != kernel:
        return None, f"{path} was recorded on {m.group(1)}, this run launches {kernel}: figure not used"
    nbytes = int((int(m.group(2)) * float(m.group(4)) + int(m.group(3)) * float(m.group(5))) * 1024)
    return nbytes, (f"recorded counter value from {path} (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE of {kernel} on this workload, "
                    "scaled by the factors of a 1 GiB copy); not measured by this run")


def bench_plumbing_c1(steps, warmup, cpu_baseline=True):
    """Config 1: one sliding-window layer forward, B1 T256 d256 H4 D64 W128, x ~ N(0,1) fp32, weights
    N(0, 0.02) seed 0: the drop-in module on the GPU, and the reference's PyTorch path on the CPU
    (bf16 parameters, dense additive mask, library SDPA -- the oracle's restatement) timed beside it."""
    from daisy_amd import CausalSelfAttention, WindowMask
    dim, H, D, T, W = 256, 4, 64, 256, 128
    torch.manual_seed(0)
    w = torch.randn(4, dim, dim) * 0.02
    x = torch.randn(1, T, dim)
    attn = CausalSelfAttention(dim=dim, num_heads=H, head_dim=D, max_seq_len=T)
    with torch.no_grad():
        attn.qkvo_w.copy_(w.bfloat16())
    attn = attn.to("cuda:0").eval()
    xd, mask = x.to("cuda:0"), WindowMask(W)
    with torch.no_grad():
        ms = time_gpu(lambda: attn.prefill(xd, None, attn_mask=mask), max(steps, 20), max(warmup, 5))
    out = {"workload": "plumbing_c1_B1_T256_d256_H4_D64_W128_layer_forward", "ms_hip_module": ms,
           "flops_attention": prefill_flops(1, T, H, D, W)}
    if cpu_baseline:
        import oracle
        torch.set_num_threads(os.cpu_count() or 1)
        wb = w.bfloat16()
        cos, sin = attn.rotary.cos.cpu()[:T], attn.rotary.sin.cpu()[:T]
        dt, runs = _repeat_for(lambda: oracle.attn_prefill(x, wb, H, D, cos, sin, W), 2.0)
        out["cpu_reference_path"] = {"ms": dt * 1e3, "cores": torch.get_num_threads(), "kind": "port",
                                     "sample": f"the whole layer, {runs} passes in {dt * runs:.1f} s"}
        out["speedup_vs_cpu_path"] = dt * 1e3 / ms
    return out


def bench_copy(steps, warmup):
    """A plain device-to-device copy of 1 GiB (reads 2^30 bytes, writes 2^30 bytes per launch)."""
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device="cuda:0").fill_(1)
    dst = torch.empty_like(src)
    ms = time_gpu(lambda: dst.copy_(src), steps, warmup)
    return {"workload": "copy_1GiB", "bytes_read": n, "bytes_written": n, "ms": ms, "gbs": 2 * n / ms / 1e6}


def bench_module_c2(steps, warmup):
    """CausalSelfAttention.prefill on config 2 (QKV GEMM, norm, RoPE, attention, output GEMM), with the
    one-pass norm + RoPE kernel and with the library's elementwise ops; plus that kernel alone."""
    from daisy_amd import CausalSelfAttention, WindowMask, ops
    from daisy_amd.functional import NORM_EPS_BF16
    B, T, H, D, W, dim = 8, 4096, 8, 128, 1024, 1024
    dev = "cuda:0"
    torch.manual_seed(0)
    attn = CausalSelfAttention(dim=dim, num_heads=H, head_dim=D, max_seq_len=T)
    with torch.no_grad():
        attn.qkvo_w.copy_((torch.randn(4, dim, dim) * 0.02).bfloat16())
    attn = attn.to(dev).eval()
    x = torch.randn(B, T, dim, generator=torch.Generator().manual_seed(0)).bfloat16().to(dev)
    mask = WindowMask(W)
    out = {"workload": "module_prefill_c2_B8_T4096_d1024_H8_D128_W1024"}
    with torch.no_grad():
        for name, fused in (("ms_fused_prep", True), ("ms_library_elementwise", False)):
            attn.fused_prep = fused
            out[name], out[name + "_first_steps_from_idle"] = time_settled(lambda: attn.prefill(x, None, attn_mask=mask), steps, warmup)
        qkv = torch.nn.functional.linear(x, attn.qkvo_w[:3].flatten(end_dim=1)).view(B, T, 3 * H, D)
        q, k, v = qkv.chunk(3, dim=-2)
        cos, sin = attn.rotary._get_cos_sin(T)
        qo, ko, vo = (torch.empty(B, T, H, D, dtype=torch.bfloat16, device=dev) for _ in range(3))
        ms = time_gpu(lambda: ops.qkv_prep(q, k, v, eps=NORM_EPS_BF16, cos=cos, sin=sin, q_out=qo, k_out=ko, v_out=vo),
                      steps, warmup)
    nbytes = 6 * B * T * H * D * 2
    out["qkv_prep_kernel"] = {"ms": ms, "bytes": nbytes, "gbs": nbytes / ms / 1e6, "frac_of_hbm_peak": nbytes / ms / 1e6 / PEAK_HBM_GBS}
    return out


def bench_prefill_c3(steps, warmup):
    """Config 3: B1 T65536 H16 D128, q/k/v ~ N(0,1) already rotated; window 2048 and full causal."""
    from daisy_amd import ops
    B, T, H, D = 1, 65536, 16, 128
    g = torch.Generator(device="cuda:0").manual_seed(0)
    q, k, v = (torch.randn(B, T, H, D, generator=g, device="cuda:0", dtype=torch.float32).bfloat16() for _ in range(3))
    o = torch.empty_like(q)
    out = {}
    for name, W, n in (("window2048", 2048, steps), ("full_causal", None, max(steps // 4, 2))):
        ms, ms_first = time_settled(lambda: ops.prefill_attention(q, k, v, window=W, scale=SCALE, out=o), n, max(warmup // 2, 1))
        fl = prefill_flops(B, T, H, D, W)
        out[name] = {"ms": ms, "ms_first_steps_from_idle": ms_first, "flops": fl, "tflops": fl / ms / 1e9,
                     "frac_of_peak": fl / ms / 1e9 / PEAK_BF16_TFLOPS}
    # The same launch on tensors of zeros: the same instructions, addresses and memory traffic, but operand bits that
    # never toggle.  Timing only (the result is meaningless); what it shows is how much of the rate on N(0,1) data the
    # chip's power management takes away (see extra.matrix_pipe_ceiling.mfma_only_*_operands for the matrix pipe alone).
    q.zero_(); k.zero_(); v.zero_()
    ms, _ = time_settled(lambda: ops.prefill_attention(q, k, v, window=None, scale=SCALE, out=o), max(steps // 4, 2), 1)
    fl = prefill_flops(B, T, H, D, None)
    out["full_causal_on_zero_tensors_timing_only"] = {"ms": ms, "tflops": fl / ms / 1e9, "frac_of_peak": fl / ms / 1e9 / PEAK_BF16_TFLOPS}
    return out


def bench_decode_c4(steps=256, warmup=16, cpu_baseline=True):
    """Config 4: batch 64, H16 D128, ring of 4096 slots holding positions up to 8192, 256 consecutive steps."""
    from daisy_amd import ops
    B, H, D, W, t0 = 64, 16, 128, 4096, 8192
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(0)
    kc = torch.randn(B, H, W, D, generator=g, device=dev, dtype=torch.float32).bfloat16()
    vc = torch.randn(B, H, W, D, generator=g, device=dev, dtype=torch.float32).bfloat16()
    n = steps + warmup
    qs = torch.randn(n, B, H, D, generator=g, device=dev, dtype=torch.float32).bfloat16()
    ks = torch.randn(n, B, H, D, generator=g, device=dev, dtype=torch.float32).bfloat16()
    vs = torch.randn(n, B, H, D, generator=g, device=dev, dtype=torch.float32).bfloat16()
    o = torch.empty(B, H, D, dtype=torch.bfloat16, device=dev)
    results = {}
    for nsplit in (1, 2):
        ws_bytes = ops.decode_workspace_bytes(B, H, D, W, nsplit)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
        step = [0]

        def one():
            i = step[0] % n
            t = t0 + step[0]
            ops.decode_attention(qs[i], ks[i], vs[i], kc, vc, n_rows=W, new_idx=t % W, write_back=True,
                                 scale=SCALE, out=o, workspace=ws, nsplit=nsplit)
            step[0] += 1

        ms = time_gpu(one, steps, warmup)
        nbytes = B * H * W * D * 2 * 2
        results[f"nsplit{nsplit}"] = {"ms_per_step": ms, "bytes": nbytes, "gbs": nbytes / ms / 1e6,
                                      "frac_of_peak": nbytes / ms / 1e6 / PEAK_HBM_GBS}
    best = max(results.values(), key=lambda r: r["gbs"])
    # The same ring through the one-launch step (rows of a QKV projection; norm, RoPE, append and attention in the
    # kernel; position in device memory), on a bf16 ring and on the reference generator's default, fp16.
    from daisy_amd.functional import NORM_EPS_BF16
    cos, sin = rope_table(D, t0 + n + 1, device=dev)
    raw = torch.cat([qs, ks, vs], dim=2)                      # [n, B, 3H, D]
    pos = torch.zeros(1, dtype=torch.int32, device=dev)
    ws = torch.empty(max(ops.decode_workspace_bytes(B, H, D, W, 0), 1), dtype=torch.uint8, device=dev)
    one_launch = {}
    for name, ring_dtype in (("bf16_ring", torch.bfloat16), ("fp16_ring", torch.float16)):
        kr, vr = kc.to(ring_dtype), vc.to(ring_dtype)
        pos.fill_(t0)
        step = [0]

        def fused():
            r = raw[step[0] % n]
            ops.attn_step(r[:, :H], r[:, H:2 * H], r[:, 2 * H:], kr, vr, pos, cos=cos, sin=sin, eps=NORM_EPS_BF16,
                          scale=SCALE, out=o, workspace=ws)
            pos.add_(1)
            step[0] += 1

        ms = time_gpu(fused, steps, warmup)
        one_launch[name] = {"ms_per_step": ms, "gbs": nbytes / ms / 1e6, "frac_of_peak": nbytes / ms / 1e6 / PEAK_HBM_GBS}
        del kr, vr
    out = {"workload": "decode_c4_B64_H16_D128_W4096_256steps", "variants": results, **best,
           "one_launch_step_device_position": one_launch}
    if cpu_baseline:
        out["cpu_baseline"] = cpu_decode_baseline(kc[:4].cpu(), vc[:4].cpu(), qs[0, :4].cpu(), ks[0, :4].cpu(), vs[0, :4].cpu(), W,
                                                  f"4 of {B} batch elements, all {H} heads")
    return out


def cpu_decode_baseline(kc, vc, q, kn, vn, W, sample):
    """The reference's step path: chronological cat of the last W-1 rows + new row, non-causal SDPA."""
    torch.set_num_threads(os.cpu_count() or 1)
    B, H, _, D = kc.shape
    k_ctx, v_ctx = kc.transpose(1, 2), vc.transpose(1, 2)   # [B, n, H, D] views, n = W
    def one_step():
        k_ = torch.cat([k_ctx[:, 1:], kn[:, None]], 1).transpose(1, 2)
        v_ = torch.cat([v_ctx[:, 1:], vn[:, None]], 1).transpose(1, 2)
        torch.nn.functional.scaled_dot_product_attention(q[:, :, None], k_, v_, scale=SCALE, is_causal=False)

    dt, runs = _repeat_for(one_step, CPU_SECONDS / 2)
    sample = f"{sample}; {runs} steps in {dt * runs:.1f} s"
    return {"value": B * H * W * D * 4 / dt / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "port", "sample": sample, "seconds_per_step": dt}


def bench_kda_c5(steps, warmup, cpu_baseline=True):
    """Config 5: B4 T8192 H16 Dk=Dv=128, chunk 64."""
    from daisy_amd import ops
    B, T, H, Dk, Dv = 4, 8192, 16, 128, 128
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, generator=g, device=dev, dtype=torch.float32)
    q = torch.nn.functional.normalize(rn(B, T, H, Dk), dim=-1).bfloat16()
    k = torch.nn.functional.normalize(rn(B, T, H, Dk), dim=-1).bfloat16()
    v = rn(B, T, H, Dv).bfloat16()
    gl = torch.nn.functional.logsigmoid(rn(B, T, H, Dk))
    beta = torch.sigmoid(rn(B, T, H))
    ws = torch.empty(max(ops.kda_workspace_bytes(B, T, H, Dk, Dv), 1), dtype=torch.uint8, device=dev)
    ms, ms_first = time_settled(lambda: ops.kda_chunk_fwd(q, k, v, gl, beta, output_final_state=True, workspace=ws), steps, warmup)
    gl16 = gl.bfloat16()     # the dtype the reference's layer hands over (the gate's output follows its bf16 input)
    ms_g16 = time_gpu(lambda: ops.kda_chunk_fwd(q, k, v, gl16, beta, output_final_state=True, workspace=ws), steps, warmup)
    min_bytes = 5 * B * T * H * Dk * 2
    flops = 7.0 * Dk * Dv * B * T * H
    out = {"workload": "kda_c5_B4_T8192_H16_D128_chunk64", "ms": ms, "ms_first_steps_from_idle": ms_first, "min_bytes": min_bytes,
           "gbs_min_io": min_bytes / ms / 1e6, "frac_of_hbm_peak": min_bytes / ms / 1e6 / PEAK_HBM_GBS,
           "naive_flops": flops, "tflops_naive": flops / ms / 1e9,
           "g_dtype": "fp32", "ms_with_bf16_g": ms_g16, "frac_of_hbm_peak_with_bf16_g": min_bytes / ms_g16 / 1e6 / PEAK_HBM_GBS}
    # One decode step of the same layer at batch 64: the token-by-token kernel reads and writes the fp32 state once.
    Bd = 64
    S = torch.zeros(Bd, H, Dk, Dv, dtype=torch.float32, device=dev)
    qd, kd, vd = (rn(Bd, 1, H, Dk).bfloat16() for _ in range(3))
    gd, bd = torch.nn.functional.logsigmoid(rn(Bd, 1, H, Dk)), torch.sigmoid(rn(Bd, 1, H))
    ms_step = time_gpu(lambda: ops.kda_recurrent_fwd(qd, kd, vd, gd, bd, initial_state=S, inplace_state=True), 64, 8)
    state_bytes = 2 * Bd * H * Dk * Dv * 4
    out["decode_step_B64"] = {"ms": ms_step, "state_bytes_rw": state_bytes, "gbs": state_bytes / ms_step / 1e6,
                              "frac_of_hbm_peak": state_bytes / ms_step / 1e6 / PEAK_HBM_GBS}
    if cpu_baseline:
        import oracle
        torch.set_num_threads(os.cpu_count() or 1)
        Ts = 2048
        qc, kc, vc, gc, bc = (t[:1, :Ts, :2].cpu() for t in (q, k, v, gl, beta))
        dt, runs = _repeat_for(lambda: oracle.kda_recurrent(qc, kc, vc, gc, bc), CPU_SECONDS / 2)
        tok_heads = Ts * 2
        out["cpu_baseline"] = {"value": tok_heads / dt, "unit": "token-heads/s", "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"B=1, H=2 of 16, T={Ts} of {T} (naive recurrence); {runs} passes in {dt * runs:.1f} s", "seconds": dt,
                               "gpu_token_heads_per_s": B * T * H / (ms / 1e3)}
    return out


def attention_stack(L, vocab, dim, H, D, window, max_len):
    """A stack of attention layers with the attributes the model-level glue walks (embed, blocks, lm_head_w, window
    sizes ...): the attention part of a Daisy model, no MLPs, random bf16 weights."""
    import torch.nn as nn
    from daisy_amd import CausalSelfAttention

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.attn = CausalSelfAttention(dim, H, D, max_seq_len=max_len)
            with torch.no_grad():
                self.attn.qkvo_w.copy_((torch.randn(4, dim, dim) * 0.02).bfloat16())

        def prefill(self, x, ve, x0, attn_mask=None, debug=False):
            y, k, v = self.attn.prefill(x, ve, attn_mask, debug=debug)
            return x + y, k, v

        def step(self, x, ve, x0, k_ctx, v_ctx, pos, window):
            y, k, v = self.attn.step(x, k_ctx, v_ctx, pos, ve, window=window)
            return x + y, k, v

    class Stack(nn.Module):
        def __init__(self):
            super().__init__()
            self.embed = nn.Embedding(vocab, dim)
            self.blocks = nn.ModuleList([Block() for _ in range(L)])
            self.skip_map, self.skip_weights, self.ve_module_map = {}, None, {}
            self.lm_head_w = nn.Parameter(torch.randn(vocab, dim) * 0.02)
            self.window_size = self.attn_window_size = window
            self.eos_token_id = 0
            self.attn_num_heads, self.attn_head_dim = H, D
            self.bfloat16()

        # the model-level contract of the reference's generator (DaisyCore.prefill / step / reset_history,
        # models/daisy/daisy_core.py:294-370)
        def reset_history(self):
            for blk in self.blocks:
                blk.attn.reset_history()

        def prefill(self, ids):
            from daisy_amd import core
            return core.prefill(self, ids)

        def step(self, token, k_ctxs, v_ctxs, pos):
            from daisy_amd.functional import norm
            x = norm(self.embed(token.view(1, 1)))
            ks, vs = [], []
            for i, blk in enumerate(self.blocks):
                x, k, v = blk.step(x, None, x, k_ctxs[i], v_ctxs[i], pos, self.window_size)
                ks.append(k)
                vs.append(v)
            return torch.nn.functional.linear(norm(x).flatten(end_dim=1), self.lm_head_w).float(), ks, vs

    return Stack()


def bench_decode_b1(steps, warmup):
    """The regime of the reference's generator (inference/generate.py:76: batch 1) at the shape of
    model_specs/daisy_milli.yml (12 heads of 128, window 8192, model dim 1536), 12 attention layers, ring full:
    per-token time of a model step, eager and as one recorded HIP graph, and of the attention launches alone
    (the one-launch step over the 12 rings, back to back), against the bytes of ring a token reads."""
    from daisy_amd import KVCache, core, ops
    from daisy_amd.functional import NORM_EPS_BF16
    dev = "cuda:0"
    L, H, D, W, dim, vocab = 12, 12, 128, 8192, 1536, 8192
    torch.manual_seed(0)
    out = {"workload": f"decode_b1_L{L}_H{H}_D{D}_W{W}_dim{dim}", "batch": 1}
    with torch.no_grad():
        model = attention_stack(L, vocab, dim, H, D, W, 2 * W + 64).to(dev).eval()
        cache = KVCache(L=L, B=1, H=H, W=W, D=D, device=dev, dtype=torch.bfloat16)
        g = torch.Generator(device=dev).manual_seed(0)
        cache.k.copy_(torch.randn(cache.k.shape, generator=g, device=dev, dtype=torch.float32))
        cache.v.copy_(torch.randn(cache.v.shape, generator=g, device=dev, dtype=torch.float32))
        cache.t = t_before = W + 100                  # the ring has wrapped: every step reads W rows per layer
        tok = torch.randint(1, vocab, (1,), device=dev)

        def step_eager():
            cache.t = t_before
            return core.step(model, tok, cache)

        # host-bound: in a fresh process the first 0.1-0.2 s of eager steps run at half the settled rate (the host's
        # clocks), so the timed steps follow 0.3 s of untimed ones (a short run, --steps below 8, skips that)
        if steps >= 8:
            t_settle = time.perf_counter()
            while time.perf_counter() - t_settle < 0.3:
                step_eager()
            torch.cuda.synchronize()
        ms_eager = time_gpu(step_eager, max(steps, 64) if steps >= 8 else steps, max(warmup, 8) if steps >= 8 else warmup)
        recorded = core.GraphedStep(model, cache)

        def step_recorded():
            cache.t = t_before
            return recorded(tok)

        ms_graph = time_gpu(step_recorded, max(4 * steps, 16), max(warmup, 8))
        # the attention launches alone: the one-launch step (norm, RoPE, append, attention) on each layer's ring
        cos, sin = model.blocks[0].attn.rotary.cos, model.blocks[0].attn.rotary.sin
        raw = torch.randn(1, 3 * H, D, generator=g, device=dev).bfloat16()
        pos = torch.full((1,), t_before, dtype=torch.int32, device=dev)
        o = torch.empty(1, H, D, dtype=torch.bfloat16, device=dev)
        variants = {}
        for nsplit in (0, 8, 16, 32, 64):
            ws = torch.empty(max(ops.decode_workspace_bytes(1, H, D, W, nsplit), 1), dtype=torch.uint8, device=dev)

            def attn_layers():
                for i in range(L):
                    ops.attn_step(raw[:, :H], raw[:, H:2 * H], raw[:, 2 * H:], cache.k[i], cache.v[i], pos, cos=cos, sin=sin,
                                  eps=NORM_EPS_BF16, scale=SCALE, out=o, workspace=ws, nsplit=nsplit)

            graph = torch.cuda.CUDAGraph()
            attn_layers()
            torch.cuda.synchronize()
            with torch.cuda.graph(graph):
                attn_layers()
            variants["library_choice" if nsplit == 0 else f"nsplit{nsplit}"] = time_gpu(graph.replay, max(4 * steps, 16), 8)
            del graph
        # the step's two projections, one activation row against each layer's own matrices (12 different matrices per
        # replay: 226 MB, nothing stays in the caches), through the few-rows kernel and through the library's GEMM
        x_row = torch.randn(1, 1, dim, generator=g, device=dev).bfloat16()
        projections = {}
        for label, weights in (("qkv_4608x1536", [b.attn.qkvo_w[:3].flatten(end_dim=1) for b in model.blocks]),
                               ("out_1536x1536", [b.attn.qkvo_w[3] for b in model.blocks])):
            outs = [torch.empty(1, 1, w.shape[0], dtype=torch.bfloat16, device=dev) for w in weights]
            per = {}
            for name, fn in (("linear_rows", lambda w, y: ops.linear_rows(x_row, w, out=y)),
                             ("library_gemm", lambda w, y: torch.nn.functional.linear(x_row, w))):
                def all_layers():
                    for w, y in zip(weights, outs):
                        fn(w, y)
                graph = torch.cuda.CUDAGraph()
                all_layers()
                torch.cuda.synchronize()
                with torch.cuda.graph(graph):
                    all_layers()
                per[name] = time_gpu(graph.replay, max(4 * steps, 16), 8) / L
                del graph
            wbytes = weights[0].numel() * 2
            projections[label] = {"weight_bytes": wbytes, "us_per_call": per["linear_rows"] * 1e3,
                                  "gbs": wbytes / per["linear_rows"] / 1e6,
                                  "frac_of_hbm_peak": wbytes / per["linear_rows"] / 1e6 / PEAK_HBM_GBS,
                                  "us_per_call_library_gemm": per["library_gemm"] * 1e3}
        # the generator itself (inference/generate.py:61-285: prefill -> cache -> sample / step loop, one sequence):
        # a prompt of 2048 tokens, 128 new ones, greedy; as the reference drives it (model.prefill / model.step, eager)
        # and with the prompt through core.prefill and the step recorded as one graph
        from daisy_amd import Generator
        prompt = torch.randint(1, vocab, (2048,), generator=g, device=dev)
        generation = {}
        for label, kw in (("as_the_reference_drives_it", {}), ("recorded_step_direct_prefill", dict(record_steps=True, direct_prefill=True))):
            gen = Generator(model, window=W, seed=0, device=torch.device(dev), dtype=torch.bfloat16, temperature=0.0, **kw)
            best = None
            for _ in range(3):
                it = gen.generate(prompt, 128)
                n_new = 0
                try:
                    while True:
                        next(it)
                        n_new += 1
                except StopIteration as stop:
                    _, t_prefill, t_decode = stop.value
                if best is None or t_decode / max(n_new, 1) < best[2] / max(best[0], 1):
                    best = (n_new, t_prefill, t_decode)
            generation[label] = {"prompt_tokens": 2048, "new_tokens": best[0], "prefill_ms": best[1] * 1e3,
                                 "decode_ms_per_token": best[2] * 1e3 / max(best[0], 1),
                                 "tokens_per_s": best[0] / best[2] if best[2] > 0 else None}
            del gen
    nbytes = L * 2 * W * H * D * 2
    row = lambda ms: {"ms_per_token": ms, "gbs": nbytes / ms / 1e6, "frac_of_hbm_peak": nbytes / ms / 1e6 / PEAK_HBM_GBS}
    out.update({"kv_bytes_per_token": nbytes, "model_step_eager": row(ms_eager), "model_step_recorded_graph": row(ms_graph),
                "attention_launches_only_recorded_graph": {k: row(v) for k, v in variants.items()},
                "projections_one_row_recorded_graph": projections,
                "generator_prompt2048_greedy_best_of_3": generation,
                "what": "model step = embed, 12 x (norm, QKV projection, one-launch attention step, output projection, residual), "
                        "final norm, vocabulary projection; attention launches only = the 12 decode launches (+ their split "
                        "combines) replayed as one graph"})
    return out


def bench_next_rows(steps, warmup):
    """The callers either side of the kernels: model-level prefill / step glue on an attention stack,
    attention under training-time block masks, and the KDA layer."""
    import torch.nn as nn
    import torch.nn.functional as F
    from daisy_amd import CausalSelfAttention, KVCache, KimiLinearSelfAttention, build_block_window_masks, core, ops
    dev = "cuda:0"
    out = {}

    # ---- glue: 4 attention layers, 16 sequences, prompt 4100, ring of 4096 (wrapped) ----------------
    torch.manual_seed(0)
    with torch.no_grad():
        model = attention_stack(L=4, vocab=1024, dim=1024, H=8, D=128, window=4096, max_len=8192).to(dev).eval()
        Bs, T0, W, L = 16, 4100, 4096, 4
        ids = torch.randint(1, 1024, (Bs, T0), device=dev)
        cache = KVCache(L=L, B=Bs, H=8, W=W, D=128, device=dev, dtype=torch.bfloat16)

        def prefill_direct():
            cache.reset_history()
            return core.prefill(model, ids, cache)

        def prefill_stacked():   # the reference's route: stack [2, L, B, H, T, D], then one bulk write
            cache.reset_history()
            logits, kv = core.prefill(model, ids)
            cache.bulk_write_packed(kv, T0)
            return logits

        ms_direct = time_gpu(prefill_direct, max(steps // 5, 3), 2)
        ms_stacked = time_gpu(prefill_stacked, max(steps // 5, 3), 2)
        # a prompt that fits the ring: the pre-attention kernel writes K and V into the ring's slots itself
        ids_full, ids, T0_full, T0 = ids, ids[:, :2048].contiguous(), T0, 2048
        ms_direct_fit = time_gpu(prefill_direct, max(steps // 5, 3), 2)
        ms_stacked_fit = time_gpu(prefill_stacked, max(steps // 5, 3), 2)
        ids, T0 = ids_full, T0_full
        prefill_direct()
        tok = torch.randint(1, 1024, (Bs,), device=dev)
        t_before = cache.t

        def step_ring():
            cache.t = t_before
            return core.step(model, tok, cache)

        def step_views():        # chronological copies, the reference's route (cache.view + write)
            cache.t = t_before
            x = x0 = F.rms_norm(model.embed(tok.view(-1, 1)), (1024,))
            for i, blk in enumerate(model.blocks):
                kc, vc = cache.view(i)
                x, kn, vn = blk.step(x, None, x0, kc, vc, cache.t, W)
                cache.write(i, kn, vn)
            cache.advance()
            return F.linear(F.rms_norm(x, (1024,)).flatten(end_dim=1), model.lm_head_w).float()

        ms_ring = time_gpu(step_ring, 64, 8)
        ms_views = time_gpu(step_views, 64, 8)
        recorded = core.GraphedStep(model, cache)

        def step_recorded():     # the same walk replayed as one HIP graph, position in device memory
            cache.t = t_before
            return recorded(tok)

        ms_recorded = time_gpu(step_recorded, 64, 8)
    out["model_glue_L4_B16_T4100_W4096"] = {
        "prefill_ms_ring_written_per_layer": ms_direct, "prefill_ms_stack_then_bulk_write": ms_stacked,
        "prefill_ms_T2048_written_in_place": ms_direct_fit, "prefill_ms_T2048_stack_then_bulk_write": ms_stacked_fit,
        "step_ms_ring_in_place": ms_ring, "step_ms_ring_in_place_recorded_graph": ms_recorded,
        "step_ms_chronological_views": ms_views,
        "kv_bytes_per_step": 2 * L * Bs * 8 * min(t_before + 1, W) * 128 * 2}
    del model, cache, recorded

    # ---- training-time block masks as per-row lower bounds: one sequence of 32768, 3 documents ----
    with torch.no_grad():
        T, H, D, wblk = 32768, 8, 128, 8          # window of 8 blocks of 128 = 1024 keys
        seq = torch.randint(1, 1000, (T,), device=dev)
        seq[[9000, 20000]] = 0
        masks = build_block_window_masks(seq, wblk, 4, eos_token_id=0)
        g = torch.Generator(device=dev).manual_seed(0)
        q, k, v = (torch.randn(1, T, H, D, generator=g, device=dev).bfloat16() for _ in range(3))
        rows = {}
        for name, m in (("long", masks[0]), ("short", masks[1])):
            lo = m.doc_start.long()
            pairs = int((torch.arange(T, device=dev) - lo + 1).sum())
            o_buf = torch.empty_like(q)
            ms, ms_first = time_settled(lambda: ops.prefill_attention(q, k, v, window=None, doc_start=m.doc_start, scale=SCALE, out=o_buf),
                                        max(steps // 2, 5), 3, seconds=0.2)
            fl = 4.0 * D * H * pairs
            rows[name] = {"ms": ms, "ms_first_steps_from_idle": ms_first, "flops": fl, "tflops": fl / ms / 1e9,
                          "frac_of_peak": fl / ms / 1e9 / PEAK_BF16_TFLOPS}
    out["block_masks_B1_T32768_H8_D128_w8blocks"] = rows

    # ---- the KDA layer: dim 2048, 16 heads of 128, B4 T8192; one decode step at batch 64 ------------
    with torch.no_grad():
        torch.manual_seed(0)
        layer = KimiLinearSelfAttention(2048, 16, max_seq_len=8192, head_dim=128).to(dev).eval()
        x = torch.randn(4, 8192, 2048, device=dev).bfloat16()
        ms_layer, ms_layer_first = time_settled(lambda: layer(x, None), max(steps // 10, 3), 2, seconds=0.3)
        xs = torch.randn(64, 64, 2048, device=dev).bfloat16()
        layer.prefill(xs, None)
        x1 = torch.randn(64, 1, 2048, device=dev).bfloat16()
        ms_step = time_gpu(lambda: layer.step(x1, None, None, 64, None, None), 32, 4)
        # the same step replayed as a HIP graph (state and windows are updated in place at fixed addresses)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            layer.step(x1, None, None, 64, None, None)
        ms_step_graph = time_gpu(graph.replay, 32, 4)
        del graph
        # one sequence (the generator's regime): the layer's bias-free projections read their weights through the few-rows kernel
        layer.reset_history()
        layer.prefill(xs[:1], None)
        ms_step_b1 = time_gpu(lambda: layer.step(x1[:1], None, None, 64, None, None), 64, 16)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            layer.step(x1[:1], None, None, 64, None, None)
        ms_step_b1_graph = time_gpu(graph.replay, 64, 8)
    out["kimi_layer_dim2048_H16"] = {"forward_ms_B4_T8192": ms_layer, "forward_ms_first_steps_from_idle": ms_layer_first, "step_ms_B64": ms_step,
                                     "step_ms_B64_recorded_graph": ms_step_graph, "step_ms_B1": ms_step_b1,
                                     "step_ms_B1_recorded_graph": ms_step_b1_graph}
    del graph
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--only", default=None, help="prefill | ceiling | plumbing | module | long | decode | decode_b1 | kda | next | copy (default: all but copy)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every kernel here works on one GPU's share of the (batch, head) "
                 "range and nothing is exchanged between GPUs; run with --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs an AMD GPU")
    from daisy_amd import _lib
    _lib.load()

    if args.only == "copy":
        print(json.dumps(bench_copy(args.steps, args.warmup)))
        return
    want = lambda name: args.only in (None, name)
    cpu = not args.no_cpu
    extra = {}
    head = bench_prefill_c2(args.steps, args.warmup, cpu) if want("prefill") else None
    if want("ceiling"):
        extra["matrix_pipe_ceiling"] = {
            "what": "register-only v_mfma_f32_32x32x16_bf16 on every SIMD, 2 wavefronts each, ~25 ms per run",
            "mfma_only": probe_matrix_rate(False, 80000),
            "mfma_only_zero_operands": probe_matrix_rate_data("zeros"),
            "mfma_only_normal_operands": dict(
                probe_matrix_rate_data("normal"),
                what="the same instruction stream on N(0,1) bf16 operands: the sustained rate of the matrix pipe ALONE on data like "
                     "the benchmark's; the power management lowers the clock until the chip stays inside its power limit"),
            "mfma_with_attention_mix_and_lds_operands_on_normal_data": dict(
                probe_matrix_rate_data("normal", iters=50000, variant=3),
                what="the stream of mfma_with_attention_mix_and_lds_operands below, sustained for a second, with the LDS tile and "
                     "the B operands holding N(0,1) values: what the attention loop's instruction mix can reach on such data"),
            "mfma_with_attention_vector_mix": probe_matrix_rate(True, 60000),
            "mfma_with_attention_mix_and_lds_operands": dict(
                probe_matrix_rate(2, 50000),
                what="per MFMA 3 fma + 1 exp2, A operands read from LDS with the kernel's K / V access patterns eight "
                     "MFMAs ahead; no global memory, barriers or masks: the stream ceiling of the two-wavefronts-per-SIMD layout"),
        }
    if want("plumbing"):
        extra["plumbing_c1"] = bench_plumbing_c1(args.steps, args.warmup, cpu)
    if want("module"):
        extra["module_c2"] = bench_module_c2(max(args.steps // 2, 4), max(args.warmup // 2, 2))
    if want("long"):
        extra["prefill_c3_B1_T65536_H16_D128"] = bench_prefill_c3(max(args.steps // 5, 4), max(args.warmup // 2, 2))
    if want("decode"):
        extra["decode_c4"] = bench_decode_c4(256, 16, cpu)
        extra["hbm_read_ceiling"] = dict(probe_read_rate(), what="read-only stream of 2 GiB, 8192 workgroups, 128 B in flight per lane")
    if want("decode_b1"):
        extra["decode_b1"] = bench_decode_b1(args.steps, args.warmup)
    if want("next"):
        extra["next_rows"] = bench_next_rows(args.steps, args.warmup)
    if want("kda"):
        try:
            extra["kda_c5"] = bench_kda_c5(max(args.steps // 5, 4), max(args.warmup // 2, 2), cpu)
        except RuntimeError as e:
            extra["kda_c5"] = {"error": str(e)}

    line = {
        "metric": "prefill attn TFLOP/s + decode KV GB/s (fraction of MI355X roofline)",
        "value": None if head is None else head["tflops_full"],
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": None if head is None else head["ms_full"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "windowed prefill attention, fused RoPE: B=8 T=4096 H=8 D=128 window=1024 (BASELINE configs[1])",
                   "timed": "K rotation pre-pass + attention kernel, inputs and outputs in HBM"},
    }
    if head is not None:
        # What precedes the timed steps, at the top level: the GPU is brought to its settled clocks by a run of the same
        # step (pre_timed_launches, then `warmup` more); the first `steps` steps from an idle GPU are reported beside it.
        line["pre_timed_launches"] = head["full_sustained_launches"]
        line["ms_per_step_first_steps_from_idle"] = head["ms_full_first_steps_from_idle"]
        line["value_first_steps_from_idle"] = head["flops"] / head["ms_full_first_steps_from_idle"] / 1e9
        line["config"]["timed"] += (f"; {args.steps} steps after {head['full_sustained_launches']} back-to-back launches of the same step "
                                    f"and {args.warmup} warm-up steps (settled clocks); from an idle GPU the first {args.steps} steps "
                                    f"take {head['ms_full_first_steps_from_idle']:.4f} ms each")
        # The roofline figure is the lower of the burst median and the sustained run (at least a second of launches).
        burst, sus = head["tflops_kernel"], head["sustained"]["tflops_kernel"]
        use_sus = sus < burst
        traffic, traffic_source = recorded_traffic(PREFILL_C2_TRAFFIC_FILE, PREFILL_C2_KERNEL)
        line["roofline"] = {"bound": "mfma", "achieved": min(burst, sus), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                            "frac": min(burst, sus) / PEAK_BF16_TFLOPS, "traffic": traffic,
                            "traffic_source": traffic_source, "traffic_min_bytes": head["min_hbm_bytes"],
                            "kernel": PREFILL_C2_KERNEL,
                            "ms": head["sustained"]["ms_kernel"] if use_sus else head["ms_kernel"],
                            "timing": ("sustained: mean over %d back-to-back launches (%.2f s)" % (head["sustained"]["launches"], head["sustained"]["seconds"]))
                                      if use_sus else "median of per-launch HIP event pairs over the timed steps",
                            "burst_tflops": burst, "sustained_tflops": sus}
        if "cpu_baseline" in head:
            line["cpu_baseline"] = head.pop("cpu_baseline")
        extra["prefill_c2"] = head
    line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
