#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

A step is one forward + backward of the headline workload (B=2, H=32, N=4096,
D=128, causal, fp16) through flash_attn_func(...).backward(dO): every kernel the
autograd path launches is inside the timed region, inputs are resident in HBM.

Prints ONE JSON line.  `value` is forward+backward TFLOP/s with the algorithmic
FLOP count 3.5 * 4*B*H*N^2*D / 2 (causal); the forward alone, the per-kernel
roofline of the slowest kernel, every other configuration, and a CPU baseline
(the fp32 oracle on the host cores, a bounded sample) ride along.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "flash-attention-v100_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_TFLOPS = 2516.6  # MI355X dense fp16 MFMA, vendor figure (256 CUs x 4 SIMDs x 1024 FLOP/clk at NOMINAL_MHZ)
NOMINAL_MHZ = 2400
PEAK_HBM_GBS = 8000.0  # MI355X HBM3E, vendor figure
SUSTAINED_LAUNCHES = 300
SETTLE_MS = 100.0  # untimed load before the warm-up steps (power management ramp)

CONFIGS = [  # name, B, H, N, D, causal
    ("plumbing_b1_h4_n128_d64", 1, 4, 128, 64, False),
    ("bert_base_b16_h12_n512_d64", 16, 12, 512, 64, False),
    ("gpt_causal_b4_h16_n1024_d64", 4, 16, 1024, 64, True),
    ("llama7b_b2_h32_n4096_d128_causal", 2, 32, 4096, 128, True),
    ("long_context_b1_h16_n16384_d128_causal", 1, 16, 16384, 128, True),
]
HEADLINE = 3


def fwd_flops(B, H, N, D, causal):
    f = 4.0 * B * H * N * N * D
    return f * 0.5 if causal else f


def min_hbm_bytes(B, H, N, D):
    """Algorithmic HBM bytes: forward reads q, k, v and writes o + lse; backward reads q, k, v, o, dO, lse
    and writes dq, dk, dv."""
    t = B * N * H * D * 2
    stat = B * H * N * 4
    return 4 * t + stat, 8 * t + stat


def load_c_abi():
    """ctypes binding of the entry points of include/fused_mha.h that the per-kernel timing uses."""
    import ctypes
    import torch  # noqa: F401  (first, so that the library binds to the HIP runtime torch loaded)

    path = os.path.join(ROOT, "flash-attention-v100_amd", "flash_attn_v100", "lib", "libfused_mha.so")
    if not os.path.exists(path):
        sys.exit("bench.py: %s is not built (python setup.py build_ext --inplace in flash-attention-v100_amd/)" % path)
    lib = ctypes.CDLL(path)
    vp, i, f, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t
    lib.fused_mha_forward.argtypes = [vp] * 5 + [i] * 5 + [f, i, vp]
    lib.fused_mha_backward_workspace_bytes.argtypes = [i] * 4
    lib.fused_mha_backward_workspace_bytes.restype = sz
    lib.fused_mha_backward_min_workspace_bytes.argtypes = [i] * 4
    lib.fused_mha_backward_min_workspace_bytes.restype = sz
    lib.fused_mha_backward_delta.argtypes = [vp, vp, vp, vp, sz] + [i] * 4 + [vp]
    lib.fused_mha_backward_dq.argtypes = [vp] * 6 + [sz, vp] + [i] * 4 + [f, i, vp]
    lib.fused_mha_backward_dkdv.argtypes = [vp] * 6 + [sz, vp, vp] + [i] * 4 + [f, i, vp]
    return lib


def sustained_ms(fn, launches=SUSTAINED_LAUNCHES, warmup=10):
    """Per-call device-event times of `launches` back-to-back calls; returns (median, list)."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(launches + 1)]
    ev[0].record()
    for n in range(launches):
        fn()
        ev[n + 1].record()
    torch.cuda.synchronize()
    ts = [ev[n].elapsed_time(ev[n + 1]) for n in range(launches)]
    return sorted(ts)[launches // 2], ts


def time_ms(fn, steps, warmup):
    """Device-event time per call on torch's current stream (the stream every
    kernel here is launched on)."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


# The shader clock and the socket power while a kernel runs.  amd-smi (or rocm-smi) is started
# by a helper process (this file run with --sampler) that was itself started before this process
# touched the GPU: a process that has initialised the GPU starts no programs.  The helper waits
# for a line on its stdin, samples, and answers with one JSON line.
def parse_amd_smi(text):
    """Socket power (W) and per-XCD shader clocks (MHz) from the text of `amd-smi metric -p -c`."""
    import re

    res = {"sclk_mhz": None, "socket_power_w": None, "xcd_mhz": None}
    m = re.search(r"SOCKET_POWER:\s*(\d+)\s*W", text)
    if m:
        res["socket_power_w"] = int(m.group(1))
    clk = [int(x) for x in re.findall(r"GFX_\d+:\s*\n\s*CLK:\s*(\d+)\s*MHz", text)]
    if clk:
        res["xcd_mhz"] = clk
        res["sclk_mhz"] = round(sum(clk) / len(clk))
    return res


def parse_rocm_smi(text):
    """Shader clock (MHz) from the text of `rocm-smi --showclocks`, or None."""
    import re

    m = re.search(r"sclk clock level:\s*\d+:\s*\((\d+)Mhz\)", text)
    return int(m.group(1)) if m else None


def sampler_main():
    import subprocess

    for _ in sys.stdin:
        res = {"sclk_mhz": None, "socket_power_w": None, "xcd_mhz": None}
        try:
            res = parse_amd_smi(subprocess.run(["amd-smi", "metric", "-p", "-c"], capture_output=True, text=True,
                                               timeout=30).stdout)
        except (OSError, subprocess.SubprocessError) as e:
            res["amd_smi_error"] = str(e)
        if res["sclk_mhz"] is None:
            try:
                res["sclk_mhz"] = parse_rocm_smi(subprocess.run(["rocm-smi", "--showclocks"], capture_output=True,
                                                                text=True, timeout=30).stdout)
            except (OSError, subprocess.SubprocessError) as e:
                res["rocm_smi_error"] = str(e)
        print(json.dumps(res), flush=True)


def start_clock_sampler():
    import subprocess

    try:
        return subprocess.Popen([sys.executable, os.path.abspath(__file__), "--sampler"], stdin=subprocess.PIPE,
                                stdout=subprocess.PIPE, text=True)
    except OSError:
        return None


def sclk_under_load(sampler, fn, settle_s=1.0, limit_s=40.0):
    """One sample of the shader clock (MHz, mean over the XCDs) and the socket power (W) while fn() is launched
    back to back; a dict of None values if they cannot be read."""
    import select
    import torch

    nothing = {"sclk_mhz": None, "socket_power_w": None, "xcd_mhz": None}
    if sampler is None or sampler.poll() is not None:
        return nothing
    t0 = time.perf_counter()
    asked = False
    while time.perf_counter() - t0 < limit_s:
        for _ in range(100):
            fn()
        torch.cuda.synchronize()
        if not asked and time.perf_counter() - t0 > settle_s:
            sampler.stdin.write("sample\n")
            sampler.stdin.flush()
            asked = True
        if asked and select.select([sampler.stdout], [], [], 0)[0]:
            try:
                return json.loads(sampler.stdout.readline())
            except ValueError:
                return nothing
    return nothing


def occupancy_sweep(path):
    """Duration of the forward, dQ and dK/dV kernels of B1 N4096 D128 non-causal as the number of heads, and with
    it the number of busy CUs, grows: every work group does the same work in every row of the table."""
    import torch

    lib = load_c_abi()
    B, N, D = 1, 4096, 128
    scale = 1.0 / math.sqrt(D)
    with open(path, "w") as fh:
        fh.write("# B1 N4096 D128 non-causal; medians of 100 launches, microseconds; 256 CUs; work groups per kernel:\n")
        fh.write("# forward heads*16 blocks (256 queries each), dQ and dK/dV heads*32 (128 rows each); forward and dQ launches are persistent\n")
        fh.write("# heads fwd_groups fwd_us fwd_us_per_round dq_us dkdv_us\n")
        for H in (2, 4, 8, 16, 32, 64):
            q, k, v, do = make_device_inputs(B, H, N, D)
            out = torch.empty_like(q)
            lse = torch.empty((B, H, N), dtype=torch.float32, device=q.device)
            nbytes = lib.fused_mha_backward_workspace_bytes(B, H, N, D)
            ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
            dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
            s = torch.cuda.current_stream().cuda_stream
            p = lambda t: t.data_ptr()
            calls = [
                lambda: lib.fused_mha_forward(p(q), p(k), p(v), p(out), p(lse), B, H, N, N, D, scale, 0, s),
                lambda: lib.fused_mha_backward_delta(p(out), p(do), p(lse), p(ws), nbytes, B, H, N, D, s),
                lambda: lib.fused_mha_backward_dkdv(p(q), p(k), p(v), p(do), p(lse), p(ws), nbytes, p(dk), p(dv),
                                                    B, H, N, D, scale, 0, s),
                lambda: lib.fused_mha_backward_dq(p(q), p(k), p(v), p(do), p(lse), p(ws), nbytes, p(dq), B, H, N, D, scale, 0, s),
            ]
            for fn in calls:  # in dependency order: the dQ pass reads the dS tiles the dK/dV pass wrote
                if fn() != 0:
                    sys.exit("bench.py: a kernel of the occupancy sweep failed")
            us = [sustained_ms(fn, 100, 20)[0] * 1e3 for fn in (calls[0], calls[3], calls[2])]
            groups = H * N // 256
            rounds = max(1, -(-groups // 256))
            fh.write("%d %d %.1f %.1f %.1f %.1f\n" % (H, groups, us[0], us[0] / rounds, us[1], us[2]))


def make_device_inputs(B, H, N, D, seed=20):
    import torch

    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return [torch.randn((B, N, H, D), generator=g, dtype=torch.float32).to(torch.float16).cuda() for _ in range(4)]


def bench_config(B, H, N, D, causal, steps, warmup):
    import torch
    from flash_attn_v100 import flash_attn_func

    q, k, v, do = make_device_inputs(B, H, N, D)
    q.requires_grad_(), k.requires_grad_(), v.requires_grad_()
    scale = 1.0 / math.sqrt(D)

    def fwd():
        with torch.no_grad():
            flash_attn_func(q, k, v, scale, causal)

    def fwd_bwd():
        out = flash_attn_func(q, k, v, scale, causal)
        out.backward(do)
        q.grad = k.grad = v.grad = None

    t_f = sustained_ms(fwd, max(50, steps), max(10, warmup))[0]
    t_fb = sustained_ms(fwd_bwd, max(50, steps), max(10, warmup))[0]
    ff = fwd_flops(B, H, N, D, causal)
    bytes_f, bytes_b = min_hbm_bytes(B, H, N, D)
    return {"fwd_ms": t_f, "fwd_bwd_ms": t_fb, "fwd_tflops": ff / t_f / 1e9, "fwd_bwd_tflops": 3.5 * ff / t_fb / 1e9,
            "fwd_hbm_frac": bytes_f / (t_f * 1e-3) / (PEAK_HBM_GBS * 1e9),
            "fwd_bwd_hbm_frac": (bytes_f + bytes_b) / (t_fb * 1e-3) / (PEAK_HBM_GBS * 1e9)}


def kernel_times(B, H, N, D, causal, steps, warmup):
    """Average duration of each kernel of the path flash_attn_func takes, timed one by one through the C ABI with
    device events on the launch stream: forward; delta; the dK/dV pass that also writes the dS tiles; the dQ pass
    that reads them.  `fmha_bwd_dq_kernel` (the dQ pass of the minimum-workspace path, which recomputes S and dP) is
    timed beside them for comparison."""
    import torch

    lib = load_c_abi()
    q, k, v, do = make_device_inputs(B, H, N, D)
    scale = 1.0 / math.sqrt(D)
    out = torch.empty_like(q)
    lse = torch.empty((B, H, N), dtype=torch.float32, device=q.device)
    nbytes = lib.fused_mha_backward_workspace_bytes(B, H, N, D)
    small = lib.fused_mha_backward_min_workspace_bytes(B, H, N, D)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    s = torch.cuda.current_stream().cuda_stream
    p = lambda t: t.data_ptr()
    c = int(causal)
    spill = nbytes > small
    calls = {
        "fmha_fwd_kernel": lambda: lib.fused_mha_forward(p(q), p(k), p(v), p(out), p(lse), B, H, N, N, D, scale, c, s),
        "fmha_bwd_delta_kernel": lambda: lib.fused_mha_backward_delta(p(out), p(do), p(lse), p(ws), nbytes, B, H, N, D, s),
        "fmha_bwd_dkdv_kernel": lambda: lib.fused_mha_backward_dkdv(p(q), p(k), p(v), p(do), p(lse), p(ws), nbytes,
                                                                     p(dk), p(dv), B, H, N, D, scale, c, s),
        ("fmha_bwd_dq_spill_kernel" if spill else "fmha_bwd_dq_kernel"):
            lambda: lib.fused_mha_backward_dq(p(q), p(k), p(v), p(do), p(lse), p(ws), nbytes, p(dq), B, H, N, D, scale, c, s),
    }
    if spill:
        calls["fmha_bwd_dq_kernel"] = lambda: lib.fused_mha_backward_dq(p(q), p(k), p(v), p(do), p(lse), p(ws), small,
                                                                         p(dq), B, H, N, D, scale, c, s)
    for name, fn in calls.items():  # each pass once, in dependency order, and every return code checked
        rc = fn()
        if rc != 0:
            sys.exit("bench.py: %s returned %d" % (name, rc))
    return {name: time_ms(fn, steps, warmup) for name, fn in calls.items()}


def cpu_baseline(B, H, N, D, causal, budget_s=12.0):
    """The fp32 oracle (forward + analytic backward) on the host cores, over as
    many (batch, head) slices of the headline workload as fit the time budget."""
    import torch
    from oracle import attention_oracle as ao

    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0")) or 1 << 30)
    torch.set_num_threads(cores)
    g = torch.Generator(device="cpu")
    g.manual_seed(20)
    q, k, v, do = (torch.randn((1, N, 1, D), generator=g).half() for _ in range(4))
    scale = 1.0 / math.sqrt(D)
    ao.attention_forward(q[:, :256], k[:, :256], v[:, :256], scale, causal)  # warm the thread pool
    others = {}
    for cname, cB, cH, cN, cD, cc in CONFIGS[:HEADLINE]:  # the smaller configurations, whole: warm-up + median of 3
        cq, ck, cv, cdo = (torch.randn((cB, cN, cH, cD), generator=g).half() for _ in range(4))
        cs, times = 1.0 / math.sqrt(cD), []
        for rep in range(4):
            t0 = time.perf_counter()
            ao.attention_forward(cq, ck, cv, cs, cc)
            ao.attention_backward(cq, ck, cv, cdo, cs, cc)
            times.append(time.perf_counter() - t0)
        med = sorted(times[1:])[1]
        others[cname] = {"seconds": round(med, 5), "tflops": round(3.5 * fwd_flops(cB, cH, cN, cD, cc) / med / 1e12, 5)}
    done, t0 = 0, time.perf_counter()
    while done < B * H:
        ao.attention_forward(q, k, v, scale, causal)
        ao.attention_backward(q, k, v, do, scale, causal)
        done += 1
        if time.perf_counter() - t0 > budget_s:
            break
    dt = time.perf_counter() - t0
    flops = 3.5 * fwd_flops(1, 1, N, D, causal) * done
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port", "other_configs": others,
            "sample": f"{done} of {B * H} (batch, head) slices of the headline workload, fwd+bwd, "
                      f"fp32 torch on {cores} threads, {dt:.1f} s; dense N^2 work done, causal-halved FLOPs counted"}


def main():
    if sys.argv[1:] == ["--sampler"]:
        return sampler_main()
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # defaults: the power management needs 20-30 ms of load after an idle period before the launch
    # durations settle, so the warm-up covers that (40 steps are about 50 ms)
    ap.add_argument("--steps", type=int, default=60)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--headline-only", action="store_true")
    ap.add_argument("--config-index", type=int, default=HEADLINE,
                    help="which entry of CONFIGS is the measured workload (default: the headline, %d); "
                         "other indices are for profiling the other configurations" % HEADLINE)
    ap.add_argument("--launch-trace", metavar="FILE",
                    help="write the duration of each back-to-back forward launch of a longer run to FILE "
                         "(launch index, milliseconds since the first launch, duration in milliseconds)")
    ap.add_argument("--launch-trace-count", type=int, default=6000,
                    help="launches in the --launch-trace run (default 6000, about two seconds)")
    ap.add_argument("--occupancy-sweep", metavar="FILE",
                    help="write kernel durations of B1 N4096 D128 for 2 .. 64 heads (32 .. 1024 forward work groups) to FILE")
    ap.add_argument("--no-clock-sample", action="store_true", help="do not read the shader clock under load (rocm-smi)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy three times (reference point for HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus %d is not supported (no multi-GPU path exists)" % args.gpus)

    # (not under a profiler: its preloaded library has initialised the GPU before this program started)
    profiled = "rocprof" in os.environ.get("LD_PRELOAD", "") or any(key.startswith("ROCPROF") for key in os.environ)
    sampler = None if args.no_clock_sample or profiled else start_clock_sampler()  # before anything touches the GPU

    import torch
    from flash_attn_v100 import flash_attn_func

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    props = torch.cuda.get_device_properties(0)
    clock_ghz = props.clock_rate / 1e6 if hasattr(props, "clock_rate") else 2.4
    peak_check = props.multi_processor_count * 4 * 1024 * clock_ghz / 1e3  # CUs x SIMDs x flop/clk x GHz

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    name, B, H, N, D, causal = CONFIGS[args.config_index]
    q, k, v, do = make_device_inputs(B, H, N, D)
    q.requires_grad_(), k.requires_grad_(), v.requires_grad_()
    scale = 1.0 / math.sqrt(D)

    def step():
        out = flash_attn_func(q, k, v, scale, causal)
        out.backward(do)
        q.grad = k.grad = v.grad = None

    # After an idle period the first 20-30 ms of load run slower while the power management ramps up
    # (profiles/headline_forward_launch_index_vs_duration.md), whatever --warmup says: SETTLE_MS of untimed steps
    # come first, then the --warmup steps, then the timed ones.
    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < SETTLE_MS:
        for _ in range(5):
            step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ff = fwd_flops(B, H, N, D, causal)
    value = 3.5 * ff / ms / 1e9

    def fwd_only():
        with torch.no_grad():
            flash_attn_func(q, k, v, scale, causal)

    fwd_ms = time_ms(fwd_only, args.steps, args.warmup)
    fwd_tflops = ff / fwd_ms / 1e9

    # sustained figures: median of per-call device-event times over many back-to-back calls
    fwd_sus_ms, fwd_trace = sustained_ms(fwd_only)
    step_sus_ms, _ = sustained_ms(step)
    if args.launch_trace:
        torch.cuda.synchronize()
        time.sleep(2.0)  # let the clocks settle back after the work above
        _, long_trace = sustained_ms(fwd_only, args.launch_trace_count, 0)
        with open(args.launch_trace, "w") as fh:
            fh.write("# %s forward, %d launches back to back after 2 s of idle: launch index, ms since the first "
                     "launch, duration in ms\n" % (name, len(long_trace)))
            at = 0.0
            for n, t in enumerate(long_trace):
                fh.write("%d %.3f %.4f\n" % (n, at, t))
                at += t

    if args.occupancy_sweep:
        occupancy_sweep(args.occupancy_sweep)

    # the shader clock the device runs at under these two loads (the published peak assumes NOMINAL_MHZ)
    fwd_load = sclk_under_load(sampler, fwd_only)
    step_load = sclk_under_load(sampler, step)
    if sampler is not None:
        sampler.stdin.close()
    fwd_mhz, step_mhz = fwd_load["sclk_mhz"], step_load["sclk_mhz"]
    clock = {"nominal_mhz": NOMINAL_MHZ, "fwd_sclk_mhz": fwd_mhz, "step_sclk_mhz": step_mhz,
             "fwd_socket_power_w": fwd_load["socket_power_w"], "step_socket_power_w": step_load["socket_power_w"],
             "fwd_xcd_mhz": fwd_load["xcd_mhz"],
             "source": "amd-smi metric -p -c (else rocm-smi --showclocks), one sample after a second of back-to-back launches",
             "peak_at_fwd_sclk_tflops": PEAK_TFLOPS * fwd_mhz / NOMINAL_MHZ if fwd_mhz else None,
             "peak_at_step_sclk_tflops": PEAK_TFLOPS * step_mhz / NOMINAL_MHZ if step_mhz else None}

    # per-kernel durations and the roofline of the slowest kernel
    kt = kernel_times(B, H, N, D, causal, args.steps, args.warmup)
    # algorithmic FLOPs per launch: the GEMMs of the 5-GEMM backward / 2-GEMM forward
    # count that each kernel produces (recomputed S and dP in the dQ pass are not counted)
    alg = {"fmha_fwd_kernel": ff, "fmha_bwd_dkdv_kernel": 2.0 * ff, "fmha_bwd_dq_spill_kernel": 0.5 * ff,
           "fmha_bwd_dq_kernel": 0.5 * ff}
    on_path = [n for n in alg if n in kt and not (n == "fmha_bwd_dq_kernel" and "fmha_bwd_dq_spill_kernel" in kt)]
    dominant = max(on_path, key=lambda n: kt[n])
    achieved = alg[dominant] / kt[dominant] / 1e9
    traffic = traffic_commit = None
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath) and args.config_index == HEADLINE:  # the counters were taken on the headline workload
        tj = json.load(open(tpath))
        traffic = tj.get(dominant)
        traffic_commit = tj.get("_commit")
    roofline = {"bound": "mfma", "kernel": dominant, "achieved": achieved, "peak": PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": achieved / PEAK_TFLOPS, "traffic": traffic,
                "traffic_measured_at_commit": traffic_commit,
                # the same against the peak at the shader clock measured under the fwd+bwd load (informative)
                "frac_at_step_sclk": achieved / clock["peak_at_step_sclk_tflops"] if clock["peak_at_step_sclk_tflops"] else None,
                "kernel_ms": kt, "peak_check_tflops": peak_check}

    others = {}
    if not args.headline_only:
        for cname, cB, cH, cN, cD, cc in CONFIGS:
            r = bench_config(cB, cH, cN, cD, cc, args.steps, args.warmup)
            r["fwd_frac_peak"] = r["fwd_tflops"] / PEAK_TFLOPS
            r["fwd_bwd_frac_peak"] = r["fwd_bwd_tflops"] / PEAK_TFLOPS
            others[cname] = {key: round(val, 5) for key, val in r.items()}

    line = {
        "metric": "fwd+bwd TFLOP/s, B%d H%d N%d D%d %s fp16 (fwd alone in 'fwd')" % (
            B, H, N, D, "causal" if causal else "non-causal"),
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "settle_ms_before_warmup": SETTLE_MS,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": name, "batch": B, "heads": H, "seq_len": N, "head_dim": D, "causal": causal},
        "frac_of_peak": value / PEAK_TFLOPS,
        "fwd": {"ms": fwd_ms, "tflops": fwd_tflops, "frac_of_peak": fwd_tflops / PEAK_TFLOPS},
        "value_sustained": {"launches": SUSTAINED_LAUNCHES, "ms_median": step_sus_ms,
                            "tflops": 3.5 * ff / step_sus_ms / 1e9,
                            "frac_of_peak": 3.5 * ff / step_sus_ms / 1e9 / PEAK_TFLOPS},
        "fwd_sustained": {"launches": SUSTAINED_LAUNCHES, "ms_median": fwd_sus_ms, "tflops": ff / fwd_sus_ms / 1e9,
                          "frac_of_peak": ff / fwd_sus_ms / 1e9 / PEAK_TFLOPS},
        "roofline": roofline,
        "clock": clock,
        "all_configs": others,
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(B, H, N, D, causal)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
