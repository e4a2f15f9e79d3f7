"""Benchmark of the MoE hot path on one MI355X.

A step = one pass of the path over one batch: routing sort -> layer0 (row gather fused into the grouped
GEMM) -> layer1 grouped GEMM (top-k weight in the epilogue) -> top-k gather-reduce to token order.
Workload at N=1: C3, the Mixtral-shape layer the metric is quoted on (T=8192, H=4096, F=14336, E=8,
top-2, bf16), synthetic data, inputs resident in HBM before the timed region.

Prints ONE JSON line: whole-step throughput in TFLOP/s (algorithmic GEMM FLOPs of the step / step
time), the roofline object of the dominant kernel (grouped GEMM, MFMA-bound) measured with HIP events
inside the timed region (mean, median and min per launch), the shader clock sampled during a sustained
loop of the same two GEMMs with the clock-adjusted peak beside the published one, per-kernel figures for
the other kernels and shapes of the path, and the CPU oracle timed on a bounded sample.
"""
import argparse
import json
import os
import statistics
import subprocess
import sys
import threading
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "grouped-GEMM TFLOP/s (% MFMA peak) + gather-reduce GB/s, Mixtral shape, 1 GPU"
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published (at the 2400 MHz peak engine clock)
PEAK_FP8_TFLOPS = 5000.0
PEAK_HBM_GBS = 8000.0
PEAK_SCLK_MHZ = 2400.0
# HBM bytes per grouped-GEMM launch on C3 (mean of layer0 and layer1): FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000
# from the two rocprofv3 --pmc runs summarised in profiles/bench_c3_pmc_counters.md (scale factors from the
# 1 GiB copy of --calib-copy).  Only valid for the C3 workload with the fp32 layer1 intermediate.
GEMM_TRAFFIC_C3_BYTES = 4.47e9


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400, help="timed steps (400 steps of C3 = 1.2 s)")
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="C3", choices=["C1", "C3", "C4"])
    ap.add_argument("--inter", default="fp32", choices=["fp32", "bf16"],
                    help="dtype of the layer1 intermediate [M, H]")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-aux", action="store_true", help="skip the measurements outside the step")
    ap.add_argument("--sustain-s", type=float, default=2.5,
                    help="seconds of the sustained GEMM loop during which the shader clock is sampled (0 = skip)")
    ap.add_argument("--no-calib", action="store_true",
                    help="skip the plain streaming kernels of known traffic (what this box gives a copy / a read "
                         "stream; also the calibration of the rocprofv3 byte counters)")
    return ap.parse_args()


class Events:
    """HIP events (torch.cuda.Event on the stream the kernels are launched on) around named spans."""

    def __init__(self, torch):
        self.torch = torch
        self.spans = {}

    def span(self, name, fn):
        e0 = self.torch.cuda.Event(enable_timing=True)
        e1 = self.torch.cuda.Event(enable_timing=True)
        e0.record()
        out = fn()
        e1.record()
        self.spans.setdefault(name, []).append((e0, e1))
        return out

    def times_ms(self, name):
        return [a.elapsed_time(b) for a, b in self.spans[name]]

    def stats(self, name):
        v = self.times_ms(name)
        return {"mean": sum(v) / len(v), "median": statistics.median(v), "min": min(v)}


def time_loop(torch, fn, iters, warm=5, reps=3):
    """Mean time of one call in ms: the median over `reps` back-to-back loops of `iters` calls.  The first loop after
    a change of kernel runs while the board settles to the new kernel's power draw and can read 10-20 % off."""
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    means = []
    for _ in range(reps):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        means.append(e0.elapsed_time(e1) / iters)
    return statistics.median(means)


class ClockSampler(threading.Thread):
    """Reads the current shader clock (the starred line of pp_dpm_sclk) every 50 ms while a loop runs."""

    PATHS = ["/sys/class/drm/card0/device/pp_dpm_sclk", "/sys/class/drm/card1/device/pp_dpm_sclk"]

    def __init__(self):
        super().__init__(daemon=True)
        self.samples = []
        self.stop_flag = threading.Event()
        self.path = next((p for p in self.PATHS if os.path.exists(p)), None)

    def read_once(self):
        if self.path is None:
            return None
        try:
            for line in open(self.path).read().splitlines():
                if line.rstrip().endswith("*"):
                    return float(line.split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
        except (OSError, ValueError, IndexError):
            return None
        return None

    def run(self):
        while not self.stop_flag.is_set():
            v = self.read_once()
            if v is not None:
                self.samples.append(v)
            time.sleep(0.05)


def smi_snapshot():
    """Per-XCD clocks and socket power from one amd-smi call (made while the sustained loop keeps the GPU busy)."""
    try:
        out = subprocess.run(["amd-smi", "metric", "-g", "0", "--clock", "--power", "--json"], capture_output=True,
                             text=True, timeout=20).stdout
        data = json.loads(out)
        g = (data.get("gpu_data") or data)[0] if isinstance(data, dict) else data[0]
        clocks = [v["clk"]["value"] for k, v in g.get("clock", {}).items() if k.startswith("gfx_") and
                  isinstance(v.get("clk"), dict) and isinstance(v["clk"].get("value"), (int, float))]
        power = g.get("power", {}).get("socket_power", {}).get("value")
        return {"xcd_clk_mhz": clocks, "socket_power_w": power}
    except Exception as exc:  # noqa: BLE001 - the snapshot is optional evidence
        return {"error": str(exc)[:120]}


def sustained_gemm(torch, fn, seconds, flops_per_call):
    """Runs fn (the two GEMMs of the step) back to back for `seconds`, sampling the shader clock; returns the
    sustained rate and the clock figures."""
    sampler = ClockSampler()
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    sampler.start()
    calls = 0
    snap = None
    t0 = time.perf_counter()
    while True:
        for _ in range(20):
            fn()
        calls += 20
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        if snap is None and dt >= seconds / 2:
            # queue more work first so that the GPU stays busy while amd-smi runs
            for _ in range(200):
                fn()
            calls += 200
            snap = smi_snapshot()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
        if dt >= seconds:
            break
    sampler.stop_flag.set()
    sampler.join(timeout=1)
    s = sampler.samples[2:] if len(sampler.samples) > 4 else sampler.samples
    out = {"seconds": round(dt, 2), "tflops": round(flops_per_call * calls / dt * 1e-12, 1), "sclk_samples": len(s)}
    if s:
        out["sclk_mhz"] = round(sum(s) / len(s), 1)
        out["sclk_mhz_min_max"] = [min(s), max(s)]
    if snap:
        out.update(snap)
    return out


def cpu_baseline(torch, wl_name, x, w1, w2, passes=3):
    """The CPU oracle (PyTorch-CPU restatement of the reference's torch layer) on a bounded sample:
    one warm-up pass and `passes` timed passes over the first `sample_tokens` tokens of the same workload (all of
    C3), full hidden / ffn sizes; the median pass is reported."""
    from oracle import configs, layers

    sample_tokens = {"C1": 256, "C3": 8192, "C4": 8192}[wl_name]
    wl, _ = configs.make_routing(wl_name, tokens=sample_tokens)
    threads = torch.get_num_threads()
    xs = x[:sample_tokens].cpu()
    w1c, w2c = w1.cpu(), w2.cpu()

    def one_pass():
        t0 = time.perf_counter()
        y = layers.layer0_fp32(xs, w1c, wl.splits, wl.gather_index).to(torch.bfloat16)
        out = layers.layer1_fp32(y, w2c, wl.splits, wl.scatter_index.reshape(-1), wl.topk,
                                 output_vec_scale=wl.row_weight)
        dt = time.perf_counter() - t0
        assert out.shape == (sample_tokens, wl.hidden)
        return dt

    one_pass()                                   # warm-up: thread pool, page faults of the temporaries
    times = [one_pass() for _ in range(passes)]  # timed passes
    dt = statistics.median(times)
    flops = 2.0 * wl.rows * wl.hidden * wl.ffn * 2
    return {"value": round(flops / dt * 1e-12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"first {sample_tokens} tokens of {wl_name} (M={wl.rows} rows, full H/F), layer0+layer1, "
                      f"fp32 matmul on bf16-valued inputs; 1 warm-up + {passes} timed passes, median {dt:.2f} s "
                      f"(min {min(times):.2f}, max {max(times):.2f})"}


def gemm_entry(t_ms, flops, peak=PEAK_BF16_TFLOPS, key="frac_bf16_peak"):
    return {"ms": round(t_ms, 4), "tflops": round(flops / t_ms * 1e-9, 1), key: round(flops / t_ms * 1e-9 / peak, 4)}


def hbm_entry(t_ms, nbytes):
    return {"ms": round(t_ms, 4), "gbs": round(nbytes / t_ms * 1e-6, 1),
            "frac_hbm": round(nbytes / t_ms * 1e-6 / PEAK_HBM_GBS, 4)}


def aux_measurements(torch, capi, configs, a, wl, dev, gen, tensors):
    """Kernels and shapes of the path that the C3 step does not exercise in this form."""
    x, w1, w2, y, out, row_w = tensors
    t, k, e, h, f, m = wl.tokens, wl.topk, wl.experts, wl.hidden, wl.ffn, wl.rows
    gemm_flops = 2.0 * m * h * f
    kernels = {}
    sp = torch.from_numpy(wl.splits).to(dev)
    sc = torch.from_numpy(wl.scatter_index.reshape(-1)).to(dev)
    tok = torch.from_numpy(wl.gather_index).to(dev)

    # -- layer1 of the workload, both forms of the reduction (the step uses the two-pass form) --
    z32 = torch.empty(m, h, dtype=torch.float32, device=dev)
    t_two = time_loop(torch, lambda: (capi.grouped_gemm(y, w2, sp, out=z32, row_scale=row_w),
                                      capi.topk_gather_reduce(z32, sc, k, out=out)), 20)
    ws = torch.empty(t * h * 4, dtype=torch.uint8, device=dev)
    t_fused = time_loop(torch, lambda: capi.grouped_gemm_topk_reduce(y, w2, sp, tok, t, out=out, workspace=ws,
                                                                     row_scale=row_w), 20)
    # the same layer with the reference's own data flow: a bf16 intermediate (each top-k term rounded before the sum;
    # the op's inter_dtype option, tolerance 2e-2 as in the reference's test of that flow)
    zb16 = torch.empty(m, h, dtype=torch.bfloat16, device=dev)
    t_two16 = time_loop(torch, lambda: (capi.grouped_gemm(y, w2, sp, out=zb16, row_scale=row_w),
                                        capi.topk_gather_reduce(zb16, sc, k, out=out)), 20)
    kernels["layer1_gemm_then_gather_reduce_bf16_intermediate"] = gemm_entry(t_two16, gemm_flops)
    del zb16
    kernels["layer1_gemm_then_gather_reduce"] = gemm_entry(t_two, gemm_flops)
    kernels["layer1_reduce_fused_in_epilogue"] = gemm_entry(t_fused, gemm_flops)
    del z32, ws

    # -- the same two GEMMs with uniform splits (rows / experts each): what the ragged routing of the workload costs --
    if m % e == 0:
        spu = torch.full((e,), m // e, dtype=torch.int32, device=dev)
        giu = torch.from_numpy(wl.gather_index).to(dev)
        z32 = torch.empty(m, h, dtype=torch.float32, device=dev)
        kernels["gemm_layer0_uniform_splits"] = gemm_entry(time_loop(torch, lambda: capi.grouped_gemm(x, w1, spu, out=y, gather_a=giu), 20), gemm_flops)
        kernels["gemm_layer1_uniform_splits"] = gemm_entry(time_loop(torch, lambda: capi.grouped_gemm(y, w2, spu, out=z32, row_scale=row_w), 20), gemm_flops)
        kernels["gemm_layer0_workload_splits"] = gemm_entry(time_loop(torch, lambda: capi.grouped_gemm(x, w1, sp, out=y, gather_a=giu), 20), gemm_flops)
        kernels["gemm_layer1_workload_splits"] = gemm_entry(time_loop(torch, lambda: capi.grouped_gemm(y, w2, sp, out=z32, row_scale=row_w), 20), gemm_flops)
        # the two forms of the MFMA kernel's ring fills, forced, on the workload's splits (the default rule runs layer0,
        # whose rows are gathered, with half lines and layer1, K = 28 KiB per row, with whole lines)
        for form, flag in (("half_line_fills", capi.SCHED_HALF_LINE_FILLS), ("whole_line_fills", capi.SCHED_WHOLE_LINE_FILLS)):
            kernels[f"gemm_layer0_{form}"] = gemm_entry(time_loop(torch, lambda: capi.grouped_gemm(x, w1, sp, out=y, gather_a=giu, sched_flags=flag), 20), gemm_flops)
            kernels[f"gemm_layer1_{form}"] = gemm_entry(time_loop(torch, lambda: capi.grouped_gemm(y, w2, sp, out=z32, row_scale=row_w, sched_flags=flag), 20), gemm_flops)
        del z32, spu

    # -- stand-alone HBM kernels --
    zb = torch.randn(m, h, generator=gen, device=dev).to(torch.bfloat16)
    t_gr = time_loop(torch, lambda: capi.topk_gather_reduce(zb, sc, k, row_w, out=out), 50)
    kernels["gather_reduce_bf16_weighted"] = hbm_entry(t_gr, m * h * 2 + m * 4 + m * 4 + t * h * 2)
    del zb
    # The reduce at the C4 and C5 shapes (top-6 of 16384 tokens x 2048, top-8 of 4096 tokens x 7168) with those
    # workloads' own routing (stable scatter index, per-row top-k weights), bf16 rows.
    for tag in ("C4", "C5"):
        wl2, _ = configs.make_routing(tag)
        t2, k2, n2, m2 = wl2.tokens, wl2.topk, wl2.hidden, wl2.rows
        z2 = torch.randn(m2, n2, generator=gen, device=dev).to(torch.bfloat16)
        idx2 = torch.from_numpy(wl2.scatter_index.reshape(-1)).to(dev)
        w2r = wl2.row_weight.to(dev)
        o2 = torch.empty(t2, n2, dtype=torch.bfloat16, device=dev)
        t_g2 = time_loop(torch, lambda: capi.topk_gather_reduce(z2, idx2, k2, w2r, out=o2), 30)
        kernels[f"gather_reduce_bf16_weighted_{tag.lower()}"] = hbm_entry(t_g2, m2 * n2 * 2 + m2 * 8 + t2 * n2 * 2)
        ch2 = wl2.choosed.to(dev)
        t_rs = time_loop(torch, lambda: capi.route_sort(ch2, wl2.experts), 50)
        kernels[f"route_sort_{tag.lower()}"] = {"ms": round(t_rs, 4), "pairs": m2, "experts": wl2.experts}
        del z2, idx2, w2r, o2
    for rows, cols in ((4096, 7168), (32768, 2048)):
        xq = torch.randn(rows, cols, generator=gen, device=dev).to(torch.bfloat16)
        qo = capi.quant_e4m3(xq)     # output tensors allocated once: the loop times the kernel, not the allocator
        t_q = time_loop(torch, lambda: capi.quant_e4m3(xq, out=qo), 50)
        kernels[f"quant_e4m3_{rows}x{cols}"] = hbm_entry(t_q, rows * cols * 3 + rows * 4)
        del xq, qo

    # -- bf16 grouped GEMM at the other BASELINE shapes --
    # C2: one expert, a plain 4096 x 12288 x 6144 GEMM; the library's kernel (torch.mm = hipBLASLt) beside it.
    m2_, k2_, n2_ = 4096, 6144, 12288
    a2 = torch.randn(m2_, k2_, generator=gen, device=dev).to(torch.bfloat16)
    b2 = (torch.randn(1, n2_, k2_, generator=gen, device=dev) * 0.02).to(torch.bfloat16)
    d2 = torch.empty(m2_, n2_, dtype=torch.bfloat16, device=dev)
    sp2 = torch.tensor([m2_], dtype=torch.int32, device=dev)
    f2 = 2.0 * m2_ * k2_ * n2_
    t_c2 = time_loop(torch, lambda: capi.grouped_gemm(a2, b2, sp2, out=d2), 50)
    t_lib = time_loop(torch, lambda: torch.mm(a2, b2[0].t(), out=d2), 50)
    kernels["gemm_bf16_c2"] = gemm_entry(t_c2, f2)
    kernels["gemm_bf16_c2"]["library_gemm_ms"] = round(t_lib, 4)
    kernels["gemm_bf16_c2"]["library_gemm_tflops"] = round(f2 / t_lib * 1e-9, 1)
    del a2, b2, d2
    # C4: 64 experts, Zipf routing (its own splits and gather index), K = 2048 / 1408.
    wl4, _ = configs.make_routing("C4")
    t4, k4, e4, h4, f4, m4 = wl4.tokens, wl4.topk, wl4.experts, wl4.hidden, wl4.ffn, wl4.rows
    x4 = torch.randn(t4, h4, generator=gen, device=dev).to(torch.bfloat16)
    w14 = (torch.randn(e4, f4, h4, generator=gen, device=dev) * 0.02).to(torch.bfloat16)
    w24 = (torch.randn(e4, h4, f4, generator=gen, device=dev) * 0.02).to(torch.bfloat16)
    y4 = torch.empty(m4, f4, dtype=torch.bfloat16, device=dev)
    z4 = torch.empty(m4, h4, dtype=torch.float32, device=dev)
    sp4 = torch.from_numpy(wl4.splits).to(dev)
    gi4 = torch.from_numpy(wl4.gather_index).to(dev)
    rw4 = wl4.row_weight.to(dev)
    f4l = 2.0 * m4 * h4 * f4
    kernels["gemm_bf16_c4_layer0"] = gemm_entry(time_loop(torch, lambda: capi.grouped_gemm(x4, w14, sp4, out=y4, gather_a=gi4), 30), f4l)
    kernels["gemm_bf16_c4_layer1"] = gemm_entry(time_loop(torch, lambda: capi.grouped_gemm(y4, w24, sp4, out=z4, row_scale=rw4), 30), f4l)
    z4b = torch.empty(m4, h4, dtype=torch.bfloat16, device=dev)
    kernels["gemm_bf16_c4_layer1_bf16_intermediate"] = gemm_entry(time_loop(torch, lambda: capi.grouped_gemm(y4, w24, sp4, out=z4b, row_scale=rw4), 30), f4l)
    del z4b
    kernels["gemm_bf16_c4_layer0"]["rows_per_expert_min_max"] = [int(wl4.splits.min()), int(wl4.splits.max())]
    del x4, w14, w24, y4, z4

    # -- fp8 grouped GEMM at the C5 shape (one GPU's expert share: E=32, M=32768) --
    e5, m5 = 32, 32768
    sp5 = torch.full((e5,), m5 // e5, dtype=torch.int32, device=dev)
    rs5 = torch.rand(m5, generator=gen, device=dev)
    for tag, k5, n5 in (("layer1", 2048, 7168), ("layer0", 7168, 2048)):
        a8 = torch.randn(m5, k5, generator=gen, device=dev).to(torch.float8_e4m3fn)
        b8 = torch.randn(e5, n5, k5, generator=gen, device=dev).to(torch.float8_e4m3fn)
        cs5 = torch.rand(e5, n5, generator=gen, device=dev)
        d5 = torch.empty(m5, n5, dtype=torch.bfloat16, device=dev)
        f5 = 2.0 * m5 * k5 * n5
        # per-row x per-output-channel scales (and the top-8 weight folded into the row scale) in the epilogue
        t_f8 = time_loop(torch, lambda: capi.grouped_gemm(a8, b8, sp5, out=d5, row_scale=rs5, col_scale=cs5), 20)
        kernels[f"gemm_fp8_c5_{tag}"] = gemm_entry(t_f8, f5, PEAK_FP8_TFLOPS, "frac_fp8_peak")
        # the same launch with whole-line ring fills forced (not the default at these K: uniform splits like these gain,
        # ragged ones lose)
        t_f8w = time_loop(torch, lambda: capi.grouped_gemm(a8, b8, sp5, out=d5, row_scale=rs5, col_scale=cs5,
                                                           sched_flags=capi.SCHED_WHOLE_LINE_FILLS), 20)
        kernels[f"gemm_fp8_c5_{tag}_whole_line_fills"] = gemm_entry(t_f8w, f5, PEAK_FP8_TFLOPS, "frac_fp8_peak")
        # 1 x 128 activation scales x 128 x 128 weight scales, promoted every 128 of K
        sa = torch.rand(m5 // 128, k5 // 128, 128, generator=gen, device=dev) + 0.5
        sb = torch.rand(e5, n5 // 128, k5 // 128, generator=gen, device=dev) + 0.5
        t_bs = time_loop(torch, lambda: capi.grouped_gemm_blockscale(a8, b8, sp5, sa, sb, out=d5), 20)
        kernels[f"gemm_fp8_blockscale_c5_{tag}"] = gemm_entry(t_bs, f5, PEAK_FP8_TFLOPS, "frac_fp8_peak")
        # This kernel on the dense problem the library's kernel is timed on below: one weight matrix for all rows
        # (E = 1, 1/32 of the weight bytes, so the weights stay cache-resident), the like-for-like comparison.
        sp1 = torch.tensor([m5], dtype=torch.int32, device=dev)
        t_d1 = time_loop(torch, lambda: capi.grouped_gemm(a8, b8[:1], sp1, out=d5, row_scale=rs5, col_scale=cs5[:1]), 20)
        kernels[f"gemm_fp8_dense_one_weight_c5_{tag}"] = gemm_entry(t_d1, f5, PEAK_FP8_TFLOPS, "frac_fp8_peak")
        # The library's fp8 GEMM (torch._scaled_mm = hipBLASLt) for scale: the same work as a loop of per-expert
        # GEMMs, and one dense GEMM of the same FLOPs with a single weight matrix (1/32 of the weight bytes).
        try:
            one = torch.ones((), device=dev)
            rows5 = m5 // e5

            def lib8_loop():
                for ei in range(e5):
                    torch._scaled_mm(a8[ei * rows5:(ei + 1) * rows5], b8[ei].t(), scale_a=one, scale_b=one,
                                     out_dtype=torch.bfloat16, out=d5[ei * rows5:(ei + 1) * rows5])

            kernels[f"library_fp8_gemm_loop_c5_{tag}"] = gemm_entry(time_loop(torch, lib8_loop, 10), f5, PEAK_FP8_TFLOPS, "frac_fp8_peak")
            t_dense = time_loop(torch, lambda: torch._scaled_mm(a8, b8[0].t(), scale_a=one, scale_b=one,
                                                                 out_dtype=torch.bfloat16, out=d5), 20)
            kernels[f"library_fp8_gemm_dense_one_weight_c5_{tag}"] = gemm_entry(t_dense, f5, PEAK_FP8_TFLOPS, "frac_fp8_peak")
        except Exception as ex:  # the library may not offer this dtype / layout
            kernels[f"library_fp8_gemm_loop_c5_{tag}"] = {"error": repr(ex)[:120]}
        del a8, b8, d5, cs5, sa, sb

    # -- the same two C3 GEMMs as a loop of library GEMMs (torch.mm = hipBLASLt), one per expert, on rows that
    # are already gathered and contiguous: the path a port without a grouped kernel would take --
    xg = torch.randn(m, h, generator=gen, device=dev).to(torch.bfloat16)
    bounds = [0] + [int(v) for v in wl.splits.cumsum()]

    def lib_loop(src, wts, dst):
        for ei in range(e):
            r0, r1 = bounds[ei], bounds[ei + 1]
            if r1 > r0:
                torch.mm(src[r0:r1], wts[ei].t(), out=dst[r0:r1])

    zl = torch.empty(m, h, dtype=torch.bfloat16, device=dev)
    for name, fn in (("library_gemm_loop_layer0", lambda: lib_loop(xg, w1, y)),
                     ("library_gemm_loop_layer1", lambda: lib_loop(y, w2, zl))):
        t_l = time_loop(torch, fn, 20)
        kernels[name] = {"ms": round(t_l, 4), "tflops": round(gemm_flops / t_l * 1e-9, 1)}
    del xg, zl
    return kernels


def main():
    a = parse()
    if a.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {a.gpus}): this build has no multi-GPU path",
              file=sys.stderr)
        sys.exit(2)
    import torch

    from flux_amd import capi
    from oracle import configs

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    capi.load()

    wl, _ = configs.make_routing(a.workload)
    t, k, e, h, f, m = wl.tokens, wl.topk, wl.experts, wl.hidden, wl.ffn, wl.rows
    gen = torch.Generator(device=dev).manual_seed(1000)
    x = torch.randn(t, h, generator=gen, device=dev).to(torch.bfloat16)
    w1 = (torch.randn(e, f, h, generator=gen, device=dev) * 0.02).to(torch.bfloat16)
    w2 = (torch.randn(e, h, f, generator=gen, device=dev) * 0.02).to(torch.bfloat16)
    choosed = wl.choosed.to(dev)
    row_w = wl.row_weight.to(dev)
    inter_dtype = torch.float32 if a.inter == "fp32" else torch.bfloat16
    y = torch.empty(m, f, dtype=torch.bfloat16, device=dev)
    z = torch.empty(m, h, dtype=inter_dtype, device=dev)
    out = torch.empty(t, h, dtype=torch.bfloat16, device=dev)

    ev = Events(torch)

    def step(rec):
        span = rec.span if rec else (lambda _n, fn: fn())
        splits, _off, scatter, gather, _tki = span("route_sort", lambda: capi.route_sort(choosed, e))
        span("gemm_layer0", lambda: capi.grouped_gemm(x, w1, splits, out=y, gather_a=gather))
        span("gemm_layer1", lambda: capi.grouped_gemm(y, w2, splits, out=z, row_scale=row_w))
        span("gather_reduce", lambda: capi.topk_gather_reduce(z, scatter.reshape(-1), k, out=out))

    for _ in range(a.warmup):
        step(None)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        step(ev)
    torch.cuda.synchronize()
    timed_s = time.perf_counter() - t0
    ms_per_step = timed_s * 1e3 / a.steps

    gemm_flops = 2.0 * m * h * f                      # per layer, actual routed rows only
    step_flops = 2 * gemm_flops
    st = {n: ev.stats(n) for n in ("route_sort", "gemm_layer0", "gemm_layer1", "gather_reduce")}
    both = [0.5 * (p + q) for p, q in zip(ev.times_ms("gemm_layer0"), ev.times_ms("gemm_layer1"))]
    gemm_ms = sum(both) / len(both)                   # average launch duration of the grouped GEMM kernel
    gemm_med, gemm_min = statistics.median(both), min(both)
    achieved = gemm_flops / gemm_ms * 1e-9            # TFLOP/s
    inter_b = 4 if a.inter == "fp32" else 2
    gr_bytes = m * h * inter_b + m * 4 + t * h * 2
    route_bytes = m * 4 * 2 + e * 4 + 3 * m * 4       # pairs read twice, three index arrays written

    def gstat(name):
        s = st[name]
        return {"ms": round(s["mean"], 4), "ms_median": round(s["median"], 4), "ms_min": round(s["min"], 4),
                "tflops": round(gemm_flops / s["mean"] * 1e-9, 1)}

    kernels = {
        "gemm_layer0": gstat("gemm_layer0"),
        "gemm_layer1": gstat("gemm_layer1"),
        "gather_reduce": dict(hbm_entry(st["gather_reduce"]["mean"], gr_bytes),
                              ms_median=round(st["gather_reduce"]["median"], 4), input=a.inter),
        "route_sort": {"ms": round(st["route_sort"]["mean"], 4), "ms_median": round(st["route_sort"]["median"], 4),
                       "ms_min": round(st["route_sort"]["min"], 4),
                       "gbs": round(route_bytes / st["route_sort"]["mean"] * 1e-6, 1)},
    }

    roofline = {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                "traffic": GEMM_TRAFFIC_C3_BYTES if (a.workload == "C3" and a.inter == "fp32") else None,
                "kernel": "grouped_gemm_mfma_kernel<bf16>", "flop_per_launch": gemm_flops,
                "avg_launch_ms": round(gemm_ms, 4), "median_launch_ms": round(gemm_med, 4),
                "min_launch_ms": round(gemm_min, 4),
                "frac_at_median": round(gemm_flops / gemm_med * 1e-9 / PEAK_BF16_TFLOPS, 4)}

    if a.sustain_s > 0:
        # The shader clock under this kernel's own load: the board holds its power limit by lowering the clock, so
        # the published peak (at 2400 MHz) is not what the MFMA pipes can deliver while the kernel runs.
        splits_d = torch.from_numpy(wl.splits).to(dev)
        gather_d = torch.from_numpy(wl.gather_index).to(dev)
        sus = sustained_gemm(torch, lambda: (capi.grouped_gemm(x, w1, splits_d, out=y, gather_a=gather_d),
                                             capi.grouped_gemm(y, w2, splits_d, out=z, row_scale=row_w)),
                             a.sustain_s, step_flops)
        roofline["sustained"] = sus
        if "sclk_mhz" in sus:
            roofline["sclk_mhz"] = sus["sclk_mhz"]
            adj = PEAK_BF16_TFLOPS * sus["sclk_mhz"] / PEAK_SCLK_MHZ
            roofline["peak_clock_adjusted"] = round(adj, 1)
            roofline["frac_of_clock_adjusted_peak"] = round(sus["tflops"] / adj, 4)
        # The same two launches on zero-valued operands of the same shapes (same instruction stream, same tile
        # schedule): without the data's switching activity the board stays under its power limit and the clock is
        # not lowered, which separates what the kernel's schedule costs from what the power limit costs.  Not a
        # throughput figure of the workload.
        xz, w1z, w2z = torch.zeros_like(x), torch.zeros_like(w1), torch.zeros_like(w2)
        yz, zz = torch.zeros_like(y), torch.empty_like(z)
        zs = sustained_gemm(torch, lambda: (capi.grouped_gemm(xz, w1z, splits_d, out=yz, gather_a=gather_d),
                                            capi.grouped_gemm(yz, w2z, splits_d, out=zz, row_scale=row_w)),
                            min(a.sustain_s, 1.5), step_flops)
        zs["frac_of_peak"] = round(zs["tflops"] / PEAK_BF16_TFLOPS, 4)
        roofline["zero_operands_same_launches"] = zs
        del xz, w1z, w2z, yz, zz

    if not a.no_aux:
        kernels.update(aux_measurements(torch, capi, configs, a, wl, dev, gen, (x, w1, w2, y, out, row_w)))

    if not a.no_calib:
        # What this box gives kernels that only stream (fluxmi_calib_stream: 16 bytes per lane and load, eight loads in
        # flight, non-temporal): a 1 GiB copy (also the known traffic that scales the profiler's byte counters), and,
        # for the byte counts the C4 / C5 reductions and the quantisation shapes move, a copy and a pure read stream.
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        t_cp = time_loop(torch, lambda: capi.calib_stream(src, dst, 1 << 30, copy=True), 5, warm=1)
        kernels["calib_copy_1GiB"] = dict(hbm_entry(t_cp, 2 * (1 << 30)), kernel="plain copy, 1 GiB read + 1 GiB written")
        t_tc = time_loop(torch, lambda: dst.copy_(src), 5, warm=1)
        kernels["calib_copy_1GiB_library"] = dict(hbm_entry(t_tc, 2 * (1 << 30)), kernel="torch copy_")
        for tag, nbytes in (("reduce_c4", 470.6e6), ("reduce_c5", 528.7e6), ("quant_4096x7168", 88.1e6)):
            nb = int(nbytes) // 32 * 32
            t_c = time_loop(torch, lambda: capi.calib_stream(src, dst, nb // 2, copy=True), 20, warm=2)
            kernels[f"calib_copy_bytes_of_{tag}"] = dict(hbm_entry(t_c, nb), kernel="plain copy, half read, half written")
            t_r = time_loop(torch, lambda: capi.calib_stream(src, dst, nb, copy=False), 20, warm=2)
            kernels[f"calib_read_bytes_of_{tag}"] = dict(hbm_entry(t_r, nb), kernel="plain read stream")
        del src, dst

    result = {
        "metric": METRIC,
        "value": round(step_flops / ms_per_step * 1e-9, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"{a.workload}: tokens={t} topk={k} experts={e} hidden={h} ffn={f} rows={m}; "
                               f"step = route sort + layer0 gather-GEMM + layer1 GEMM + top-k gather-reduce",
                   "layer1_intermediate": a.inter,
                   "rows_per_expert_min_max": [int(wl.splits.min()), int(wl.splits.max())],
                   "timed_region_s": round(timed_s, 3)},
        "roofline": roofline,
        "kernels": kernels,
    }
    if not a.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(torch, a.workload, x, w1, w2)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
