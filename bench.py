"""Benchmark of the MoE hot path on one MI355X.

A step = one pass of the path over one batch: routing sort -> layer0 (row gather fused into the grouped
GEMM) -> layer1 grouped GEMM (top-k weight in the epilogue) -> top-k gather-reduce to token order.
Workload at N=1: C3, the Mixtral-shape layer the metric is quoted on (T=8192, H=4096, F=14336, E=8,
top-2, bf16), synthetic data, inputs resident in HBM before the timed region.

Prints ONE JSON line: whole-step throughput in TFLOP/s (algorithmic GEMM FLOPs of the step / step
time), the roofline object of the dominant kernel (grouped GEMM, MFMA-bound) measured with HIP events
inside the timed region, per-kernel figures, and the CPU oracle timed on a bounded sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "grouped-GEMM TFLOP/s (% MFMA peak) + gather-reduce GB/s, Mixtral shape, 1 GPU"
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA, published
PEAK_FP8_TFLOPS = 5000.0
PEAK_HBM_GBS = 8000.0
# HBM bytes per grouped-GEMM launch on C3 (mean of layer0 and layer1): FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000
# from the two rocprofv3 --pmc runs summarised in profiles/bench_c3_pmc_counters.md (scale factors from the
# 1 GiB copy of --calib-copy).  Only valid for the C3 workload with the fp32 layer1 intermediate.
GEMM_TRAFFIC_C3_BYTES = 4.970e9


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="C3", choices=["C1", "C3", "C4"])
    ap.add_argument("--inter", default="fp32", choices=["fp32", "bf16"],
                    help="dtype of the layer1 intermediate [M, H]")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-aux", action="store_true", help="skip the stand-alone HBM kernel measurements")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (known traffic) to calibrate rocprofv3 byte counters")
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

    def mean_ms(self, name):
        v = [a.elapsed_time(b) for a, b in self.spans[name]]
        return sum(v) / len(v)


def time_loop(torch, fn, iters, warm=3):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def cpu_baseline(torch, wl_name, x, w1, w2):
    """The CPU oracle (PyTorch-CPU restatement of the reference's torch layer) on a bounded sample:
    one pass over the first `sample_tokens` tokens of the same workload (all of C3), full hidden / ffn sizes."""
    from oracle import configs, layers

    sample_tokens = {"C1": 256, "C3": 8192, "C4": 8192}[wl_name]
    wl, _ = configs.make_routing(wl_name, tokens=sample_tokens)
    threads = torch.get_num_threads()
    xs = x[:sample_tokens].cpu()
    w1c, w2c = w1.cpu(), w2.cpu()
    t0 = time.perf_counter()
    y = layers.layer0_fp32(xs, w1c, wl.splits, wl.gather_index).to(torch.bfloat16)
    out = layers.layer1_fp32(y, w2c, wl.splits, wl.scatter_index.reshape(-1), wl.topk,
                             output_vec_scale=wl.row_weight)
    dt = time.perf_counter() - t0
    flops = 2.0 * wl.rows * wl.hidden * wl.ffn * 2
    assert out.shape == (sample_tokens, wl.hidden)
    return {"value": round(flops / dt * 1e-12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"first {sample_tokens} tokens of {wl_name} (M={wl.rows} rows, full H/F), layer0+layer1, "
                      f"fp32 matmul on bf16-valued inputs, {dt:.2f} s wall"}


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
    ms_per_step = (time.perf_counter() - t0) * 1e3 / a.steps

    gemm_flops = 2.0 * m * h * f                      # per layer, actual routed rows only
    step_flops = 2 * gemm_flops
    ms = {n: ev.mean_ms(n) for n in ("route_sort", "gemm_layer0", "gemm_layer1", "gather_reduce")}
    gemm_ms = 0.5 * (ms["gemm_layer0"] + ms["gemm_layer1"])
    achieved = gemm_flops / gemm_ms * 1e-9            # TFLOP/s
    inter_b = 4 if a.inter == "fp32" else 2
    gr_bytes = m * h * inter_b + m * 4 + t * h * 2
    route_bytes = m * 4 * 2 + e * 4 + 3 * m * 4       # pairs read twice, three index arrays written

    kernels = {
        "gemm_layer0": {"ms": round(ms["gemm_layer0"], 4), "tflops": round(gemm_flops / ms["gemm_layer0"] * 1e-9, 1)},
        "gemm_layer1": {"ms": round(ms["gemm_layer1"], 4), "tflops": round(gemm_flops / ms["gemm_layer1"] * 1e-9, 1)},
        "gather_reduce": {"ms": round(ms["gather_reduce"], 4), "gbs": round(gr_bytes / ms["gather_reduce"] * 1e-6, 1),
                          "frac_hbm": round(gr_bytes / ms["gather_reduce"] * 1e-6 / PEAK_HBM_GBS, 4),
                          "input": a.inter},
        "route_sort": {"ms": round(ms["route_sort"], 4), "gbs": round(route_bytes / ms["route_sort"] * 1e-6, 1)},
    }

    if not a.no_aux:
        # Stand-alone HBM kernels of the path that the step above does not exercise in this form.
        zb = torch.randn(m, h, generator=gen, device=dev).to(torch.bfloat16)
        sc = torch.from_numpy(wl.scatter_index.reshape(-1)).to(dev)
        t_gr = time_loop(torch, lambda: capi.topk_gather_reduce(zb, sc, k, row_w, out=out), 50)
        b_gr = m * h * 2 + m * 4 + m * 4 + t * h * 2
        kernels["gather_reduce_bf16_weighted"] = {"ms": round(t_gr, 4), "gbs": round(b_gr / t_gr * 1e-6, 1),
                                                  "frac_hbm": round(b_gr / t_gr * 1e-6 / PEAK_HBM_GBS, 4)}
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
            b_g2 = m2 * n2 * 2 + m2 * 8 + t2 * n2 * 2
            kernels[f"gather_reduce_bf16_weighted_{tag.lower()}"] = {
                "ms": round(t_g2, 4), "gbs": round(b_g2 / t_g2 * 1e-6, 1),
                "frac_hbm": round(b_g2 / t_g2 * 1e-6 / PEAK_HBM_GBS, 4)}
            del z2, idx2, w2r, o2
        for rows, cols in ((4096, 7168), (32768, 2048)):
            xq = torch.randn(rows, cols, generator=gen, device=dev).to(torch.bfloat16)
            qo = capi.quant_e4m3(xq)     # output tensors allocated once: the loop times the kernel, not the allocator
            t_q = time_loop(torch, lambda: capi.quant_e4m3(xq, out=qo), 50)
            b_q = rows * cols * 3 + rows * 4
            kernels[f"quant_e4m3_{rows}x{cols}"] = {"ms": round(t_q, 4), "gbs": round(b_q / t_q * 1e-6, 1),
                                                    "frac_hbm": round(b_q / t_q * 1e-6 / PEAK_HBM_GBS, 4)}
        del zb
        # fp8 grouped GEMM at the C5 shape (one GPU's expert share: E=32, M=32768, K=2048, N=7168), row x column
        # scales and top-8 weight in the epilogue.
        e5, m5, k5, n5 = 32, 32768, 2048, 7168
        a8 = torch.randn(m5, k5, generator=gen, device=dev).to(torch.float8_e4m3fn)
        b8 = (torch.randn(e5, n5, k5, generator=gen, device=dev)).to(torch.float8_e4m3fn)
        sp5 = torch.full((e5,), m5 // e5, dtype=torch.int32, device=dev)
        rs5 = torch.rand(m5, generator=gen, device=dev)
        cs5 = torch.rand(e5, n5, generator=gen, device=dev)
        d5 = torch.empty(m5, n5, dtype=torch.bfloat16, device=dev)
        t_f8 = time_loop(torch, lambda: capi.grouped_gemm(a8, b8, sp5, out=d5, row_scale=rs5, col_scale=cs5), 20)
        f_f8 = 2.0 * m5 * k5 * n5
        kernels["gemm_fp8_c5_layer1"] = {"ms": round(t_f8, 4), "tflops": round(f_f8 / t_f8 * 1e-9, 1),
                                         "frac_fp8_peak": round(f_f8 / t_f8 * 1e-9 / PEAK_FP8_TFLOPS, 4)}
        del a8, b8, d5
        # ... and layer0 of the same share: K = 7168, N = 2048 (per-row and per-column scales, no top-k weight)
        a8 = torch.randn(m5, n5, generator=gen, device=dev).to(torch.float8_e4m3fn)
        b8 = (torch.randn(e5, k5, n5, generator=gen, device=dev)).to(torch.float8_e4m3fn)
        cs0 = torch.rand(e5, k5, generator=gen, device=dev)
        d5 = torch.empty(m5, k5, dtype=torch.bfloat16, device=dev)
        t_f8 = time_loop(torch, lambda: capi.grouped_gemm(a8, b8, sp5, out=d5, row_scale=rs5, col_scale=cs0), 20)
        kernels["gemm_fp8_c5_layer0"] = {"ms": round(t_f8, 4), "tflops": round(f_f8 / t_f8 * 1e-9, 1),
                                         "frac_fp8_peak": round(f_f8 / t_f8 * 1e-9 / PEAK_FP8_TFLOPS, 4)}
        del a8, b8, d5, cs0
        # The same two C3 GEMMs as a loop of library GEMMs (torch.mm = hipBLASLt), one per expert, on rows that
        # are already gathered and contiguous: the path a port without a grouped kernel would take.  Reported
        # beside the grouped kernel for comparison; not part of the step.
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

    if a.calib_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        t_cp = time_loop(torch, lambda: dst.copy_(src), 5, warm=1)
        kernels["calib_copy_1GiB"] = {"ms": round(t_cp, 4), "gbs": round(2 * (1 << 30) / t_cp * 1e-6, 1)}
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
                   "rows_per_expert_min_max": [int(wl.splits.min()), int(wl.splits.max())]},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                     "traffic": GEMM_TRAFFIC_C3_BYTES if (a.workload == "C3" and a.inter == "fp32") else None,
                     "kernel": "grouped_gemm_mfma_kernel<bf16>", "flop_per_launch": gemm_flops,
                     "avg_launch_ms": round(gemm_ms, 4)},
        "kernels": kernels,
    }
    if not a.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(torch, a.workload, x, w1, w2)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
