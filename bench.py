#!/usr/bin/env python3
"""Benchmark of the quantized-inference operator path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-others] [--skip-cpu] [--eager]

A "step" is one npu_quant_matmul call on the headline configuration (W8A8, x int8
[1024, 4096], weight int8 logical [4096, 11008] stored [N, K] and passed as its transposed
view the way torch_npu's LinearQuant passes it, per-token x per-channel dequantisation, bf16
bias, bf16 output).  Inputs are resident in HBM before the timed region; the weight/activation
sets are rotated over more than the 256 MB Infinity Cache so that repeated steps do not run
out of cache.  One JSON line is printed; the remaining configurations (dynamic_quant, W8A16,
W4A16, the MLP chain) are reported under "others" with their own roofline figures.

The CPU oracle is used only to check the timed outputs and as the reported CPU baseline.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
INT8_PEAK_TOPS = 5000.0      # dense int8 MFMA
BF16_PEAK_TFLOPS = 2500.0    # dense bf16 MFMA
CACHE_BYTES = 256 << 20      # Infinity Cache
TRAFFIC_FILE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "hbm_traffic_pmc_all_kernels.txt")


def _load_traffic():
    """HBM bytes per launch, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (each scaled by what the same counter
    reads for a plain 256 MiB copy).  The figures live in the profile summary, one `TRAFFIC tag=... kernel=...
    hbm_bytes=...` line per kernel and workload; a tag without a line reports traffic null, so a kernel that was
    replaced after the profile was taken cannot inherit a stale figure (the line names the kernel it was measured on)."""
    table = {}
    try:
        with open(TRAFFIC_FILE) as f:
            for line in f:
                if not line.startswith("TRAFFIC "):
                    continue
                kv = dict(tok.split("=", 1) for tok in line.split()[1:] if "=" in tok)
                table[kv["tag"]] = {"hbm_bytes": int(kv["hbm_bytes"]), "kernel": kv.get("kernel", "")}
    except OSError:
        pass
    return table


TRAFFIC = _load_traffic()


def _traffic(tag):
    return TRAFFIC[tag]["hbm_bytes"] if tag in TRAFFIC else None


def _parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--skip-others", action="store_true")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--graph", action="store_true",
                    help="launch the timed headline steps from one captured HIP graph instead of one by one")
    ap.add_argument("--eager", action="store_true", help="accepted for compatibility: one-by-one launches are the default")
    ap.add_argument("--only", default="", help="comma-separated subset of: c1,c2kn,c2i8,c3,c4,qd,a4w4,c5,aq,qz for the 'others' section")
    ap.add_argument("--pmc-summarize", nargs=2, metavar=("FETCH_DIR", "WRITE_DIR"),
                    help="print the TRAFFIC lines from the output directories of the two rocprofv3 --pmc runs of --pmc-pass")
    ap.add_argument("--pmc-pass", action="store_true",
                    help="launch a 256 MiB device copy and then each main kernel once on fresh buffers (for "
                         "`rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` runs: the copy calibrates the counters)")
    return ap.parse_args()


def _bits(t):
    import numpy as np
    import torch
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _event_time_ms(torch, fn, iters):
    """Average GPU time of fn() over `iters` back-to-back calls, HIP events on the launch stream."""
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) / iters


def _graph_time_us(torch, calls, reps=20):
    """Capture the list of launches in one HIP graph (removes host launch gaps for microsecond-scale
    kernels), replay it `reps` times between two events and return the average time per launch in us."""
    # warm-up on the stream that will capture: one-time initialisation and the per-stream workspace must exist before
    # the capture, so that the graph holds nothing but the launches
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for c in calls:
            c()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=side):
        for c in calls:
            c()
    g.replay()
    torch.cuda.synchronize()
    # after an idle period the chip needs about 30 ms of continuous work to reach the clocks it then holds (the headline
    # launch: 45 us for the first twenty launches, 47-54 us for the next few hundred, 43.5-44.5 us from about the 700th on):
    # replay untimed for that long, so that every line is measured in the settled state
    w0 = time.perf_counter()
    while time.perf_counter() - w0 < 0.03:
        for _ in range(4):
            g.replay()
        torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(reps):
        g.replay()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) * 1e3 / (reps * len(calls))


def _nsets(bytes_per_set):
    return max(2, min(16, int(1.5 * CACHE_BYTES / max(bytes_per_set, 1)) + 1))


def _pmc_pass(torch, pa, workloads, dev):
    """One launch of every benchmarked kernel (or chain of kernels) on operands that no earlier kernel of this process
    touched, for `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` runs.  Every item is preceded by a 1 GiB fill that
    pushes earlier data out of the caches; an empty kernel whose workgroup count is 1000 + index opens the item and one
    with 999 workgroups closes it.  Item 0 is a plain device copy of known size that calibrates the two counters.
    `bench.py --pmc-summarize <dir of the FETCH_SIZE run> <dir of the WRITE_SIZE run>` turns the two counter files into
    the TRAFFIC lines of profiles/hbm_traffic_pmc_all_kernels.txt."""
    from pytorch_amd import _capi
    gen = torch.Generator(device=dev).manual_seed(7)
    ri8 = lambda *sh: torch.randint(-127, 128, sh, generator=gen, dtype=torch.int8, device=dev)  # noqa: E731
    ri32 = lambda *sh: torch.randint(-2 ** 31, 2 ** 31 - 1, sh, generator=gen, dtype=torch.int32, device=dev)  # noqa: E731
    up = lambda d: {k: (v.to(dev) if torch.is_tensor(v) else v) for k, v in d.items()}  # noqa: E731
    items = []

    # one-time set-up (per-stream workspaces, function attributes) on small shapes: no big traffic, no allocation later
    w0 = up(workloads.w4a16_inputs(seed=9, M=8, K=1024, N=512))
    pa.npu_weight_quant_batchmatmul(w0["x"], w0["weight"], w0["antiquant_scale"], w0["antiquant_offset"], None, None, None, 128)
    pa.npu_quant_matmul(ri8(64, 14336), ri8(256, 14336).t(), torch.rand(256, device=dev), output_dtype=torch.bfloat16)
    torch.cuda.synchronize()

    src = torch.empty(256 << 20, dtype=torch.int8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    items.append(("copy", lambda: dst.copy_(src)))
    d1 = workloads.dynamic_quant_input(seed=0).to(dev)
    items.append(("c1", lambda: pa.npu_dynamic_quant(d1)))
    g2 = up(workloads.quant_matmul_inputs(seed=0, weight_nk=True))
    items.append(("c2", lambda: pa.npu_quant_matmul(g2["x1"], g2["x2"], g2["scale"], pertoken_scale=g2["pertoken_scale"], bias=g2["bias"],
                                                    output_dtype=torch.bfloat16)))
    w2kn = ri8(4096, 11008)
    items.append(("c2_kn", lambda: pa.npu_quant_matmul(g2["x1"], w2kn, g2["scale"], pertoken_scale=g2["pertoken_scale"], bias=g2["bias"],
                                                       output_dtype=torch.bfloat16)))
    qp = pa.npu_trans_quant_param(torch.rand(11008, device=dev) * 1e-4 + 1e-4, torch.randint(-8, 8, (11008,), device=dev).float())
    bi = torch.randint(-1000, 1000, (11008,), device=dev, dtype=torch.int32)
    x2i8, w2i8 = ri8(1024, 4096), ri8(11008, 4096).t()
    items.append(("c2_i8", lambda: pa.npu_quant_matmul(x2i8, w2i8, qp, bias=bi, output_dtype=torch.int8)))
    xa4, wa4 = ri32(1024, 512), ri32(11008, 512).t()
    items.append(("a4w4", lambda: pa.npu_quant_matmul(xa4, wa4, g2["scale"], pertoken_scale=g2["pertoken_scale"], output_dtype=torch.bfloat16)))
    g3 = up(workloads.w8a16_inputs(seed=0))
    items.append(("c3", lambda: pa.npu_weight_quant_batchmatmul(g3["x"], g3["weight"], g3["antiquant_scale"], g3["antiquant_offset"])))
    w3nk = ri8(28672, 8192).t()
    items.append(("c3_nk", lambda: pa.npu_weight_quant_batchmatmul(g3["x"], w3nk, g3["antiquant_scale"], g3["antiquant_offset"])))
    for m_rows in (1, 8, 32, 128):
        g4 = up(workloads.w4a16_inputs(seed=m_rows, M=m_rows))
        items.append((f"c4_m{m_rows}", lambda g4=g4: pa.npu_weight_quant_batchmatmul(g4["x"], g4["weight"], g4["antiquant_scale"],
                                                                                      g4["antiquant_offset"], None, None, None, 128)))
        wk = ri32(14336, 512).t()
        s4t, o4t = g4["antiquant_scale"].t().contiguous().t(), g4["antiquant_offset"].t().contiguous().t()
        items.append((f"c4k_m{m_rows}", lambda g4=g4, wk=wk, s4t=s4t, o4t=o4t: pa.npu_weight_quant_batchmatmul(
            g4["x"], wk, s4t, o4t, None, None, None, 128)))
    xa, sa = torch.randint(-128, 128, (4096, 14336), dtype=torch.int8, device=dev), torch.rand(14336, device=dev) + 0.5
    items.append(("aq_int8", lambda: pa.npu_anti_quant(xa, sa, offset=sa, dst_dtype=torch.bfloat16)))
    for (Kx, Nx) in ((4096, 28672), (14336, 4096)):
        wq, xq = ri8(Nx, Kx).t(), ri8(16, Kx)
        sq, pq = torch.rand(Nx, device=dev), torch.rand(16, device=dev)
        items.append((f"qd_{Kx}x{Nx}_m16", lambda wq=wq, xq=xq, sq=sq, pq=pq: pa.npu_quant_matmul(xq, wq, sq, pertoken_scale=pq,
                                                                                                  output_dtype=torch.bfloat16)))
    H, I = 4096, 14336
    for Mx in (16, 64, 2048):
        x5 = torch.randn(Mx, H, device=dev).to(torch.bfloat16)
        wgu, wd = ri8(2 * I, H).t(), ri8(H, I).t()
        sgu, sd = torch.rand(2 * I, device=dev) * 1e-2, torch.rand(H, device=dev) * 1e-2

        def mlp(x5=x5, wgu=wgu, wd=wd, sgu=sgu, sd=sd):
            xq, xsc = pa.npu_dynamic_quant(x5)
            gu = pa.npu_quant_matmul(xq, wgu, sgu, pertoken_scale=xsc, output_dtype=torch.bfloat16)
            aq, asc = pa.npu_swiglu_quant(gu, activate_left=True, quant_mode=1)
            return pa.npu_quant_matmul(aq, wd, sd, pertoken_scale=asc, output_dtype=torch.bfloat16)
        items.append((f"c5_m{Mx}", mlp))

    flush = torch.empty(1 << 30, dtype=torch.int8, device=dev)
    keep = []
    for idx, (tag, fn) in enumerate(items):
        flush.fill_(idx & 127)
        torch.cuda.synchronize()
        _capi.empty_launch(1000 + idx)                 # opens item idx
        keep.append(fn())
        _capi.empty_launch(999)                        # closes it
        torch.cuda.synchronize()
    print(json.dumps({"pmc_pass": [t for t, _ in items]}))


_PMC_TAGS = ["copy", "c1", "c2", "c2_kn", "c2_i8", "a4w4", "c3", "c3_nk", "c4_m1", "c4k_m1", "c4_m8", "c4k_m8", "c4_m32", "c4k_m32",
             "c4_m128", "c4k_m128", "aq_int8", "qd_4096x28672_m16", "qd_14336x4096_m16", "c5_m16", "c5_m64", "c5_m2048"]


def _pmc_summarize(fetch_dir, write_dir):
    """Reads the counter files of the two `rocprofv3 --pmc` runs of `bench.py --pmc-pass` and prints, per item, the
    kernels it launched and its HBM bytes (FETCH_SIZE and WRITE_SIZE, each scaled by what it reads for the 256 MiB copy)."""
    import csv
    import glob
    import re

    def load(d, counter):
        files = glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)
        if not files:
            raise SystemExit(f"no *counter_collection.csv under {d}")
        rows = []
        for f in files:
            with open(f, newline="") as fh:
                for r in csv.DictReader(fh):
                    if r.get("Counter_Name") == counter:
                        rows.append((int(r["Dispatch_Id"]), r["Kernel_Name"], int(r["Grid_Size"]) // max(int(r["Workgroup_Size"]), 1),
                                     float(r["Counter_Value"])))
        rows.sort()
        segs, cur = {}, None
        for _, name, wgs, val in rows:
            if "empty_kernel" in name:
                cur = wgs - 1000 if wgs >= 1000 else None
                continue
            if cur is not None:
                segs.setdefault(cur, []).append((name, val))
        return segs

    fetch, write = load(fetch_dir, "FETCH_SIZE"), load(write_dir, "WRITE_SIZE")
    kib = 256 * 1024.0
    f_scale = kib / sum(v for _, v in fetch[0])
    w_scale = kib / sum(v for _, v in write[0])
    print(f"calibration (plain copy, 262,144 KiB read and written): FETCH_SIZE reads {sum(v for _, v in fetch[0]):,.0f} -> factor {f_scale:.3f}; "
          f"WRITE_SIZE reads {sum(v for _, v in write[0]):,.0f} -> factor {w_scale:.3f}")
    for idx, tag in enumerate(_PMC_TAGS):
        if idx == 0 or idx not in fetch:
            continue
        # zero fills and small copies are the host layer growing a workspace on first use, not the operator's traffic
        own = lambda seg: [(n, v) for n, v in seg if "FillFunctor" not in n and "copyBuffer" not in n]  # noqa: E731
        fk = sum(v for _, v in own(fetch[idx])) * f_scale
        wk = sum(v for _, v in own(write.get(idx, []))) * w_scale
        names = []
        for n, _ in own(fetch[idx]):
            m = re.search(r"([A-Za-z_0-9]+_kernel[A-Za-z_0-9]*|copyBuffer)(<[^()]*>)?", n.replace("(anonymous namespace)::", ""))
            short = (m.group(1) + (m.group(2) or "")) if m else n[:40]
            if short not in names:
                names.append(short)
        print(f"TRAFFIC tag={tag} kernel={'+'.join(names).replace(' ', '')} hbm_bytes={int((fk + wk) * 1024)} fetch_kib={fk:.0f} write_kib={wk:.0f}")


def main():
    args = _parse()
    if args.pmc_summarize:
        _pmc_summarize(*args.pmc_summarize)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: this operator path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    import numpy as np
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    import pytorch_amd as pa          # fails loudly when the native libraries are missing
    from pytorch_amd.testing import workloads

    dev = torch.device("cuda:0")
    props = torch.cuda.get_device_properties(0)
    torch.cuda.set_device(0)
    if args.pmc_pass:
        _pmc_pass(torch, pa, workloads, dev)
        return

    from pytorch_amd import _capi
    clock_mhz = _capi.device_info()[0]               # nominal engine clock from the runtime

    # ------------------------------------------------------------------ headline: C2 quant_matmul
    M, K, N = 1024, 4096, 11008
    d0 = workloads.quant_matmul_inputs(seed=0, M=M, K=K, N=N, weight_nk=True, bias=True)
    set_bytes = M * K + K * N + M * N * 2
    nsets = _nsets(set_bytes)
    gen = torch.Generator(device=dev).manual_seed(1)
    sets = []
    for i in range(nsets):
        if i == 0:
            x1, w_nk = d0["x1"].to(dev), d0["x2"].t().contiguous().to(dev)
        else:
            x1 = torch.randint(-127, 128, (M, K), generator=gen, dtype=torch.int8, device=dev)
            w_nk = torch.randint(-127, 128, (N, K), generator=gen, dtype=torch.int8, device=dev)
        sets.append((x1, w_nk.t()))
    ps, sc, bias = d0["pertoken_scale"].to(dev), d0["scale"].to(dev), d0["bias"].to(dev)

    state = {"i": 0, "out": None}

    def step():
        x1, w = sets[state["i"] % nsets]
        state["i"] += 1
        state["out"] = pa.npu_quant_matmul(x1, w, sc, pertoken_scale=ps, bias=bias, output_dtype=torch.bfloat16)

    # The K timed steps are K calls of torch.ops.npu.npu_quant_matmul issued back to back on the current stream, the way
    # a model's forward pass issues them (the host needs ~7 us per call, the kernel ~45, so the GPU never waits for the
    # host); --graph replays them from one captured HIP graph instead.  The timed region is bracketed by synchronisation.
    graph = None
    if args.graph:
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            step()                                   # one-time set-up on the stream that captures the timed steps
        torch.cuda.synchronize()
        state["i"] = 0
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(args.steps):
                step()
    step()                                           # one-time set-up (workspace, function attributes) is not a step
    torch.cuda.synchronize()
    state["i"] = 0
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    if graph is not None:
        graph.replay()
    else:
        for _ in range(args.steps):
            step()
    ev1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall_ms = (t1 - t0) * 1e3 / args.steps
    kern_ms = ev0.elapsed_time(ev1) / args.steps
    ops = 2.0 * M * N * K
    value_tops = ops / (wall_ms * 1e-3) / 1e12
    achieved_tops = ops / (kern_ms * 1e-3) / 1e12
    # The same launch over a longer run (200 launches, untimed for `value`): what the kernel takes once the first
    # launches after an idle queue (launch latency, clock ramp) no longer weigh, for comparison with launch_us.
    ev2 = torch.cuda.Event(enable_timing=True)
    ev3 = torch.cuda.Event(enable_timing=True)
    ev2.record()
    for _ in range(200):
        step()
    ev3.record()
    torch.cuda.synchronize()
    long_run_us = ev2.elapsed_time(ev3) * 1e3 / 200
    # ... and once the clocks have settled under continuous load (about 30 ms after an idle period: launches 1500-1700)
    for _ in range(1300):
        step()
    ev4 = torch.cuda.Event(enable_timing=True)
    ev5 = torch.cuda.Event(enable_timing=True)
    ev4.record()
    for _ in range(200):
        step()
    ev5.record()
    torch.cuda.synchronize()
    settled_us = ev4.elapsed_time(ev5) * 1e3 / 200
    # the clock the chip holds while all matrix cores are busy (measured after the headline: the probe saturates every
    # SIMD for about a millisecond)
    _capi.sustained_mfma_clock_mhz(iters=2000)       # warm-up
    sustained_mhz = round(_capi.sustained_mfma_clock_mhz(), 1)

    # parity of the timed configuration (set 0), against the oracle on a row sample
    state["i"] = 0
    step()
    out0 = state["out"].cpu()
    parity = {}
    cpu_baseline = None
    if not args.skip_cpu:
        from oracle import golden
        threads = min(16, os.cpu_count() or 1)
        golden.set_threads(threads)
        rows = M          # the whole configuration: ~1.5 s on 16 host threads, and every output element is checked
        a = d0["x1"][:rows].numpy()
        b = d0["x2"].numpy()
        golden.quant_matmul(a[:4], b, d0["scale"].numpy(), d0["pertoken_scale"][:4].numpy(), _bits(d0["bias"]))
        c0 = time.perf_counter()
        want, _ = golden.quant_matmul(a, b, d0["scale"].numpy(), d0["pertoken_scale"][:rows].numpy(), _bits(d0["bias"]))
        c1 = time.perf_counter()
        parity["c2_bit_identical_to_oracle"] = bool(np.array_equal(_bits(out0[:rows]), want))
        cpu_baseline = {"value": round(2.0 * rows * N * K / (c1 - c0) / 1e12, 5), "unit": "TOP/s", "cores": threads,
                        "kind": "port",
                        "sample": f"one pass over the full headline configuration ({rows} rows; int32 GEMM + dequant "
                                  f"epilogue of oracle/golden.c, OpenMP), {c1 - c0:.2f} s"}

    result = {
        "metric": "npu_quant_matmul int8 TOPS (W8A8, int32 accumulate, fused dequant to bf16)",
        "value": round(value_tops, 2),
        "unit": "TOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "configs[1]: npu_quant_matmul x int8[1024,4096] . weight int8[4096,11008] "
                               "(stored [N,K], passed as transposed view), pertoken_scale f32[1024], scale f32[11008], "
                               "bias bf16[11008], out bf16[1024,11008]",
                   "rotating_sets": nsets, "launch": "one captured graph of the timed steps" if args.graph else "one call per step on the current stream", "device": props.name, "compute_units": props.multi_processor_count,
                   "clock_mhz": clock_mhz, "sustained_mfma_clock_mhz": sustained_mhz},
        "roofline": {"bound": "mfma", "achieved": round(achieved_tops, 2), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                     "frac": round(achieved_tops / INT8_PEAK_TOPS, 4), "traffic": _traffic("c2"),
                     "kernel": "qmm_kernel", "launch_us": round(kern_ms * 1e3, 3), "launch_us_over_200_launches": round(long_run_us, 3),
                     "launch_us_settled": round(settled_us, 3),
                     "bit_identical_to_oracle": parity.get("c2_bit_identical_to_oracle"),
                     "peak_at_sustained_clock": round(INT8_PEAK_TOPS * sustained_mhz / 2400.0, 1) if sustained_mhz else None,
                     "frac_at_sustained_clock": round(achieved_tops / (INT8_PEAK_TOPS * sustained_mhz / 2400.0), 4)
                     if sustained_mhz else None},
        "cpu_baseline": cpu_baseline,
        "parity": parity,
    }

    # ------------------------------------------------------------------ the other configurations
    others = []
    only = set(filter(None, args.only.split(",")))

    def want(tag):
        return not args.skip_others and (not only or tag in only)

    copy_cache = {}

    def copy_ceiling_us(nbytes):
        """Time of a plain device-to-device copy that moves `nbytes` in all (half read, half written), launched the same
        way (captured graph, buffers rotated past the Infinity Cache): what a launch of this size can reach on this chip,
        next to which the microsecond-scale kernels are to be read (an empty launch alone takes about 2 us)."""
        half = max(int(nbytes) // 2 // 4096 * 4096, 4096)
        if half not in copy_cache:
            ns = _nsets(2 * half)
            src = [torch.empty(half, dtype=torch.int8, device=dev).fill_(1) for _ in range(ns)]
            dst = [torch.empty(half, dtype=torch.int8, device=dev) for _ in range(ns)]
            calls = [(lambda a=a, b=b: b.copy_(a)) for a, b in zip(src, dst)] * 2
            copy_cache[half] = round(_graph_time_us(torch, calls), 3)
            del src, dst
        return copy_cache[half]

    def hbm_entry(name, bytes_per_launch, us, traffic=None, **extra):
        gbs = bytes_per_launch / (us * 1e-6) / 1e9
        e = {"name": name, "launch_us": round(us, 3), "bytes": int(bytes_per_launch),
             "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": traffic,
                          "copy_ceiling_us": copy_ceiling_us(bytes_per_launch)}}
        e.update(extra)
        return e

    def wq_gate(entry, d, out, group_size, flops):
        """Oracle leg of a weight-only configuration (untimed): the bf16 gate on every output element and the CPU
        baseline (the oracle's own float32 evaluation of the golden formula, timed on the host cores)."""
        if args.skip_cpu:
            return
        from oracle import golden
        from pytorch_amd.testing import bf16_gate
        c0 = time.perf_counter()
        _, gold = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(d["antiquant_scale"]),
                                             _bits(d["antiquant_offset"]), group_size=group_size)
        c1 = time.perf_counter()
        try:
            st = bf16_gate(out, torch.from_numpy(gold))
            entry["parity_bf16_gate"] = True
        except AssertionError as exc:
            entry["parity_bf16_gate"] = False
            entry["parity_error"] = str(exc)[:300]
            st = None
        if st:
            entry["within_1ulp_strict"] = round(st["within_1ulp_strict"], 6)
            entry["bit_identical"] = round(st["bit_identical"], 6)
            entry["max_ulp"] = st["max_ulp"]
        entry["cpu_baseline"] = {"value": round(flops / (c1 - c0) / 1e9, 2), "unit": "GFLOP/s", "cores": golden.get_threads(),
                                 "kind": "port", "sample": f"the full configuration, one pass of the oracle, {c1 - c0:.2f} s"}

    if want("c2kn"):
        # same problem with the weight contiguous as [K,N] (transposed into the workspace first)
        w_kn = d0["x2"].contiguous().to(dev)
        x1 = sets[0][0]
        f = lambda: pa.npu_quant_matmul(x1, w_kn, sc, pertoken_scale=ps, bias=bias, output_dtype=torch.bfloat16)  # noqa: E731
        for _ in range(3):
            f()
        ms = _event_time_ms(torch, f, 20)
        others.append({"name": "c2 quant_matmul, weight contiguous [K,N]", "launch_us": round(ms * 1e3, 2),
                       "roofline": {"bound": "mfma", "achieved": round(ops / (ms * 1e-3) / 1e12, 2), "peak": INT8_PEAK_TOPS,
                                    "unit": "TOP/s", "frac": round(ops / (ms * 1e-3) / 1e12 / INT8_PEAK_TOPS, 4),
                                    "traffic": _traffic("c2_kn")}})
        del w_kn

    if want("c1"):
        rows, cols = 2048, 4096
        nb = rows * cols * 3 + rows * 4
        ns = _nsets(nb)
        xs = [workloads.dynamic_quant_input(seed=0, rows=rows, cols=cols).to(dev)]
        for i in range(1, ns):
            xs.append((torch.randn(rows, cols, generator=gen, device=dev)).to(torch.bfloat16))
        keep = []
        calls = [(lambda x=x: keep.append(pa.npu_dynamic_quant(x))) for x in xs] * 2
        us = _graph_time_us(torch, calls)
        e = hbm_entry("c1 dynamic_quant bf16[2048,4096] (rotating, > Infinity Cache)", nb, us, _traffic("c1"))
        keep.clear()
        calls = [(lambda: keep.append(pa.npu_dynamic_quant(xs[0])))] * 8
        e["cache_hot_us"] = round(_graph_time_us(torch, calls), 3)
        # what a launch of this grid costs when the kernel does nothing: the floor under the 3.1 us that 25 MB take at 8 TB/s
        e["empty_launch_us"] = round(_graph_time_us(torch, [lambda: _capi.empty_launch(2048)] * 16), 3)
        if not args.skip_cpu:
            from oracle import golden
            y, s = pa.npu_dynamic_quant(xs[0])
            c0 = time.perf_counter()
            yg, sg = golden.dynamic_quant(_bits(xs[0]))
            c1 = time.perf_counter()
            e["parity_bit_exact"] = bool(np.array_equal(y.cpu().numpy(), yg) and np.array_equal(s.cpu().numpy(), sg))
            e["cpu_baseline"] = {"value": round(nb / (c1 - c0) / 1e9, 3), "unit": "GB/s", "cores": golden.get_threads(),
                                 "kind": "port", "sample": "the full configuration, one pass"}
        others.append(e)
        # the asymmetric variant on the same inputs (three outputs: codes, scale, offset)
        keep.clear()
        calls = [(lambda x=x: keep.append(pa.npu_dynamic_quant_asymmetric(x))) for x in xs] * 2
        us = _graph_time_us(torch, calls)
        others.append(hbm_entry("dynamic_quant_asymmetric bf16[2048,4096] (rotating, > Infinity Cache)", nb + rows * 4, us, None))
        # SmoothQuant activations: the row is multiplied by per-column smooth scales before it is quantised
        keep.clear()
        smq = (torch.rand(xs[0].shape[-1], generator=gen, device=dev) + 0.5).to(torch.bfloat16)
        calls = [(lambda x=x: keep.append(pa.npu_dynamic_quant(x, smooth_scales=smq))) for x in xs] * 2
        us = _graph_time_us(torch, calls)
        others.append(hbm_entry("dynamic_quant with smooth_scales bf16[2048,4096] (rotating, > Infinity Cache)",
                                nb + xs[0].shape[-1] * 2, us, None))
        del xs, keep

    if want("c3"):
        Mx, Kx, Nx = 16, 8192, 28672
        nb = Kx * Nx + Mx * Kx * 2 + 2 * Nx * 2 + Mx * Nx * 2
        d3 = workloads.w8a16_inputs(seed=0, M=Mx, K=Kx, N=Nx)
        ws = [d3["weight"].to(dev)] + [torch.randint(-127, 128, (Kx, Nx), generator=gen, dtype=torch.int8, device=dev)
                                       for _ in range(1)]
        x, s3, o3 = d3["x"].to(dev), d3["antiquant_scale"].to(dev), d3["antiquant_offset"].to(dev)
        keep = []
        calls = [(lambda w=w: keep.append(pa.npu_weight_quant_batchmatmul(x, w, s3, o3))) for w in ws] * 4
        us = _graph_time_us(torch, calls, reps=10)
        e = hbm_entry("c3 W8A16 x bf16[16,8192] . int8[8192,28672] (weight contiguous [K,N])", nb, us,
                      _traffic("c3"), tflops=round(2.0 * Mx * Kx * Nx / (us * 1e-6) / 1e12, 2))
        wq_gate(e, d3, pa.npu_weight_quant_batchmatmul(x, ws[0], s3, o3), 0, 2.0 * Mx * Kx * Nx)
        others.append(e)
        del ws, keep
        # the layout torch_npu's LinearWeightQuant passes (linear_weight_quant.py:71,106): weight stored [N, K], given as its
        # transposed view; set 0 holds the seeded values the oracle checks
        ws = [d3["weight"].t().contiguous().to(dev).t()] + [torch.randint(-127, 128, (Nx, Kx), generator=gen, dtype=torch.int8, device=dev).t()]
        keep = []
        calls = [(lambda w=w: keep.append(pa.npu_weight_quant_batchmatmul(x, w, s3, o3))) for w in ws] * 4
        us = _graph_time_us(torch, calls, reps=10)
        e = hbm_entry("c3 W8A16 x bf16[16,8192] . int8[8192,28672] (weight stored [N,K] and passed as its transposed view: the contrib module's layout)",
                      nb, us, _traffic("c3_nk"), tflops=round(2.0 * Mx * Kx * Nx / (us * 1e-6) / 1e12, 2))
        wq_gate(e, d3, pa.npu_weight_quant_batchmatmul(x, ws[0], s3, o3), 0, 2.0 * Mx * Kx * Nx)
        others.append(e)
        del ws, keep

    if want("c4"):
        Kx, Nx = 4096, 14336
        for Mx in (1, 8, 32, 128):
            nb = Kx * Nx // 2 + 2 * (Kx // 128) * Nx * 2 + Mx * Kx * 2 + Mx * Nx * 2
            d4 = workloads.w4a16_inputs(seed=0, M=Mx, K=Kx, N=Nx)
            ns = _nsets(nb)
            ws = [d4["weight"].to(dev)] + [torch.randint(-2 ** 31, 2 ** 31 - 1, (Kx, Nx // 8), generator=gen,
                                                         dtype=torch.int32, device=dev) for _ in range(ns - 1)]
            x, s4, o4 = d4["x"].to(dev), d4["antiquant_scale"].to(dev), d4["antiquant_offset"].to(dev)
            keep = []
            calls = [(lambda w=w: keep.append(pa.npu_weight_quant_batchmatmul(x, w, s4, o4, None, None, None, 128)))
                     for w in ws] * 2
            us = _graph_time_us(torch, calls)
            e = hbm_entry(f"c4 W4A16 g128 x bf16[{Mx},4096] . int4[4096,14336]", nb, us,
                          _traffic(f"c4_m{Mx}"),
                          tflops=round(2.0 * Mx * Kx * Nx / (us * 1e-6) / 1e12, 2))
            wq_gate(e, d4, pa.npu_weight_quant_batchmatmul(x, ws[0], s4, o4, None, None, None, 128), 128, 2.0 * Mx * Kx * Nx)
            if Mx == 128:
                tf = 2.0 * Mx * Kx * Nx / (us * 1e-6) / 1e12
                e["roofline_mfma"] = {"bound": "mfma", "achieved": round(tf, 1), "peak": BF16_PEAK_TFLOPS,
                                      "unit": "TFLOP/s", "frac": round(tf / BF16_PEAK_TFLOPS, 4), "traffic": None}
            # the same launches on weights prepared once (pytorch_amd.prepare_weight_quant_weight: rows of 7168 bytes get a
            # padded pitch; values and layout are unchanged)
            wsp = [pa.prepare_weight_quant_weight(w) for w in ws]
            keep.clear()
            e["prepared_weight_us"] = round(_graph_time_us(
                torch, [(lambda w=w: keep.append(pa.npu_weight_quant_batchmatmul(x, w, s4, o4, None, None, None, 128))) for w in wsp] * 2), 3)
            e["prepared_weight_bit_identical"] = bool(torch.equal(pa.npu_weight_quant_batchmatmul(x, wsp[0], s4, o4, None, None, None, 128),
                                                                  pa.npu_weight_quant_batchmatmul(x, ws[0], s4, o4, None, None, None, 128)))
            others.append(e)
            del ws, wsp, keep
            # the layout torch_npu's LinearWeightQuant passes: weight stored [N, K/8] (words along K), per-group
            # parameters stored [N, G], all three given as transposed views
            wks = [torch.randint(-2 ** 31, 2 ** 31 - 1, (Nx, Kx // 8), generator=gen, dtype=torch.int32, device=dev).t()
                   for _ in range(ns)]
            s4t, o4t = s4.t().contiguous().t(), o4.t().contiguous().t()
            keep = []
            calls = [(lambda w=w: keep.append(pa.npu_weight_quant_batchmatmul(x, w, s4t, o4t, None, None, None, 128)))
                     for w in wks] * 2
            us = _graph_time_us(torch, calls)
            others.append(hbm_entry(f"c4 W4A16 g128 x bf16[{Mx},4096] . int4 stored [14336,4096/8] (words along K, parameters "
                                    "[N,G]: the module's transposed views)", nb, us, _traffic(f"c4k_m{Mx}"),
                                    tflops=round(2.0 * Mx * Kx * Nx / (us * 1e-6) / 1e12, 2)))
            del wks, keep

    if want("c2i8"):
        # the headline product with the re-quantised int8 output (packed int64 scale from npu_trans_quant_param, int32 bias)
        Mx, Kx, Nx = 1024, 4096, 11008
        nset = _nsets(Mx * Kx + Kx * Nx)
        xs = [torch.randint(-128, 128, (Mx, Kx), generator=gen, dtype=torch.int8, device=dev) for _ in range(nset)]
        wsn = [torch.randint(-128, 128, (Nx, Kx), generator=gen, dtype=torch.int8, device=dev).t() for _ in range(nset)]
        qp = pa.npu_trans_quant_param(torch.rand(Nx, generator=gen, device=dev) * 1e-4 + 1e-4,
                                      torch.randint(-8, 8, (Nx,), generator=gen, device=dev).float())
        bi = torch.randint(-1000, 1000, (Nx,), generator=gen, device=dev, dtype=torch.int32)
        keep = []
        calls = [(lambda a=a, w=w: keep.append(pa.npu_quant_matmul(a, w, qp, bias=bi, output_dtype=torch.int8)))
                 for a, w in zip(xs, wsn)] * 4
        us = _graph_time_us(torch, calls, reps=10)
        tops = 2.0 * Mx * Kx * Nx / (us * 1e-6) / 1e12
        others.append({"name": "c2 quant_matmul with int8 output (int64 packed scale + offset, int32 bias)", "launch_us": round(us, 3),
                       "roofline": {"bound": "mfma", "achieved": round(tops, 2), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                                    "frac": round(tops / INT8_PEAK_TOPS, 4), "traffic": _traffic("c2_i8")}})
        del xs, wsn, keep

    if want("qd"):
        # W8A8 projections of a Llama-3-8B-shaped layer at decode batch sizes (weights [N,K], rotated so that none is
        # cache-resident): the decode kernel of quant_matmul
        for (Kx, Nx) in ((4096, 6144), (4096, 4096), (4096, 28672), (14336, 4096)):
            nset = _nsets(Kx * Nx)
            wsn = [torch.randint(-128, 128, (Nx, Kx), generator=gen, dtype=torch.int8, device=dev).t() for _ in range(nset)]
            sc = torch.rand(Nx, generator=gen, device=dev) * 1e-2
            # 128 rows on two of them: past the decode kernel's 64 rows, the tiled kernel with the planner's tile and split
            for Mx in (1, 16) + ((128,) if (Kx, Nx) in ((4096, 6144), (14336, 4096)) else ()):
                xs = [torch.randint(-128, 128, (Mx, Kx), generator=gen, dtype=torch.int8, device=dev) for _ in range(nset)]
                ps = torch.rand(Mx, generator=gen, device=dev) * 1e-2
                keep = []
                calls = [(lambda a=a, w=w: keep.append(pa.npu_quant_matmul(a, w, sc, pertoken_scale=ps, output_dtype=torch.bfloat16)))
                         for a, w in zip(xs, wsn)] * 2
                us = _graph_time_us(torch, calls, reps=10)
                nb = Kx * Nx + Mx * Kx + Mx * Nx * 2 + Nx * 4 + Mx * 4
                gate = {}
                if not args.skip_cpu and Mx >= 16:
                    from oracle import golden
                    gold, _ = golden.quant_matmul(xs[0].cpu().numpy(), wsn[0].cpu().numpy(), sc.cpu().numpy(), ps.cpu().numpy())
                    got = pa.npu_quant_matmul(xs[0], wsn[0], sc, pertoken_scale=ps, output_dtype=torch.bfloat16)
                    gate = {"parity_bit_exact": bool(np.array_equal(_bits(got), gold))}
                others.append({"name": f"quant_matmul {'decode ' if Mx <= 64 else ''}int8[{Mx},{Kx}] . int8 stored [{Nx},{Kx}] -> bf16", "launch_us": round(us, 3), **gate,
                               "roofline": {"bound": "hbm", "achieved": round(nb / (us * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBS,
                                            "unit": "GB/s", "frac": round(nb / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                                            "traffic": _traffic(f"qd_{Kx}x{Nx}_m{Mx}"), "copy_ceiling_us": copy_ceiling_us(nb)},
                               "algorithmic_bytes": int(nb)})
                if Kx == 4096 and Mx == 16:
                    # the same launch on weights prepared once (pytorch_amd.prepare_quant_matmul_weight: rows of 4096
                    # bytes get a pitch of 4224)
                    wsp = [pa.prepare_quant_matmul_weight(w) for w in wsn]
                    keep = []
                    calls = [(lambda a=a, w=w: keep.append(pa.npu_quant_matmul(a, w, sc, pertoken_scale=ps, output_dtype=torch.bfloat16)))
                             for a, w in zip(xs, wsp)] * 2
                    usp = _graph_time_us(torch, calls, reps=10)
                    same = bool(torch.equal(pa.npu_quant_matmul(xs[0], wsp[0], sc, pertoken_scale=ps, output_dtype=torch.bfloat16),
                                            pa.npu_quant_matmul(xs[0], wsn[0], sc, pertoken_scale=ps, output_dtype=torch.bfloat16)))
                    others[-1]["prepared_weight_us"] = round(usp, 3)
                    others[-1]["prepared_weight_bit_identical"] = same
                    del wsp
                del xs, keep
            del wsn

    if want("a4w4"):
        # both operands packed int4 (A4W4) at the headline shape: the operator widens them to int8 and runs the int8 GEMM
        Mx, Kx, Nx = 1024, 4096, 11008
        rnd = lambda *sh: torch.randint(-2 ** 31, 2 ** 31 - 1, sh, generator=gen, dtype=torch.int32, device=dev)  # noqa: E731
        nb = Mx * Kx // 2 + Kx * Nx // 2 + Mx * Nx * 2
        xs, wsk = [rnd(Mx, Kx // 8) for _ in range(4)], [rnd(Nx, Kx // 8).t() for _ in range(4)]
        sc = torch.rand(Nx, generator=gen, device=dev) * 1e-2
        ps = torch.rand(Mx, generator=gen, device=dev) * 1e-2
        keep = []
        calls = [(lambda a=a, w=w: keep.append(pa.npu_quant_matmul(a, w, sc, pertoken_scale=ps, output_dtype=torch.bfloat16)))
                 for a, w in zip(xs, wsk)] * 4
        us = _graph_time_us(torch, calls, reps=10)
        others.append({"name": "a4w4 quant_matmul int4[1024,4096] . int4 stored [11008,4096/8] -> bf16 (unpack kernels + int8 GEMM)",
                       "us": round(us, 2), "tops": round(2.0 * Mx * Kx * Nx / (us * 1e-6) / 1e12, 1),
                       "frac_int8_peak": round(2.0 * Mx * Kx * Nx / (us * 1e-6) / 1e12 / INT8_PEAK_TOPS, 4),
                       "roofline": {"bound": "mfma", "achieved": round(2.0 * Mx * Kx * Nx / (us * 1e-6) / 1e12, 2), "peak": INT8_PEAK_TOPS,
                                    "unit": "TOP/s", "frac": round(2.0 * Mx * Kx * Nx / (us * 1e-6) / 1e12 / INT8_PEAK_TOPS, 4),
                                    "traffic": _traffic("a4w4")}, "algorithmic_bytes": int(nb)})
        del xs, wsk, keep

    if want("c5"):
        H, I = 4096, 14336
        for Mx in (16, 64, 2048):
            d5 = workloads.mlp_inputs(seed=0, M=Mx, hidden=H, inter=I)
            x = d5["x"].to(dev)
            sgu, sd = d5["scale_gate_up"].to(dev), d5["scale_down"].to(dev)
            # weight sets: 176 MB each; two sets exceed the 256 MB Infinity Cache, so alternating them keeps every
            # replay on weights that are not cache-resident (set 0 is the seeded one the oracle checks)
            wsets = [(d5["w_gate_up"].to(dev).t(), d5["w_down"].to(dev).t())]
            wsets.append((torch.randint(-127, 128, (2 * I, H), generator=gen, dtype=torch.int8, device=dev).t(),
                          torch.randint(-127, 128, (H, I), generator=gen, dtype=torch.int8, device=dev).t()))

            def mlp(wgu, wd, stages=False):
                xq, xsc = pa.npu_dynamic_quant(x)
                gu = pa.npu_quant_matmul(xq, wgu, sgu, pertoken_scale=xsc, output_dtype=torch.bfloat16)
                act = pa.npu_swiglu(gu)
                aq, asc = pa.npu_dynamic_quant(act)
                out = pa.npu_quant_matmul(aq, wd, sd, pertoken_scale=asc, output_dtype=torch.bfloat16)
                return (xq, xsc, gu, act, aq, asc, out) if stages else out

            def mlp_fused(wgu, wd):
                xq, xsc = pa.npu_dynamic_quant(x)
                gu = pa.npu_quant_matmul(xq, wgu, sgu, pertoken_scale=xsc, output_dtype=torch.bfloat16)
                aq, asc = pa.npu_swiglu_quant(gu, activate_left=True, quant_mode=1)
                return pa.npu_quant_matmul(aq, wd, sd, pertoken_scale=asc, output_dtype=torch.bfloat16)

            same = bool(torch.equal(mlp(*wsets[0]), mlp_fused(*wsets[0])))
            mops = 2.0 * Mx * H * 2 * I + 2.0 * Mx * I * H
            wbytes = H * 2 * I + I * H
            # algorithmic bytes of the fused chain: weights, activations in and out of every stage, scales
            abytes = wbytes + Mx * (H * 2 + H + 4) + Mx * (H + 2 * I * 2) + Mx * (2 * I * 2 + I + 4) + Mx * (I + H * 2) + (2 * I + H) * 4
            gate, cpu = {}, None
            if not args.skip_cpu and Mx >= 64:
                # stage-wise gate: every GPU stage against the oracle applied to that stage's actual GPU input; every stage
                # works row by row, so at M=2048 the oracle checks a sample of 64 rows spread over the row tiles
                from oracle import golden
                rows = np.arange(Mx) if Mx == 64 else np.sort(np.concatenate([np.arange(0, Mx, 64) + 7, np.arange(0, Mx, 64) + 40]))
                xq, xsc, gu, act, aq, asc, out = (t.cpu()[torch.from_numpy(rows)] for t in mlp(*wsets[0], stages=True))
                c0 = time.perf_counter()
                yg, sg = golden.dynamic_quant(_bits(d5["x"][torch.from_numpy(rows)]))
                gate["dynamic_quant_1_bit_exact"] = bool(np.array_equal(xq.numpy(), yg) and np.array_equal(xsc.numpy(), sg))
                want_gu, _ = golden.quant_matmul(xq.numpy(), d5["w_gate_up"].t().numpy(), d5["scale_gate_up"].numpy(), xsc.numpy())
                gate["gate_up_bit_exact"] = bool(np.array_equal(_bits(gu), want_gu))
                dist = golden.bf16_ulp_distance(_bits(act), golden.swiglu(_bits(gu)))
                gate["swiglu_within_1ulp"] = bool(dist.max() <= 1)
                gate["swiglu_bit_identical_frac"] = round(float((dist == 0).mean()), 6)
                yg2, sg2 = golden.dynamic_quant(_bits(act))
                gate["dynamic_quant_2_bit_exact"] = bool(np.array_equal(aq.numpy(), yg2) and np.array_equal(asc.numpy(), sg2))
                want_out, _ = golden.quant_matmul(aq.numpy(), d5["w_down"].t().numpy(), d5["scale_down"].numpy(), asc.numpy())
                gate["down_bit_exact"] = bool(np.array_equal(_bits(out), want_out))
                gate["rows_checked"] = int(rows.size)
                c1 = time.perf_counter()
                cpu = {"value": round(2.0 * rows.size * H * 3 * I / (c1 - c0) / 1e12, 5), "unit": "TOP/s", "cores": golden.get_threads(), "kind": "port",
                       "sample": f"one pass of the oracle over the five stages on {rows.size} rows (stage-wise, on the GPU's stage inputs), {c1 - c0:.2f} s"}
            for fn, label in ((mlp, "5 kernels"), (mlp_fused, "4 kernels, fused SwiGLU + dynamic_quant")):
                keep = []
                calls = [(lambda w=w: keep.append(fn(*w))) for w in wsets] * 2
                us = _graph_time_us(torch, calls, reps=10)
                keep.clear()
                hot = _graph_time_us(torch, [lambda: keep.append(fn(*wsets[0]))] * 4, reps=10)
                e = {"name": f"c5 Llama-3-8B-shaped W8A8 MLP, M={Mx} ({label}; two weight sets alternate, 352 MB > Infinity Cache)",
                     "chain_us": round(us, 2), "chain_us_cache_resident_weights": round(hot, 2),
                     "int8_tops": round(mops / (us * 1e-6) / 1e12, 2),
                     "roofline": ({"bound": "hbm", "achieved": round(abytes / (us * 1e-6) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                   "frac": round(abytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                                   "traffic": _traffic(f"c5_m{Mx}") if fn is mlp_fused else None, "copy_ceiling_us": copy_ceiling_us(abytes)} if Mx <= 64 else
                                  {"bound": "mfma", "achieved": round(mops / (us * 1e-6) / 1e12, 2), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                                   "frac": round(mops / (us * 1e-6) / 1e12 / INT8_PEAK_TOPS, 4),
                                   "traffic": _traffic(f"c5_m{Mx}") if fn is mlp_fused else None}),
                     "algorithmic_bytes": int(abytes)}
                if fn is mlp_fused:
                    e["bit_identical_to_5_kernel_chain"] = same
                    if Mx <= 64:
                        # the same chain on weights prepared once (rows of 4096 bytes get a padded pitch)
                        wprep = [(pa.prepare_quant_matmul_weight(wg), wdn) for wg, wdn in wsets]
                        keep.clear()
                        e["chain_us_prepared_weights"] = round(_graph_time_us(
                            torch, [(lambda w=w: keep.append(fn(*w))) for w in wprep] * 2, reps=10), 2)
                        e["prepared_weights_bit_identical"] = bool(torch.equal(fn(*wprep[0]), fn(*wsets[0])))
                        del wprep
                elif gate:
                    e["parity_stagewise"] = gate
                    e["parity_all_stages"] = bool(all(v for k, v in gate.items() if k not in ("swiglu_bit_identical_frac", "rows_checked")))
                    e["cpu_baseline"] = cpu
                others.append(e)
                del keep
            del wsets

    if want("aq"):
        # standalone antiquantisation of a decoder-MLP-sized weight: int8 / packed int4 [4096, 14336] -> bf16
        R, C = 4096, 14336
        sc_f = (torch.rand(C, generator=gen, device=dev) * 9e-3 + 1e-3)
        of_f = (torch.rand(C, generator=gen, device=dev) * 8 - 4)
        for bits in (8, 4):
            nb = R * C * bits // 8 + R * C * 2 + 2 * C * 4
            ns = _nsets(nb)
            if bits == 8:
                xs = [torch.randint(-128, 128, (R, C), generator=gen, dtype=torch.int8, device=dev) for _ in range(ns)]
            else:
                xs = [torch.randint(-2 ** 31, 2 ** 31 - 1, (R, C // 8), generator=gen, dtype=torch.int32, device=dev)
                      for _ in range(ns)]
            keep = []
            calls = [(lambda x=x: keep.append(pa.npu_anti_quant(x, sc_f, offset=of_f, dst_dtype=torch.bfloat16))) for x in xs] * 2
            us = _graph_time_us(torch, calls)
            others.append(hbm_entry(f"npu_anti_quant int{bits}[4096,14336] -> bf16 (per-column float32 scale and offset)", nb, us,
                                    _traffic("aq_int8") if bits == 8 else None))
            del xs, keep

    if want("qz"):
        # static quantisation of an activation matrix with per-channel scales and zero points: bf16 [2048, 14336] -> int8
        R, C = 2048, 14336
        sc_q = torch.rand(C, generator=gen, device=dev) * 0.05 + 0.01
        zp_q = torch.randint(-8, 8, (C,), generator=gen, device=dev, dtype=torch.int32)
        nb = R * C * 2 + R * C + 2 * C * 4
        xs = [(torch.randn(R, C, generator=gen, device=dev)).to(torch.bfloat16) for _ in range(_nsets(nb))]
        keep = []
        calls = [(lambda x=x: keep.append(pa.npu_quantize(x, sc_q, zp_q, torch.qint8, -1))) for x in xs] * 2
        us = _graph_time_us(torch, calls)
        others.append(hbm_entry("npu_quantize bf16[2048,14336] -> int8 (per-channel float32 scales, int32 zero points)", nb, us, None))
        del xs, keep

    if others:
        result["others"] = others
        # the same lines in short, inside `config` (a consumer that keeps only the contract's keys still sees them):
        # [us per launch or chain, fraction of the bounding peak, us of a plain copy of the same bytes, oracle gate]
        def gate(e):
            flags = [v for k, v in e.items() if k.startswith("parity") and isinstance(v, bool)]
            return all(flags) if flags else None
        result["config"]["lines"] = {e["name"][:64]: [e.get("launch_us", e.get("chain_us", e.get("us"))), e.get("roofline", {}).get("frac"),
                                                       e.get("roofline", {}).get("copy_ceiling_us"), gate(e)] for e in others}
    print(json.dumps(result))


if __name__ == "__main__":
    main()
