#!/usr/bin/env python3
"""Benchmark of the matmult hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu] [--only NAME[,NAME...]] [--context] [--shapes SPEC[,SPEC...]]

One "step" is one pass of nt::matmult over the headline workload of BASELINE.json
(config 3): a 4096 x 4096 x 4096 BFloat16 product, inputs randn*0.02 already resident in
HBM, fp32 accumulation, C += A.B (the accumulate contract of nt_matmult).  The timed
region brackets exactly K launches between device synchronisations; the per-launch
duration used for the roofline comes from HIP events recorded on the launch stream
inside that region.  Prints ONE JSON line.

Besides the headline value the line carries
  roofline      achieved vs. MI355X dense-MFMA peak for the dominant kernel,
  cpu_baseline  the CPU oracle's tiled restatement of the reference's TBB/SIMD GEMM, timed
                on this host's cores on a bounded sample (reported, not a target),
  extras        the other dtypes at 4096^3 and the remaining BASELINE configurations; every entry is timed after the
                same settling load as the headline (see settle()), so the figures do not depend on --warmup.

--only NAME[,NAME...] times just those extras entries (for one rocprofv3 run per workload); the settling load is a
different kernel instantiation than the workload, so a kernel-trace summary of such a run averages the workload's
kernels over its --warmup + timed launches only.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "fp32": 157.3, "fp64": 78.6, "int8": 5000.0}   # MI355X dense MFMA (int8: Top/s)
PEAK_HBM_GBS = 8000.0


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # the GPU needs some 20-30 ms of load before its clocks settle: 200 untimed launches (27 ms) put the timed
    # region into the steady state that a training or serving loop runs in
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-extras", action="store_true", help="only the headline workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="comma-separated extras entries to time alone (skips the headline and the CPU leg)")
    ap.add_argument("--power", default="", help="comma-separated extras entries that are ALSO run back to back for --power-seconds while amd-smi is "
                                                "sampled (average socket power, clocks): what the power manager does under each workload")
    ap.add_argument("--power-seconds", type=float, default=2.5)
    ap.add_argument("--shapes", default="",
                    help="comma-separated extra products DTYPE:MxKxN[:nn|nt|tn|tt] (bf16, fp16, fp32, fp64; results overwritten) to time "
                         "like the extras entries; with --only none just these are run (planner studies, e.g. under NTG_TILE_EDGE)")
    ap.add_argument("--context", action="store_true",
                    help="also time torch's own operators (hipBLASLt / MIOpen behind torch.matmul, bmm, _int_mm, conv2d) on the same "
                         "operands, alternating with this library in one process: context for the figures, never part of `value`")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy (known HBM traffic) so that counter runs "
                         "(rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) can be scaled")
    return ap.parse_args()


def context_table(torch, F, _lib, lib, dev, stream, make_gemm, settle):
    """torch's operators on the same operands as this library, same process, alternating: five blocks of back-to-back
    launches per side after one settling load, the median block's microseconds per launch.  What torch dispatches to
    (hipBLASLt, rocBLAS, MIOpen) is torch's choice; its outputs are not compared here (the parity tests do that against the
    oracle)."""
    table = {}

    def block(fn, n):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / n

    def compare(name, ours, theirs, op):
        for fn in (ours, theirs):
            for _ in range(3):
                fn()
        torch.cuda.synchronize()
        settle("context_" + name)
        est = max(block(ours, 3), 1.0)
        n = int(min(max(20, 4000.0 / est), 400))
        a, b = [], []
        for _ in range(5):
            a.append(block(ours, n))
            b.append(block(theirs, n))
        a.sort()
        b.sort()
        table[name] = {"this_library_us": round(a[2], 2), "torch_us": round(b[2], 2), "torch_op": op, "launches_per_block": n}

    def gemm(name, dtype, m, k, n, tb=False, batch=1, scale=0.05):
        ours = make_gemm(dtype, m, k, n, tb=tb, batch=batch, scale=scale, mode=_lib.C_OVERWRITE)
        a, b, c = ours.keep[0], ours.keep[1], ours.keep[2]
        if batch == 1:
            a2, b2, c2 = a[0], b[0], torch.empty_like(c[0])
            theirs = (lambda: torch.matmul(a2, b2.t(), out=c2)) if tb else (lambda: torch.matmul(a2, b2, out=c2))
            op = "torch.matmul(out=)"
        else:
            c2 = torch.empty_like(c)
            theirs = (lambda: torch.bmm(a, b.transpose(1, 2), out=c2)) if tb else (lambda: torch.bmm(a, b, out=c2))
            op = "torch.bmm(out=)"
        compare(name, ours, theirs, op)

    bf, hf, f32, f64 = torch.bfloat16, torch.float16, torch.float32, torch.float64
    gemm("bf16_4096", bf, 4096, 4096, 4096, scale=0.02)
    gemm("fp16_4096", hf, 4096, 4096, 4096, scale=0.02)
    gemm("fp32_4096", f32, 4096, 4096, 4096)
    gemm("fp64_4096", f64, 4096, 4096, 4096)
    gemm("fp32_512", f32, 512, 512, 512)
    gemm("fp32_b32_1024x768x1024", f32, 1024, 768, 1024, batch=32)
    gemm("bf16_2048", bf, 2048, 2048, 2048)
    gemm("bf16_3072", bf, 3072, 3072, 3072)
    gemm("bf16_2048x4096x4096", bf, 2048, 4096, 4096)
    gemm("bf16_256x4096x11008", bf, 256, 4096, 11008, scale=0.1)
    gemm("bf16_linear_8192x4096x11008_x_wT", bf, 8192, 4096, 11008, tb=True, scale=0.1)
    gemm("fp32_linear_8192x4096x11008_x_wT", f32, 8192, 4096, 11008, tb=True, scale=0.1)
    gemm("bf16_b32_1024", bf, 1024, 1024, 1024, batch=32)
    gemm("bf16_16x8192x8192", bf, 16, 8192, 8192)
    gemm("fp32_16x8192x8192", f32, 16, 8192, 8192)
    if hasattr(torch, "_int_mm"):
        a = torch.randint(-128, 128, (4096, 4096), device=dev, dtype=torch.int8)
        b = torch.randint(-128, 128, (4096, 4096), device=dev, dtype=torch.int8)
        ours = make_gemm(torch.int8, 4096, 4096, 4096, ints=True, mode=_lib.C_OVERWRITE)
        compare("int8_4096", ours, lambda: torch._int_mm(a, b), "torch._int_mm (int32 result; this library stores the wrapped int8)")
    for half in (True, False):
        x = torch.randn(64, 256, 56, 56, device=dev)
        w = torch.randn(256, 256, 3, 3, device=dev) / 48.0
        g = torch.randn(64, 256, 56, 56, device=dev)
        if half:
            x, w, g = x.bfloat16(), w.bfloat16(), g.bfloat16()
        tag = "bf16" if half else "fp32"
        compare("conv2d_64x256x56x56_3x3_" + tag, lambda: F.conv2d(x, w, padding=1), lambda: torch.nn.functional.conv2d(x, w, padding=1),
                "torch.nn.functional.conv2d")
        compare("conv2d_backward_64x256x56x56_3x3_" + tag, lambda: F.conv2d_backward(x, w, g, padding=1),
                lambda: torch.ops.aten.convolution_backward(g, x, w, None, [1, 1], [1, 1], [1, 1], False, [0, 0], 1, [True, True, False]),
                "aten.convolution_backward (input and weight gradients)")
        del x, w, g
    return table


def read_traffic_note():
    """HBM bytes per launch of the headline kernel, measured offline with rocprofv3 --pmc
    (FETCH_SIZE / WRITE_SIZE, scaled by a copy kernel); None until that profile exists."""
    path = os.path.join(ROOT, "profiles", "gemm_ring_bf16_4096_hbm_traffic.txt")
    try:
        for line in open(path):
            if line.startswith("hbm_traffic_bytes_per_launch:"):
                return float(line.split(":", 1)[1].strip())
    except OSError:
        pass
    return None


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no sharding); "
              f"--gpus {args.gpus} is not supported. Re-run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch

    from neurotensor_amd import _lib
    from neurotensor_amd import functional as F

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.manual_seed(1003)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def make_gemm(dtype, m, k, n, ta=False, tb=False, batch=1, scale=1.0, mode=_lib.C_ACCUMULATE, ints=False, bias_relu=False):
        ashape = (batch, k, m) if ta else (batch, m, k)
        bshape = (batch, n, k) if tb else (batch, k, n)
        if ints:
            lo, hi = (-128, 128) if dtype == torch.int8 else (-8, 9)      # int8: the full value range
            a = torch.randint(lo, hi, ashape, device=dev, dtype=dtype)
            b = torch.randint(lo, hi, bshape, device=dev, dtype=dtype)
        else:
            a = (torch.randn(ashape, device=dev) * scale).to(dtype)
            b = (torch.randn(bshape, device=dev) * scale).to(dtype)
        c = torch.zeros((batch, m, n), device=dev, dtype=dtype)
        d = _lib.GemmDesc()
        d.dtype = F.ntg_dtype(a)
        d.transpose_a, d.transpose_b, d.c_mode = int(ta), int(tb), mode
        d.m, d.k, d.n, d.batches = m, k, n, batch
        d.stride_a, d.stride_b, d.stride_c = m * k, k * n, m * n
        ws_bytes = lib.ntg_gemm_workspace_bytes(ctypes.byref(d))     # > 0 only for few-tile, deep-k shapes (split along k)
        ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dev) if ws_bytes > 0 else None
        if ws is not None:
            d.workspace, d.workspace_bytes = ws.data_ptr(), ws_bytes

        bias = None
        if bias_relu:                       # Linear -> ReLU in one launch: bias row as starting value, clamp in the epilogue
            bias = (torch.randn((n,), device=dev) * scale).to(dtype)
            d.c_mode, d.bias, d.bias_col_stride = _lib.C_BIAS, bias.data_ptr(), 1
        entry = lib.ntg_gemm_relu_dev if bias_relu else lib.ntg_gemm_dev

        def launch():
            _lib.check(entry(ctypes.byref(d), a.data_ptr(), b.data_ptr(), c.data_ptr(), stream))

        launch.keep = (a, b, c, d, ws, bias)
        return launch

    def time_steps(fn, steps, warmup):
        """(wall ms per step over the whole timed region, mean ms per launch from a pair of HIP
        events recorded on the launch stream around the same K launches).  One event pair, not
        one per launch: an event between two kernels drains the queue and would add a gap of
        several microseconds to every launch."""
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        ev_ms = e0.elapsed_time(e1) / steps
        return wall_ms, ev_ms

    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(3)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)          # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    N = 4096
    flops = 2.0 * N * N * N
    only = [x for x in args.only.split(",") if x]
    power = [x for x in args.power.split(",") if x]

    def smi_sample():
        """One reading of amd-smi: socket power in W and the graphics clock in MHz averaged over the XCDs (None without the tool)."""
        import subprocess
        try:
            txt = subprocess.run(["amd-smi", "metric", "--power", "--clock", "--json"], capture_output=True, text=True, timeout=10).stdout
            data = json.loads(txt)
            gpu = (data["gpu_data"] if isinstance(data, dict) else data)[0]
        except Exception:
            return None
        out = {}
        try:
            out["power_w"] = float(gpu["power"]["socket_power"]["value"])
        except (KeyError, TypeError, ValueError):
            pass
        clks = []
        for key, val in gpu.get("clock", {}).items():
            try:
                if key.startswith("gfx_"):
                    clks.append(float(val["clk"]["value"]))
                elif key.startswith("mem_") and "mclk_mhz" not in out:
                    out["mclk_mhz"] = float(val["clk"]["value"])
            except (KeyError, TypeError, ValueError):
                pass
        if clks:
            out["sclk_mhz"] = sum(clks) / len(clks)
        return out or None

    def power_run(fn, seconds):
        """fn() back to back for `seconds` (launches queued a few milliseconds ahead) while a thread samples amd-smi;
        the first 0.5 s of samples are dropped (clocks and the power average settling)."""
        import threading
        samples, stop = [], threading.Event()

        def sampler():
            t0 = time.perf_counter()
            while not stop.is_set():
                smp = smi_sample()
                if smp and time.perf_counter() - t0 > 0.5:
                    samples.append(smp)

        th = threading.Thread(target=sampler, daemon=True)
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        per = max(time.perf_counter() - t0, 2e-5)
        chunk = max(1, int(0.004 / per))
        th.start()
        n, t0 = 0, time.perf_counter()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        while time.perf_counter() - t0 < seconds:
            for _ in range(chunk):
                fn()
            n += chunk
            torch.cuda.synchronize()
        e1.record()
        torch.cuda.synchronize()
        stop.set()
        th.join(timeout=15)
        res = {"launches": n, "ms_per_launch": round(e0.elapsed_time(e1) / n, 5), "smi_samples": len(samples)}
        for key in ("power_w", "sclk_mhz", "mclk_mhz"):
            vals = [smp[key] for smp in samples if key in smp]
            if vals:
                res[key + "_avg"] = round(sum(vals) / len(vals), 1)
                res[key + "_max"] = round(max(vals), 1)
        return res

    # Coming from idle the GPU runs its first 20-30 ms of work at lower clocks.  Every measurement (20 or more timed steps)
    # is therefore preceded by SETTLE_MS of back-to-back 4096^3 16-bit products -- the Float16 instantiation for every
    # workload but the Float16 one, which gets the BFloat16 instantiation: a load of the same kind under another kernel
    # name, so that a kernel-trace summary of the run averages the measured kernel over its own launches only.  The
    # workload's --warmup launches and its timed launches follow without a gap.  Counter-collection runs (a handful of
    # steps) skip the load.
    SETTLE_MS = 40.0
    settle_f16 = make_gemm(torch.float16, N, N, N, scale=0.02, mode=_lib.C_OVERWRITE)
    settle_bf16 = make_gemm(torch.bfloat16, N, N, N, scale=0.02, mode=_lib.C_OVERWRITE)
    settled_launches = {}

    def settle(name, load=None):
        if args.steps < 20:
            return
        load = load or settle_f16
        n = int(SETTLE_MS / 0.105) + 1
        for _ in range(n):
            load()
        settled_launches[name] = n

    out = {}
    extras = {}
    if not only:
        # the driver's protocol from a cold start: what --steps / --warmup alone read, first thing after start-up (the
        # two launches before the pause load the code object; the pause lets the clocks fall back to idle)
        head = make_gemm(torch.bfloat16, N, N, N, scale=0.02)
        head(); head()
        torch.cuda.synchronize()
        time.sleep(0.5)
        _, cold_ms = time_steps(head, args.steps, args.warmup)
        extras["c3_bf16_4096_cold"] = {"ms": round(cold_ms, 5), "rate": round(flops / (cold_ms * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
                                       "frac_of_peak": round(flops / (cold_ms * 1e-3) / 1e12 / PEAK_TFLOPS["bf16"], 4),
                                       "note": f"the headline workload from an idle GPU: {args.warmup} warm-up launches, no settling load"}

        # ---------------- headline: config 3, BFloat16 4096^3, C += A.B ----------------
        settle("headline")
        wall_ms, ev_ms = time_steps(head, args.steps, args.warmup)
        value = flops / (wall_ms * 1e-3) / 1e12
        achieved = flops / (ev_ms * 1e-3) / 1e12

        out = {
            "metric": "matmult TFLOP/s at 4096^3 (BFloat16, fp32 accumulate)",
            "value": round(value, 2),
            "unit": "TFLOP/s",
            "n_gpus": 1,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": round(wall_ms, 5),
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": "bf16",
            "data": "synthetic",
            "config": {"workload": "nt::matmult A[4096,4096].B[4096,4096] BFloat16, inputs randn*0.02 resident in HBM, "
                                   "C += A.B (BASELINE config 3)", "m": N, "k": N, "n": N, "c_mode": "accumulate",
                       "untimed_launches_before_timed_region": settled_launches.get("headline", 0) + args.warmup,
                       "settling_load": f"{settled_launches.get('headline', 0)} launches of the Float16 4096^3 product (about {SETTLE_MS:.0f} ms) "
                                        "before the warm-up launches of every timed workload"},
            "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS["bf16"], "unit": "TFLOP/s",
                         "frac": round(achieved / PEAK_TFLOPS["bf16"], 4), "traffic": read_traffic_note(),
                         "traffic_source": "profiles/gemm_ring_bf16_4096_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured in this run)",
                         "kernel": "ntg::gemm_ring_kernel<BFloat16, NN>", "launch_ms": round(ev_ms, 5)},
        }
        del head

    # ---------------- extras: the other dtypes and configurations ----------------
    if not args.no_extras or only:
        steps, warm = max(20, args.steps), max(5, args.warmup)

        def run(name, make, work, peak=None, unit="TFLOP/s", scale=1e12, load=None):
            """make() builds the workload (its buffers live only while it is timed); timed over at least `steps`
            launches and about 10 ms, after the settling load and `warm` warm-up launches"""
            if only and name not in only:
                return
            fn = make()
            fn()                                    # (loads the kernel's code object: host time during which the GPU would idle)
            settle(name, load)                      # every other launch of the workload's own kernels comes after the settling load
            fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            est_ms = max((time.perf_counter() - t0) * 1e3, 1e-3)
            st = int(min(max(steps, 10.0 / est_ms), 1000))
            _, ms = time_steps(fn, st, warm)
            rate = work / (ms * 1e-3) / scale
            e = {"ms": round(ms, 5), "rate": round(rate, 2), "unit": unit, "timed_launches": st}
            if peak:
                e["frac_of_peak"] = round(rate / peak, 4)
            if name in power:
                pw = power_run(fn, args.power_seconds)
                pw["rate"] = round(work / (pw["ms_per_launch"] * 1e-3) / scale, 2)
                e["sustained"] = pw
            extras[name] = e
            del fn

        G = lambda *a, **k: (lambda: make_gemm(*a, **k))
        if only:      # (the headline workload as an extras entry, for runs that time single workloads)
            run("c3_bf16_4096_accumulate", G(torch.bfloat16, N, N, N, scale=0.02), flops, PEAK_TFLOPS["bf16"])
        run("c3_fp16_4096", G(torch.float16, N, N, N, scale=0.02), flops, PEAK_TFLOPS["fp16"], load=settle_bf16)
        run("c3_bf16_4096_overwrite", G(torch.bfloat16, N, N, N, scale=0.02, mode=_lib.C_OVERWRITE), flops, PEAK_TFLOPS["bf16"])
        # diagnostic: the same kernel on all-zero operands (no operand toggling: the clock stays higher) -- the difference to the
        # line above is what the power manager takes, not what the instruction stream costs
        run("c3_bf16_4096_zero_operands", G(torch.bfloat16, N, N, N, scale=0.0, mode=_lib.C_OVERWRITE), flops, PEAK_TFLOPS["bf16"])
        # (Float16 runs the same instruction stream: equal to BFloat16 on zeros, slower on random operands by what its wider mantissa draws)
        run("c3_fp16_4096_zero_operands", G(torch.float16, N, N, N, scale=0.0, mode=_lib.C_OVERWRITE), flops, PEAK_TFLOPS["fp16"], load=settle_bf16)
        run("c3_fp16_4096_overwrite", G(torch.float16, N, N, N, scale=0.02, mode=_lib.C_OVERWRITE), flops, PEAK_TFLOPS["fp16"], load=settle_bf16)

        # the same matrix instruction on operands that stay in registers (no LDS, no global memory in the loop; 256 workgroups
        # of four wavefronts with the 256 x 256 tile's accumulator blocks): what the matrix pipes sustain on these operand
        # values before any data movement -- the ceiling of a product kernel on such data
        def mfma_only(scale):
            def make():
                ops = (torch.randn(_lib.DIAG_MFMA_OPERAND_BYTES // 2, device=dev) * scale).bfloat16()
                sink = torch.empty(256 * 256, device=dev, dtype=torch.float32)
                call = lambda: _lib.check(lib.ntg_diag_mfma_rate_dev(_lib.BFLOAT16, ops.data_ptr(), 100, 256, sink.data_ptr(), stream))
                call.keep = (ops, sink)
                return call
            return make
        mf = 256 * 100 * float(_lib.DIAG_MFMA_FLOPS_PER_PASS)
        run("mfma_registers_only_bf16_random_operands", mfma_only(0.02), mf, PEAK_TFLOPS["bf16"])
        run("mfma_registers_only_bf16_zero_operands", mfma_only(0.0), mf, PEAK_TFLOPS["bf16"])
        run("c3_fp32_4096", G(torch.float32, N, N, N), flops, PEAK_TFLOPS["fp32"])
        run("c3_fp64_4096", G(torch.float64, N, N, N), flops, PEAK_TFLOPS["fp64"])
        run("c1_fp32_512", G(torch.float32, 512, 512, 512), 2.0 * 512 ** 3, PEAK_TFLOPS["fp32"])
        f2 = 2.0 * 32 * 1024 * 768 * 1024
        run("c2a_fp32_b32_1024x768x1024", G(torch.float32, 1024, 768, 1024, batch=32), f2, PEAK_TFLOPS["fp32"])
        run("c2b_fp32_b32_transpose_b", G(torch.float32, 1024, 768, 1024, tb=True, batch=32), f2, PEAK_TFLOPS["fp32"])
        run("c2c_int32_b8_1024", G(torch.int32, 1024, 1024, 1024, batch=8, ints=True), 2.0 * 8 * 1024 ** 3, None, "Top/s")
        run("c3_int8_4096", G(torch.int8, N, N, N, ints=True, mode=_lib.C_OVERWRITE), flops, PEAK_TFLOPS["int8"], "Top/s")
        f4 = 2.0 * 8192 * 4096 * 11008
        for dt, nm in ((torch.float32, "fp32"), (torch.bfloat16, "bf16")):
            pk = PEAK_TFLOPS[nm]
            run(f"c4_linear_fwd_{nm}", G(dt, 8192, 4096, 11008, tb=True, mode=_lib.C_OVERWRITE, scale=0.1), f4, pk)
            run(f"c4_linear_fwd_bias_relu_{nm}", G(dt, 8192, 4096, 11008, tb=True, scale=0.1, bias_relu=True), f4, pk)
            run(f"c4_linear_dx_{nm}", G(dt, 8192, 11008, 4096, mode=_lib.C_OVERWRITE, scale=0.1), f4, pk)
            run(f"c4_linear_dw_{nm}", G(dt, 11008, 8192, 4096, ta=True, mode=_lib.C_OVERWRITE, scale=0.1), f4, pk)
        # the same Linear layer on 16 and 256 rows (inference-sized batches): HBM-bound streaming kernel, split along k
        wbytes = 2.0 * 4096 * 11008
        run("linear_bf16_16_rows_4096x11008", G(torch.bfloat16, 16, 4096, 11008, mode=_lib.C_OVERWRITE, scale=0.1),
            wbytes + 2.0 * 16 * (4096 + 11008), PEAK_HBM_GBS, "GB/s", 1e9)
        run("linear_bf16_256_rows_4096x11008", G(torch.bfloat16, 256, 4096, 11008, mode=_lib.C_OVERWRITE, scale=0.1),
            2.0 * 256 * 4096 * 11008, PEAK_TFLOPS["bf16"])
        # mid-sized squares: the 128 x 128 (16-bit) and 64/128 (Float32) tiles of the DMA-fed kernel
        f2k = 2.0 * 2048 ** 3
        run("mid_bf16_2048", G(torch.bfloat16, 2048, 2048, 2048, scale=0.05, mode=_lib.C_OVERWRITE), f2k, PEAK_TFLOPS["bf16"])
        run("mid_fp32_2048", G(torch.float32, 2048, 2048, 2048, mode=_lib.C_OVERWRITE), f2k, PEAK_TFLOPS["fp32"])
        # 192 tiles of 192 x 256 (144 of 256 x 256)
        run("mid_bf16_3072", G(torch.bfloat16, 3072, 3072, 3072, scale=0.05, mode=_lib.C_OVERWRITE), 2.0 * 3072 ** 3, PEAK_TFLOPS["bf16"])
        # one round of 256 tiles of 128 x 256 (the square tiles give 128 or 512)
        run("mid_bf16_2048x4096x4096", G(torch.bfloat16, 2048, 4096, 4096, scale=0.05, mode=_lib.C_OVERWRITE), 2.0 * 2048 * 4096 * 4096,
            PEAK_TFLOPS["bf16"])
        # a batch as a strided launch and as device pointer tables whose entries the caller vouches for (ntg_gemm_ptrs_dev with
        # NTG_GEMM_PTRS_ALIGNED16: the same DMA-fed kernels; without the vouch the register-staged ones)
        fb = 2.0 * 32 * 1024 ** 3
        run("batch_bf16_32x1024_strided", G(torch.bfloat16, 1024, 1024, 1024, batch=32, scale=0.05, mode=_lib.C_OVERWRITE), fb, PEAK_TFLOPS["bf16"])

        def ptr_tables(vouch):
            def make():
                a = (torch.randn(32, 1024, 1024, device=dev) * 0.05).bfloat16()
                b = (torch.randn(32, 1024, 1024, device=dev) * 0.05).bfloat16()
                c = torch.zeros(32, 1024, 1024, device=dev, dtype=torch.bfloat16)
                tab = torch.tensor([x[i].data_ptr() for x in (a, b, c) for i in range(32)], dtype=torch.int64, device=dev)
                d = _lib.GemmDesc()
                d.dtype, d.c_mode, d.m, d.k, d.n, d.batches = _lib.BFLOAT16, _lib.C_OVERWRITE, 1024, 1024, 1024, 32
                d.flags = _lib.GEMM_PTRS_ALIGNED16 if vouch else 0
                call = lambda: _lib.check(lib.ntg_gemm_ptrs_dev(ctypes.byref(d), tab.data_ptr(), tab.data_ptr() + 256, tab.data_ptr() + 512, stream))
                call.keep = (a, b, c, tab, d)
                return call
            return make
        run("batch_bf16_32x1024_pointer_tables_vouched", ptr_tables(True), fb, PEAK_TFLOPS["bf16"])
        run("batch_bf16_32x1024_pointer_tables", ptr_tables(False), fb, PEAK_TFLOPS["bf16"])
        # rows that are not 16-byte multiples: operands copied into zero-padded rows in the workspace, then the DMA-fed kernel
        # (A, whose rows of 4001 elements miss the rule, is copied; B, stored [k][n], is read where it lies and only its last k-rows are copied)
        run("c3_fp32_4096x4001x4096_padded_copies", G(torch.float32, N, 4001, N, mode=_lib.C_OVERWRITE), 2.0 * N * 4001 * N, PEAK_TFLOPS["fp32"])
        run("c3_bf16_4096x4001x4096_padded_copies", G(torch.bfloat16, N, 4001, N, scale=0.02, mode=_lib.C_OVERWRITE), 2.0 * N * 4001 * N, PEAK_TFLOPS["bf16"])
        fc = 2.0 * 200704 * 2304 * 256

        def conv_case(half, backward):
            def make():
                x = torch.randn(64, 256, 56, 56, device=dev)
                w = torch.randn(256, 256, 3, 3, device=dev) / 48.0
                g = torch.randn(64, 256, 56, 56, device=dev) if backward else None
                if half:
                    x, w, g = x.bfloat16(), w.bfloat16(), (g.bfloat16() if backward else None)
                if backward:
                    return lambda: F.conv2d_backward(x, w, g, padding=1)
                return lambda: F.conv2d(x, w, padding=1)
            return make

        run("c5a_conv2d_fp32", conv_case(False, False), fc, PEAK_TFLOPS["fp32"])
        run("c5a_conv2d_backward_fp32", conv_case(False, True), 2.0 * fc, PEAK_TFLOPS["fp32"])
        run("c5a_conv2d_bf16", conv_case(True, False), fc, PEAK_TFLOPS["bf16"])
        run("c5a_conv2d_backward_bf16", conv_case(True, True), 2.0 * fc, PEAK_TFLOPS["bf16"])
        skinny_bytes = 4.0 * (16 * 8192 + 8192 * 8192 + 2 * 16 * 8192)
        run("c5b_skinny_fp32_16x8192x8192", G(torch.float32, 16, 8192, 8192), skinny_bytes, PEAK_HBM_GBS, "GB/s", 1e9)

        # the host-pointer drop-in entry points (nt_matmult / nt_matmult_batch's signatures, operands in pageable host
        # memory): H2D of A, B and C (the accumulate contract makes C an input), the kernel, D2H of C -- wall clock
        import numpy as np
        vp = lambda x: x.ctypes.data_as(ctypes.c_void_p)

        def host_entry(name, m, k, n, batch, note, zero_c=False):
            """zero_c: C is zeroed before every call (outside the timed span) -- what functional::matmult hands to nt_matmult
            (zeros, then accumulate); otherwise every call accumulates onto the previous result, so C is uploaded too"""
            if only and name not in only:
                return
            rng = np.random.default_rng(7)
            ha = rng.standard_normal((batch, m, k)).astype(np.float32)
            hb = rng.standard_normal((batch, k, n)).astype(np.float32)
            hc = np.zeros((batch, m, n), np.float32)
            if batch == 1:
                call = lambda: _lib.check(lib.ntg_matmult(_lib.FLOAT32, vp(ha), vp(hb), vp(hc), m, k, k, n, 0, 0))
            else:
                arr = lambda x: (ctypes.c_void_p * batch)(*[x[i].ctypes.data for i in range(batch)])
                pa, pb, pc = arr(ha), arr(hb), arr(hc)
                call = lambda: _lib.check(lib.ntg_matmult_batch(_lib.FLOAT32, pa, pb, pc, batch, m, k, k, n, 0, 0))
            call(); call(); call()
            times, t_begin = [], time.perf_counter()
            while len(times) < 5 or (time.perf_counter() - t_begin < 0.3 and len(times) < 200):
                if zero_c:
                    hc.fill(0.0)
                t0 = time.perf_counter()
                call()
                times.append(time.perf_counter() - t0)
            # (the median: one call in fifty takes two to eight times as long -- page faults of the host process, not the path)
            ms = sorted(times)[len(times) // 2] * 1e3
            extras[name] = {"ms": round(ms, 4), "rate": round(2.0 * batch * m * k * n / (ms * 1e-3) / 1e12, 3), "unit": "TFLOP/s", "calls": len(times),
                            "mean_ms": round(sum(times) / len(times) * 1e3, 4), "note": note}

        host_entry("c1_fp32_512_host_pointer_entry", 512, 512, 512, 1, "ntg_matmult: 3 MiB host->device, 1 MiB device->host")
        host_entry("c3_fp32_4096_host_pointer_entry", N, N, N, 1, "ntg_matmult: 192 MiB host->device, 64 MiB device->host")
        host_entry("c3_fp32_4096_host_pointer_entry_zero_c", N, N, N, 1, "ntg_matmult on a zeroed C (functional::matmult's call): C is found to be zeros "
                   "and not uploaded, 128 MiB host->device, 64 MiB device->host", zero_c=True)
        host_entry("c2a_fp32_b32_host_pointer_entry", 1024, 768, 1024, 32, "ntg_matmult_batch, 32 items: 320 MiB host->device, 128 MiB device->host")
        host_entry("c2a_fp32_b32_host_pointer_entry_zero_c", 1024, 768, 1024, 32, "ntg_matmult_batch, 32 items, zeroed C: 192 MiB host->device, "
                   "128 MiB device->host", zero_c=True)
        lib.ntg_release_host_buffers()
    if extras:
        out["extras"] = extras
    if args.context:
        out["context"] = context_table(torch, F, _lib, lib, dev, stream, make_gemm, settle)
    if args.shapes:
        dts = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32, "fp64": torch.float64}
        res = {}
        for spec in [x for x in args.shapes.split(",") if x]:
            parts = spec.split(":")
            m, k, n = (int(v) for v in parts[1].split("x"))
            form = parts[2] if len(parts) > 2 else "nn"
            fn = make_gemm(dts[parts[0]], m, k, n, ta=form[0] == "t", tb=form[1] == "t", scale=0.02 if parts[0] in ("bf16", "fp16") else 1.0,
                           mode=_lib.C_OVERWRITE)
            settle(spec)
            steps = max(args.steps, int(0.01 / max(2.0 * m * k * n / 1.0e15, 1e-6)))       # about 10 ms of launches
            _, ev_ms = time_steps(fn, steps, args.warmup)
            res[spec] = {"us": round(ev_ms * 1e3, 2), "TFLOP/s": round(2.0 * m * k * n / (ev_ms * 1e-3) / 1e12, 1), "timed_launches": steps}
            del fn
        out["shapes"] = res
    if only:
        print(json.dumps(out))
        return

    # ---------------- CPU baseline: the oracle's restatement of the reference loop nest ----------------
    if not args.no_cpu:
        import numpy as np

        import oracle
        threads = oracle.lib().oracle_tiled_threads(0)
        rng = np.random.default_rng(1003)
        a = rng.standard_normal((N, N)).astype(np.float32)
        b = rng.standard_normal((N, N)).astype(np.float32)
        c = np.zeros((N, N), np.float32)
        oracle.matmult2d(a[:256], b, np.zeros((256, N), np.float32), kind="tiled")     # warm the pool
        reps, t_cpu = 0, 0.0
        while reps < 1 or (t_cpu < 10.0 and reps < 8):
            t0 = time.perf_counter()
            oracle.matmult2d(a, b, c, kind="tiled")
            t_cpu += time.perf_counter() - t0
            reps += 1
        out["cpu_baseline"] = {
            "value": round(flops * reps / t_cpu / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"Float32 4096x4096x4096, {reps} pass(es) of the tiled/packed k-outer restatement "
                      f"(tile 16, pack block 7056, thread cap 21 -> {threads} threads); the reference has no BFloat16",
        }

        # the same restatement on the other CPU-runnable configurations (one or a few passes each)
        def cpu_time(fn, min_s=0.5, max_reps=20):
            fn()
            n, t = 0, 0.0
            while n < 1 or (t < min_s and n < max_reps):
                t0 = time.perf_counter()
                fn()
                t += time.perf_counter() - t0
                n += 1
            return t / n

        others = {}
        a1 = rng.standard_normal((512, 512)).astype(np.float32)
        b1 = rng.standard_normal((512, 512)).astype(np.float32)
        c1 = np.zeros((512, 512), np.float32)
        t = cpu_time(lambda: oracle.matmult2d(a1, b1, c1, kind="tiled"))
        others["c1_fp32_512"] = {"ms": round(t * 1e3, 3), "rate": round(2.0 * 512 ** 3 / t / 1e12, 4), "unit": "TFLOP/s"}
        a2 = rng.standard_normal((4, 1024, 768)).astype(np.float32)
        b2 = rng.standard_normal((4, 768, 1024)).astype(np.float32)
        t = cpu_time(lambda: oracle.matmult(a2, b2, kind="tiled"), max_reps=3)
        others["c2a_fp32_1024x768x1024_per_item"] = {"ms": round(t / 4 * 1e3, 3), "rate": round(2.0 * 4 * 1024 * 768 * 1024 / t / 1e12, 4),
                                                     "unit": "TFLOP/s", "sample": "4 of the 32 batch items (the reference runs items serially)"}
        a5 = rng.standard_normal((16, 8192)).astype(np.float32)
        b5 = rng.standard_normal((8192, 8192)).astype(np.float32)
        c5 = np.zeros((16, 8192), np.float32)
        t = cpu_time(lambda: oracle.matmult2d(a5, b5, c5, kind="tiled"), max_reps=5)
        others["c5b_skinny_fp32_16x8192x8192"] = {"ms": round(t * 1e3, 3), "rate": round(4.0 * (16 * 8192 + 8192 * 8192 + 2 * 16 * 8192) / t / 1e9, 2),
                                                  "unit": "GB/s"}
        out["cpu_baseline"]["others"] = others

    print(json.dumps(out))


if __name__ == "__main__":
    main()
