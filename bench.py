#!/usr/bin/env python3
"""bench.py — the Linear2D per-rank block GEMM on one MI355X, next to the CPU path.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one pass of the hot path over one batch of synthetic input: rank
(0, 1) of a q = 2 SUMMA grid computing
    out[8192, 2048] = GeLU_tanh(A_0 B_0 + A_1 B_1 + bias)        (bf16, fp32 accumulation)
with the operands a row/column broadcast would deliver already resident in HBM
(the benchmark definition's second configuration; 137,438,953,472 FLOP per step). One step is one call
of cw_gemm_ksteps through the C ABI = one kernel launch.

Prints ONE JSON line. `value` is TFLOP/s over the timed region (wall clock
around K steps, synchronised on both sides). `roofline` prices the GEMM kernel
against the MI355X dense bf16 MFMA peak with the average launch duration from
HIP events on the launch stream over a SUSTAINED run (--sustained launches back
to back, 10000 by default, more than a second: a short run finds the board below
its power limit and the clock high; the figure from the K timed steps is
reported beside it), together with the shader
clock and the socket power read from the driver's sysfs files during that run.
`aux` reports the bandwidth-bound kernels of
the same path (LayerNorm2D, vocab-parallel CE: the third and fourth configurations)
against the 8 TB/s HBM peak, on buffers rotated through > 512 MiB so that the
256 MiB Infinity Cache cannot serve them. `cpu_baseline` times the reference's
CPU path (torch, gloo, world size 1) restated by oracle/ on the host cores, on
a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

MFMA_BF16_PEAK_TFLOPS = 2516.6  # 256 CU x 2.4 GHz x 4096 FLOP/clk/CU, dense
HBM_PEAK_GBPS = 8000.0

M, N, K, STEPS_K = 8192, 2048, 2048, 2
GEMM_FLOP = 2 * M * N * K * STEPS_K


class SmiSampler:
    """Shader clock and socket power of card 0 from the amdgpu driver's sysfs files, sampled by a thread
    while the caller runs its timed loop. The driver reports low-pass filtered values (they settle within
    about a second), so the figures kept are those of the last 40 % of the sampled interval."""

    def __init__(self, period_s=0.002, metrics=None):
        import glob
        self.period = period_s
        self.metrics = metrics if metrics is not None and metrics.handle is not None else None
        self.tables = []   # distinct gpu_metrics tables seen during the run (one reading every 50 ms)
        dev = "/sys/class/drm/card0/device"
        hw = sorted(glob.glob(dev + "/hwmon/hwmon*"))
        self.power_path = hw[0] + "/power1_input" if hw and os.path.exists(hw[0] + "/power1_input") else None
        self.cap_path = hw[0] + "/power1_cap" if hw and os.path.exists(hw[0] + "/power1_cap") else None
        self.sclk_path = dev + "/pp_dpm_sclk" if os.path.exists(dev + "/pp_dpm_sclk") else None
        self.samples = []
        self._stop = False
        self._thread = None

    def available(self):
        return (self.power_path is not None and self.sclk_path is not None) or self.metrics is not None

    def _read(self):
        if self.power_path is None or self.sclk_path is None:
            raise OSError("no sysfs power / clock files")
        with open(self.power_path) as f:
            watts = int(f.read()) / 1e6
        mhz = None
        with open(self.sclk_path) as f:
            for line in f:
                if line.rstrip().endswith("*"):  # the level the shader clock is at now
                    mhz = float(line.split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
        return watts, mhz

    def _run(self):
        next_table = 0.0
        while not self._stop:
            try:
                w, m = self._read()
                self.samples.append((time.perf_counter(), w, m))
            except (OSError, ValueError, IndexError):
                pass
            if self.metrics is not None and time.perf_counter() >= next_table:
                tab = self.metrics.read()
                if tab is not None and (not self.tables or tab["firmware_timestamp"] != self.tables[-1]["firmware_timestamp"]):
                    self.tables.append(tab)
                next_table = time.perf_counter() + 0.05
            time.sleep(self.period)

    def __enter__(self):
        if self.available():
            import threading
            self._thread = threading.Thread(target=self._run, daemon=True)
            self._thread.start()
        self.t0 = time.perf_counter()
        return self

    def __exit__(self, *exc):
        self.t1 = time.perf_counter()
        self._stop = True
        if self._thread is not None:
            self._thread.join()

    def summary(self):
        if not self.samples:
            return None
        lo = self.t0 + 0.6 * (self.t1 - self.t0)
        tail = [s for s in self.samples if lo <= s[0] <= self.t1 and s[2] is not None]
        if not tail:
            return None
        out = {"shader_clock_MHz": round(sum(s[2] for s in tail) / len(tail), 1),
               "socket_power_W": round(sum(s[1] for s in tail) / len(tail), 1),
               "samples": len(tail), "source": "sysfs pp_dpm_sclk / hwmon power1_input, last 40% of the run"}
        if self.cap_path:
            try:
                with open(self.cap_path) as f:
                    out["power_cap_W"] = int(f.read()) / 1e6
            except (OSError, ValueError):
                pass
        return out


class GpuMetrics:
    """The driver's gpu_metrics table of GPU 0 through ROCm's amdsmi binding (shipped under /opt/rocm): the
    socket energy accumulator (15.259 uJ units), the firmware's own timestamp (10 ns units) and its residency
    counters of the limiters (package power, PROCHOT, socket / regulator / HBM temperature: one count per
    millisecond in which the limiter held the clock down). The firmware refreshes the table about once a second,
    so only differences between two DISTINCT tables mean anything, and only tables whose whole period lies inside
    the interval of interest describe it. Everything is optional: without the binding the fields are left out."""

    FIELDS = ("energy_accumulator", "firmware_timestamp", "accumulation_counter", "ppt_residency_acc",
              "prochot_residency_acc", "socket_thm_residency_acc", "vr_thm_residency_acc", "hbm_thm_residency_acc")
    LIMITERS = (("package_power_ppt", "ppt_residency_acc"), ("prochot", "prochot_residency_acc"),
                ("socket_thermal", "socket_thm_residency_acc"), ("regulator_thermal", "vr_thm_residency_acc"),
                ("hbm_thermal", "hbm_thm_residency_acc"))
    REFRESH_S = 1.0

    def __init__(self):
        self.handle = None
        try:
            if "/opt/rocm/share/amd_smi" not in sys.path:
                sys.path.append("/opt/rocm/share/amd_smi")
            import amdsmi
            self.amdsmi = amdsmi
            amdsmi.amdsmi_init()
            self.handle = amdsmi.amdsmi_get_processor_handles()[0]
            if self.read() is None:
                self.handle = None
        except Exception:  # no binding, no permission, another table revision
            self.handle = None

    def read(self):
        if self.handle is None:
            return None
        try:
            m = self.amdsmi.amdsmi_get_gpu_metrics_info(self.handle)
        except Exception:
            return None
        out = {k: m.get(k) for k in self.FIELDS}
        if not all(isinstance(out[k], int) for k in ("energy_accumulator", "firmware_timestamp")):
            return None
        out["t"] = time.perf_counter()
        out["xcd_clocks_MHz"] = m.get("current_gfxclks")
        return out

    @classmethod
    def window(cls, tables, t0, t1, launch_us=None):
        """tables: distinct readings (by firmware timestamp) taken while a kernel ran back to back from host time
        t0 to t1 (each is seen within 50 ms of its refresh). Uses the first and the last table refreshed inside
        the run, after a margin for the clock to settle: average socket power from the energy counter over the firmware's own clock, the share of the
        firmware's samples in which each limiter was active, and, given the launch duration, energy per launch."""
        inside = [m for m in tables if t0 + 0.4 <= m["t"] <= t1]
        if len(inside) < 2:
            return {"note": "the run was too short for two refreshes of the firmware's table (about one a second)"}
        a, b = inside[0], inside[-1]
        dt = (b["firmware_timestamp"] - a["firmware_timestamp"]) * 1e-8
        if dt <= 0:
            return None
        watts = (b["energy_accumulator"] - a["energy_accumulator"]) * 15.259e-6 / dt
        out = {"socket_power_W_from_energy_counter": round(watts, 1), "window_s": round(dt, 3), "tables": len(inside)}
        if launch_us:
            out["energy_mJ_per_launch"] = round(watts * launch_us * 1e-3, 2)
        n = (b["accumulation_counter"] - a["accumulation_counter"]) if isinstance(a.get("accumulation_counter"), int) else 0
        if n > 0:
            out["limiter_residency"] = {name: round((b[key] - a[key]) / n, 4) for name, key in cls.LIMITERS
                                        if isinstance(a.get(key), int) and isinstance(b.get(key), int)}
        if b.get("xcd_clocks_MHz"):
            clk = [c for c in b["xcd_clocks_MHz"] if isinstance(c, int)]
            if clk:
                out["xcd_clocks_MHz"] = clk
        return out


_GPU_METRICS = None


def gpu_metrics():
    global _GPU_METRICS
    if _GPU_METRICS is None:
        _GPU_METRICS = GpuMetrics()
    return _GPU_METRICS


def sustained_us(fn, launches):
    """Average duration of fn() over `launches` back-to-back calls (events on the current stream), with the
    clock and power the driver reports while they run and, when the run is long enough for the firmware's
    table to refresh twice inside it, the socket energy counter and the limiters' residencies."""
    import torch
    for _ in range(20):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with SmiSampler(metrics=gpu_metrics()) as smi:
        e0.record()
        for _ in range(launches):
            fn()
        e1.record()
        torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / launches
    summary = smi.summary()
    if smi.tables:
        w = GpuMetrics.window(smi.tables, smi.t0, smi.t1, us)
        if w is not None:
            summary = dict(summary or {})
            summary["gpu_metrics"] = w
    return us, summary


def measured_traffic():
    """Bytes per launch that cross the L2 <-> fabric boundary for the GEMM kernel, from the committed
    hardware-counter summary (two rocprofv3 --pmc runs of this script, scaled by a plain copy of known
    size); None when the summary is not there."""
    import re
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles",
                        "gemm_bf16_dma_kernel_linear2d_q2_counters.txt")
    try:
        with open(path) as f:
            m = re.search(r"^traffic_bytes_per_launch:\s*(\d+)", f.read(), re.M)
        return int(m.group(1)) if m else None
    except OSError:
        return None


def _seeded(shape, seed, std, dtype):
    import torch
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)


def make_gemm_inputs(n_sets, device):
    """Seeded synthetic operands: A_i ~ N(0,1), B_i ~ N(0,0.02), bias ~ N(0,0.02), generated on the
    CPU, rounded to bf16, then copied to the device."""
    import torch
    sets = []
    for s in range(n_sets):
        A = [_seeded((M, K), 1000 * s + i, 1.0, torch.bfloat16).to(device) for i in range(STEPS_K)]
        B = [_seeded((K, N), 1000 * s + 10 + i, 0.02, torch.bfloat16).to(device) for i in range(STEPS_K)]
        sets.append((A, B))
    bias = _seeded((N,), 7, 0.02, torch.bfloat16).to(device)
    return sets, bias


def graph_time_us(fn, calls, replays=3, min_ms=100.0):
    """Average duration of one fn() call when `calls` of them are replayed from
    a HIP graph: the host cost of the Python wrappers (tens of microseconds,
    more than these kernels run) stays outside the timed region, which is
    bracketed by events on the replay stream."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(calls):
            fn()
    graph.replay()
    torch.cuda.synchronize()

    def timed(n):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (n * calls)

    pilot = timed(replays)
    n = int(min_ms * 1e3 / max(pilot * calls, 1.0)) + 1  # replays for min_ms of work: the rate the chip sustains
    return timed(n) if n > replays else pilot


def bench_bandwidth_kernels(device, parts=("ln", "ln_wide", "ce")):
    """LayerNorm2D (config 3) and vocab-parallel CE (config 4) kernels: algorithmic
    bytes per launch / average launch duration. Each call below is one C-ABI
    entry point; the launches are replayed from a HIP graph. The LayerNorm2D
    backward is timed as the layers run it: cw_ln_bwd_partials_open (one launch,
    leaves the column sums as partial rows) and cw_ln_bwd_dx_close (one launch
    whose leading workgroups finish them); cw_ln_bwd_partials with its own
    finalize launch is kept beside them as ln_bwd_partials_two_launches."""
    import torch
    from cubework_amd import ops

    out = {}
    R, C, H = 16384, 1024, 2048
    nb = 17  # 17 x 32 MiB = 544 MiB of distinct activations
    xs = [_seeded((R, C), 100 + i, 1.0, torch.bfloat16).to(device) for i in range(nb)]
    dys = [_seeded((R, C), 200 + i, 1.0, torch.bfloat16).to(device) for i in range(nb)]
    g = torch.Generator().manual_seed(3)
    gamma = (torch.rand(C, generator=g) * 0.2 + 0.9).to(torch.bfloat16).to(device)
    beta = _seeded((C,), 4, 0.02, torch.bfloat16).to(device)
    peer = _seeded((R, C), 5, 1.0, torch.bfloat16).to(device)
    stats = ops.ln_partial_stats(xs[0]) + ops.ln_partial_stats(peer)
    _, mr = ops.ln_normalize(xs[0], stats, H, 1e-5, gamma, beta)
    rs, pending = ops.ln_bwd_partials_open(dys[0], xs[0], mr, gamma)
    rs = rs * 2
    mr_whole = ops.ln_forward_fused(xs[0], 1e-5, gamma, beta)[1]  # the same rows taken as whole (H = 1024)
    i = [0]

    def rot(lst):
        i[0] += 1
        return lst[i[0] % len(lst)]

    cases = [
        ("ln_partial_stats", 33554432 + 131072, lambda: ops.ln_partial_stats(rot(xs))),
        ("ln_normalize", 2 * 33554432 + 2 * 131072 + 4096, lambda: ops.ln_normalize(rot(xs), stats, H, 1e-5, gamma, beta)),
        ("ln_bwd_partials", 2 * 33554432 + 2 * 131072 + 8192,
         lambda: ops.ln_bwd_partials_open(rot(dys), xs[i[0] % nb], mr, gamma)),
        ("ln_bwd_dx", 3 * 33554432 + 2 * 131072 + 2048 + 8192,
         lambda: ops.ln_bwd_dx_close(rot(dys), xs[i[0] % nb], mr, rs, H, pending, gamma)),
        ("ln_bwd_partials_two_launches", 2 * 33554432 + 2 * 131072 + 8192,
         lambda: ops.ln_bwd_partials(rot(dys), xs[i[0] % nb], mr, gamma)),
        # rows complete on the rank (tensor-parallel size 1): partials + dx in one pass, dy and x read once
        ("ln_backward_fused", 3 * 33554432 + 2 * 131072 + 8192,
         lambda: ops.ln_backward_fused(rot(dys), xs[i[0] % nb], mr_whole, gamma)),
    ]
    for name, nbytes, fn in cases if "ln" in parts else ():
        us = graph_time_us(fn, 2 * nb)
        out[name] = {"us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1), "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 3),
                     "bytes": nbytes}
    del xs, dys
    if "ln_wide" not in parts and "ce" not in parts:
        return out
    # wide rows held whole by the rank: the fp32 residual stream under autocast (hidden 2048 and 4096) and a
    # 16-bit hidden size of 4096; fused forward (x read, y written) and fused backward (dy, x read, dx written)
    for tag, Rw, Cw, dt in (("fp32_8192x2048", 8192, 2048, torch.float32), ("fp32_4096x4096", 4096, 4096, torch.float32),
                            ("bf16_8192x4096", 8192, 4096, torch.bfloat16)) if "ln_wide" in parts else ():
        nw = 6
        es = 4 if dt == torch.float32 else 2
        xw = [_seeded((Rw, Cw), 400 + k, 1.0, dt).to(device) for k in range(nw)]
        dw = [_seeded((Rw, Cw), 500 + k, 1.0, dt).to(device) for k in range(nw)]
        gw = torch.ones(Cw, dtype=dt, device=device)
        bw = torch.zeros(Cw, dtype=dt, device=device)
        mrw = ops.ln_forward_fused(xw[0], 1e-5, gw, bw)[1]
        for name, nbytes, fn in (
                ("ln_forward_fused_" + tag, 2 * Rw * Cw * es + 2 * Cw * es + 8 * Rw,
                 lambda: ops.ln_forward_fused(rot(xw), 1e-5, gw, bw)),
                ("ln_backward_fused_" + tag, 3 * Rw * Cw * es + Cw * es + 8 * Rw + 8 * Cw,
                 lambda: ops.ln_backward_fused(rot(dw), xw[i[0] % nw], mrw, gw))):
            us = graph_time_us(fn, 2 * nw)
            out[name] = {"us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1),
                         "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 3), "bytes": nbytes}
        del xw, dw
    if "ce" not in parts:
        return out
    T, V, V0 = 8192, 12568, 12568
    lg = [_seeded((T, V), 300 + k, 2.0, torch.bfloat16).to(device) for k in range(3)]  # 3 x 196 MiB
    tg = torch.randint(0, 50272, (T,), generator=torch.Generator().manual_seed(9)).to(device)
    st = ops.vpce_fwd_local(lg[0], tg, V0)
    loss, gmax, gsum = ops.vpce_finalize(*(s.unsqueeze(0) for s in st))
    cases = [
        ("vpce_fwd_local", T * V * 2 + T * 8 + 4 * T * 4, lambda: ops.vpce_fwd_local(rot(lg), tg, V0)),
        ("vpce_bwd_bf16_grad", 2 * T * V * 2 + T * 8 + 2 * T * 4, lambda: ops.vpce_bwd(rot(lg), tg, V0, gmax, gsum, None, 1.0 / T)),
        ("vpce_bwd_fp32_grad", T * V * 2 + T * V * 4 + T * 8 + 2 * T * 4,
         lambda: ops.vpce_bwd(rot(lg), tg, V0, gmax, gsum, None, 1.0 / T, grad_dtype=torch.float32)),
    ]
    for name, nbytes, fn in cases:
        us = graph_time_us(fn, 6)
        out[name] = {"us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1), "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 3),
                     "bytes": nbytes}
    return out


def event_time_us(fn, iters, warmup, min_ms=150.0):
    """Average duration of fn() per call from events on the current stream. A first pass of `iters` calls is a
    pilot; the figure comes from a second pass long enough (min_ms) for the clock to have settled - a burst of 30
    launches right after host-side set-up still runs on a chip that is waking up."""
    import torch

    def timed(n):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / n

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    pilot = timed(iters)
    n = int(min_ms * 1e3 / max(pilot, 1.0)) + 1
    return timed(n) if n > iters else pilot


class AbiCallTimer:
    """Stands in for the loaded library during one instrumented pass: every C-ABI compute call is bracketed by two
    events on the launch stream, so that each entry point's device time inside a composite step (the OPT-shaped
    block) can be told apart. The events stretch the step; the step's own time is measured without them."""

    # entry point -> (what the call's work is priced in, function of the call's arguments giving FLOP or bytes)
    @staticmethod
    def _es(code):
        return 4 if code == 1 else 2

    def __init__(self, lib):
        self._lib = lib
        self.records = []   # (name, shape text, kind, work, ev0, ev1)

    def _work(self, name, a):
        es = self._es
        if name in ("cw_gemm_ksteps_ws", "cw_gemm_ksteps"):
            lay, m, n, k, steps = a[0], a[1], a[2], a[3], a[4]
            return ("%s %dx%dx%d" % ("NN NT TN".split()[lay], m, n, k * max(steps, 1)), "flop", 2.0 * m * n * k * steps)
        if name == "cw_attn_fwd":
            b, h, s, d, causal = a[0], a[1], a[2], a[3], a[11]
            return ("b%d h%d s%d d%d" % (b, h, s, d), "flop", 4.0 * b * h * s * s * d / (2 if causal else 1))
        if name == "cw_attn_bwd":
            b, h, s, d, causal = a[0], a[1], a[2], a[3], a[17]
            return ("b%d h%d s%d d%d" % (b, h, s, d), "flop", 10.0 * b * h * s * s * d / (2 if causal else 1))
        if name == "cw_ln_forward_fused":
            return ("%dx%d" % (a[0], a[1]), "bytes", 2.0 * a[0] * a[1] * es(a[11]))
        if name == "cw_ln_backward_fused":
            return ("%dx%d" % (a[0], a[1]), "bytes", (4.0 if a[11] else 3.0) * a[0] * a[1] * es(a[18]))
        if name == "cw_colsum":
            return ("%dx%d" % (a[0], a[1]), "bytes", 1.0 * a[0] * a[1] * es(a[8]))
        if name == "cw_act_bwd_colsum":
            return ("%dx%d" % (a[1], a[2]), "bytes", 3.0 * a[1] * a[2] * es(a[13]))
        return ("", None, 0.0)

    def __getattr__(self, name):
        fn = getattr(self._lib, name)
        if not name.startswith("cw_") or name.endswith("_bytes") or name.endswith("_supported") or name in (
                "cw_version", "cw_device_arch", "cw_last_error"):
            return fn

        def timed(*args):
            import torch
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            rc = fn(*args)
            e1.record()
            shape, kind, work = self._work(name, args)
            self.records.append((name, shape, kind, work, e0, e1))
            return rc
        return timed

    def table(self, passes, step_us):
        """Per (entry point, shape): calls per step, device time per step, share of the step, and the fraction of
        the call's own roofline (dense bf16 MFMA peak for FLOP, 8 TB/s for bytes)."""
        rows = {}
        for name, shape, kind, work, e0, e1 in self.records:
            r = rows.setdefault((name, shape), {"entry_point": name, "shape": shape, "calls": 0, "us": 0.0, "kind": kind, "work": work})
            r["calls"] += 1
            r["us"] += e0.elapsed_time(e1) * 1e3
        out = []
        for r in sorted(rows.values(), key=lambda r: -r["us"]):
            calls = r["calls"] / passes
            us = r["us"] / passes
            row = {"entry_point": r["entry_point"], "shape": r["shape"], "calls_per_step": round(calls, 2),
                   "us_per_step": round(us, 1), "share_of_step": round(us / step_us, 4)}
            per_call = us / max(calls, 1e-9)
            if r["kind"] == "flop":
                row["frac_of_mfma_peak"] = round(r["work"] / per_call / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)
            elif r["kind"] == "bytes":
                row["frac_of_hbm_peak"] = round(r["work"] / per_call / 1e3 / HBM_PEAK_GBPS, 4)
            out.append(row)
        return out


def bench_other_configs(device, sets):
    """The other GEMM orientations at config 2's FLOP count (the backward products of the same layer),
    config 1's fp32 forward GEMM, and one OPT-1.3B-shaped block (config 5) forward+backward."""
    import torch
    from cubework_amd import ops
    from cubework_amd.distributed import initialize
    from cubework_amd.opt_block import OPTBlock

    out = {}
    n_sets = len(sets)
    i = [0]

    def rot():
        i[0] += 1
        return sets[i[0] % n_sets]

    # dX = sum_i dY_i W_i^T (NT): A_i [8192,2048], B_i [2048,2048] read as [N,K]
    dx = torch.empty((M, N), dtype=torch.bfloat16, device=device)
    us = event_time_us(lambda: ops.gemm_ksteps("NT", *rot(), out=dx), 50, 10)
    out["gemm_nt_dX"] = {"us": round(us, 2), "TFLOPs": round(GEMM_FLOP / us / 1e6, 1),
                         "frac": round(GEMM_FLOP / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
    # dW = sum_i X_i^T dY_i (TN): A_i [8192,2048] read as [K,M], B_i [8192,2048] -> [2048,2048], k = 2 x 8192
    dw = torch.empty((K, N), dtype=torch.bfloat16, device=device)

    def tn():
        a, _ = rot()
        b, _ = rot()
        ops.gemm_ksteps("TN", a, b, out=dw)
    us = event_time_us(tn, 50, 10)
    out["gemm_tn_dW_splitk"] = {"us": round(us, 2), "TFLOPs": round(GEMM_FLOP / us / 1e6, 1),
                                "frac": round(GEMM_FLOP / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
    # Vendor anchor, outside the product path: torch.matmul (hipBLASLt) beside cw_gemm_ksteps on the same operands,
    # without bias or activation on either side - config 2's product with its two k-steps concatenated
    # ([8192,4096] x [4096,2048], operands rotated like the headline's) and one 8192^3 product.
    cat_sets = [(torch.cat(a, dim=1), torch.cat(b, dim=0)) for a, b in sets]
    o_cat = torch.empty((M, N), dtype=torch.bfloat16, device=device)
    c_ = [0]

    def rot_cat():
        c_[0] += 1
        return cat_sets[c_[0] % n_sets]
    anchor = {}
    for name, fn in (("cw_gemm_ksteps", lambda: ops.gemm_ksteps("NN", *[[t] for t in rot_cat()], out=o_cat)),
                     ("torch_matmul", lambda: torch.matmul(*rot_cat(), out=o_cat))):
        us = event_time_us(fn, 50, 10)
        anchor[name] = {"us": round(us, 2), "TFLOPs": round(GEMM_FLOP / us / 1e6, 1),
                        "frac": round(GEMM_FLOP / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
    out["vendor_anchor_config2_concatenated_8192x2048x4096"] = anchor
    del cat_sets, o_cat
    big = [(_seeded((8192, 8192), 60 + 2 * j_, 1.0, torch.bfloat16).to(device),
            _seeded((8192, 8192), 61 + 2 * j_, 0.02, torch.bfloat16).to(device)) for j_ in range(2)]
    o_big = torch.empty((8192, 8192), dtype=torch.bfloat16, device=device)
    flop_big = 2.0 * 8192 ** 3

    def rot_big():
        c_[0] += 1
        return big[c_[0] % 2]
    anchor = {}
    for name, fn in (("cw_gemm_ksteps", lambda: ops.gemm_ksteps("NN", *[[t] for t in rot_big()], out=o_big)),
                     ("torch_matmul", lambda: torch.matmul(*rot_big(), out=o_big))):
        us = event_time_us(fn, 10, 3)
        anchor[name] = {"us": round(us, 2), "TFLOPs": round(flop_big / us / 1e6, 1),
                        "frac": round(flop_big / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
    anchor["note"] = ("torch.matmul is the vendor library (hipBLASLt) on the same bf16 operands in the same process: a "
                      "comparison line only, nothing on the product path calls it")
    out["vendor_anchor_8192x8192x8192"] = anchor
    del big, o_big
    # the four weight-gradient products of the OPT-1.3B-shaped block (config 5): dW = X^T dY over 8192 tokens (TN),
    # [in, out] = qkv 2048 x 6144 (192 tiles of 256 x 256: three quarters of the compute units), out 2048 x 2048
    # (64 tiles: split along k), fc1 2048 x 8192 and fc2 8192 x 2048 (256 tiles each)
    tok = 8192
    x_in = {2048: _seeded((tok, 2048), 71, 1.0, torch.bfloat16).to(device), 8192: _seeded((tok, 8192), 72, 1.0, torch.bfloat16).to(device)}
    dy_out = {n_: _seeded((tok, n_), 73 + k_, 1.0, torch.bfloat16).to(device) for k_, n_ in enumerate((2048, 6144, 8192))}
    for name, k_in, n_out in (("qkv_2048x6144", 2048, 6144), ("out_2048x2048", 2048, 2048), ("fc1_2048x8192", 2048, 8192),
                              ("fc2_8192x2048", 8192, 2048)):
        xa, dya = x_in[k_in], dy_out[n_out]
        flop = 2.0 * tok * k_in * n_out
        us = event_time_us(lambda: ops.gemm_ksteps("TN", [xa], [dya]), 20, 5)
        out["config5_dW_" + name] = {"us": round(us, 2), "TFLOPs": round(flop / us / 1e6, 1),
                                     "frac": round(flop / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
                                     "tiles_256": (k_in // 256) * (n_out // 256)}
    del x_in, dy_out
    # config 2's product with float16 operands (what a plain torch.autocast hands the GEMM-type operators):
    # the same kernel with the other MFMA opcode and conversion
    a16 = [t.to(torch.float16) for t in sets[0][0]]
    b16 = [t.to(torch.float16) for t in sets[0][1]]
    o16 = torch.empty((M, N), dtype=torch.float16, device=device)
    us = event_time_us(lambda: ops.gemm_ksteps("NN", a16, b16, out=o16), 50, 10)
    out["gemm_nn_float16"] = {"us": round(us, 2), "TFLOPs": round(GEMM_FLOP / us / 1e6, 1),
                              "frac": round(GEMM_FLOP / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
    del a16, b16, o16
    # vocabulary-slice classifier of the OPT-1.3B-shaped model (one rank of four: 12568 of 50272 classes):
    # logits = x W^T, and the two gradients. 12568 is not a tile multiple: it is N, M and K in turn.
    xc = _seeded((8192, 2048), 51, 1.0, torch.bfloat16).to(device)
    wc = _seeded((12568, 2048), 52, 0.02, torch.bfloat16).to(device)
    dcl = _seeded((8192, 12568), 53, 1.0, torch.bfloat16).to(device)
    cls_flop = 2.0 * 8192 * 12568 * 2048
    for name, fn in (("classifier_logits_nt", lambda: ops.gemm_ksteps("NT", [xc], [wc])),
                     ("classifier_dW_tn", lambda: ops.gemm_ksteps("TN", [dcl], [xc])),
                     ("classifier_dX_nn", lambda: ops.gemm_ksteps("NN", [dcl], [wc]))):
        us = event_time_us(fn, 10, 3)
        out[name] = {"us": round(us, 2), "TFLOPs": round(cls_flop / us / 1e6, 1),
                     "frac": round(cls_flop / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
    del xc, wc, dcl
    # config 1 forward: x [4096,1024] fp32, W [4096,1024] fp32 (NT), fp32 MFMA
    x1 = _seeded((4096, 1024), 1, 1.0, torch.float32).to(device)
    w1 = ((torch.rand((4096, 1024), generator=torch.Generator().manual_seed(2)) * 2 - 1) * (6.0 / 5120) ** 0.5).to(device)
    b1 = torch.zeros(4096, dtype=torch.float32, device=device)
    o1 = torch.empty((4096, 4096), dtype=torch.float32, device=device)
    us = event_time_us(lambda: ops.gemm_ksteps("NT", [x1], [w1], b1, None, out=o1), 30, 5)
    flop1 = 2.0 * 4096 * 1024 * 4096
    out["linear1d_fp32_fwd"] = {"us": round(us, 2), "TFLOPs": round(flop1 / us / 1e6, 1),
                                "frac_fp32_mfma": round(flop1 / us / 1e6 / 157.3, 4)}
    # config 1 backward: dX = dY W (NN, [4096,4096] x [4096,1024]) and dW = dY^T X (TN), the same FLOP each
    dy1 = _seeded((4096, 4096), 3, 1.0, torch.float32).to(device)
    for name, fn in (("linear1d_fp32_dX", lambda: ops.gemm_ksteps("NN", [dy1], [w1])),
                     ("linear1d_fp32_dW", lambda: ops.gemm_ksteps("TN", [dy1], [x1]))):
        us = event_time_us(fn, 30, 5)
        out[name] = {"us": round(us, 2), "TFLOPs": round(flop1 / us / 1e6, 1),
                     "frac_fp32_mfma": round(flop1 / us / 1e6 / 157.3, 4)}
    del dy1
    # vocab-parallel embedding (rank 1 of 4 of OPT's 50272 x 2048 table, 8192 tokens): bytes = ids + the rows
    # actually read (about a quarter of the tokens are live) + the output written
    e_tok, e_dim, e_vloc = 8192, 2048, 12568
    ids = torch.randint(0, 50272, (e_tok,), generator=torch.Generator().manual_seed(31)).to(device)
    tabs = [_seeded((e_vloc, e_dim), 32 + j, 0.02, torch.bfloat16).to(device) for j in range(6)]  # 6 x 49 MiB
    live = int(((ids >= e_vloc) & (ids < 2 * e_vloc)).sum().item())
    j = [0]

    def emb_fwd():
        j[0] += 1
        ops.embedding_fwd(ids, tabs[j[0] % 6], e_vloc)
    us = graph_time_us(emb_fwd, 12)  # replayed from a HIP graph: the wrapper's host time exceeds the kernel's
    nbytes = e_tok * 8 + live * e_dim * 2 + e_tok * e_dim * 2
    out["vocab_embedding_fwd"] = {"us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1), "bytes": nbytes,
                                  "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 3)}
    dys_e = [_seeded((e_tok, e_dim), 40 + j_, 1.0, torch.bfloat16).to(device) for j_ in range(4)]
    def emb_bwd():
        j[0] += 1
        ops.embedding_bwd(ids, dys_e[j[0] % 4], e_vloc, e_vloc)
    us = graph_time_us(emb_bwd, 8)
    nbytes = e_tok * 8 + live * e_dim * 2 + e_vloc * e_dim * 2
    out["vocab_embedding_bwd"] = {"us": round(us, 2), "GBps": round(nbytes / us / 1e3, 1), "bytes": nbytes,
                                  "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 3),
                                  "note": "one launch from the unsorted ids (cw_embed_bwd_ids): sums and the zeros of the rows without tokens"}
    del tabs, dys_e
    # attention core of config 5: batch 4, 32 heads of 64, 2048 tokens, causal; FLOP counted on the
    # unmasked half only (4 b h s^2 d / 2 forward, 2.5 x that backward)
    b_, s_, h_, d_ = 4, 2048, 32, 64
    qkv = _seeded((b_, s_, h_ * 3 * d_), 21, 1.0, torch.bfloat16).to(device)
    t4 = qkv.view(b_, s_, h_, 3 * d_)
    q_, k_, v_ = t4[..., :d_], t4[..., d_:2 * d_], t4[..., 2 * d_:]
    attn_flop = 4.0 * b_ * h_ * s_ * s_ * d_ / 2
    us = event_time_us(lambda: ops.attn_fwd(q_, k_, v_), 30, 5)
    out["attention_fwd_causal"] = {"us": round(us, 2), "TFLOPs": round(attn_flop / us / 1e6, 1),
                                   "frac": round(attn_flop / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
    o_, lse_ = ops.attn_fwd(q_, k_, v_, want_lse=True)
    do_ = _seeded((b_, s_, h_ * d_), 22, 1.0, torch.bfloat16).to(device)
    g_ = torch.empty_like(t4)
    us = event_time_us(lambda: ops.attn_bwd(q_, k_, v_, o_, do_, lse_, g_[..., :d_], g_[..., d_:2 * d_], g_[..., 2 * d_:]), 30, 5)
    out["attention_bwd_causal"] = {"us": round(us, 2), "TFLOPs": round(2.5 * attn_flop / us / 1e6, 1),
                                   "frac": round(2.5 * attn_flop / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
    # the same launches back to back for 3.5 s each: what holds the clock while these kernels run (clock, socket power,
    # share of the firmware's samples in which the package-power limiter was active, energy per launch)
    for key, fn in (("attention_fwd_causal", lambda: ops.attn_fwd(q_, k_, v_)),
                    ("attention_bwd_causal", lambda: ops.attn_bwd(q_, k_, v_, o_, do_, lse_, g_[..., :d_], g_[..., d_:2 * d_],
                                                                  g_[..., 2 * d_:]))):
        us_s, smi = sustained_us(fn, int(3.5e6 / out[key]["us"]) + 1)
        row = {"us": round(us_s, 2)}
        if smi:
            row.update({k: smi[k] for k in ("shader_clock_MHz", "socket_power_W") if k in smi})
            gm = smi.get("gpu_metrics") or {}
            row.update({k: gm[k] for k in ("energy_mJ_per_launch", "limiter_residency") if k in gm})
        out[key]["sustained"] = row
    del qkv, t4, o_, do_, g_
    # config 5: OPT-1.3B-shaped block, batch 4 x seq 2048, bf16, forward + backward
    initialize("2d", 1)
    torch.manual_seed(0)
    blk = OPTBlock(hidden=2048, heads=32, ffn=8192, dtype=torch.bfloat16, activation="relu").to(device)
    xb = _seeded((4, 2048, 2048), 11, 1.0, torch.bfloat16).to(device).requires_grad_(True)
    dyb = _seeded((4, 2048, 2048), 12, 1.0, torch.bfloat16).to(device)

    def block_step():
        blk.zero_grad(set_to_none=True)
        xb.grad = None
        y = blk(xb)
        y.backward(dyb)
    us = event_time_us(block_step, 10, 3)
    # where the step's time goes: the same step with every C-ABI call bracketed by events (instrumented passes,
    # not the timed ones); what is left is torch's own kernels between the calls (gradient accumulation at the
    # residual forks, dtype casts of the parameter gradients, zero_grad)
    from cubework_amd import _lib as _cw_lib
    real_lib = _cw_lib.load()
    timer = AbiCallTimer(real_lib)
    passes = 5
    _cw_lib._lib = timer
    try:
        for _ in range(passes):
            block_step()
        torch.cuda.synchronize()
    finally:
        _cw_lib._lib = real_lib
    per_kernel = timer.table(passes, us)
    in_calls = sum(r["us_per_step"] for r in per_kernel)
    per_kernel.append({"entry_point": "(torch kernels and gaps between the calls)", "shape": "", "calls_per_step": None,
                       "us_per_step": round(us - in_calls, 1), "share_of_step": round((us - in_calls) / us, 4)})
    # gradient-norm clipping over the block's 12 parameter gradients (one read for the norm, read + write
    # for the scaling)
    from cubework_amd.clip_grad import clip_grad_norm
    params = [p for p in blk.parameters() if p.grad is not None]
    grad_bytes = sum(p.grad.numel() * p.grad.element_size() for p in params)
    us_clip = event_time_us(lambda: clip_grad_norm(params, 1.0), 20, 3)
    out["clip_grad_norm_block"] = {"us": round(us_clip, 2), "bytes": 3 * grad_bytes, "tensors": len(params),
                                   "GBps": round(3 * grad_bytes / us_clip / 1e3, 1),
                                   "frac": round(3 * grad_bytes / us_clip / 1e3 / HBM_PEAK_GBPS, 3)}
    # the same step with the residual additions as separate passes (torch's add after out_proj / fc2, autograd's
    # accumulation at the two LayerNorm forks) instead of the GEMM epilogue / LayerNorm backward kernel: same process,
    # right after the figure above
    fused_plus, fused_fork = OPTBlock.__dict__["_linear_plus"], OPTBlock.__dict__["_norm_fork"]
    try:
        OPTBlock._linear_plus = staticmethod(lambda layer, inp, residual: residual + layer(inp))
        OPTBlock._norm_fork = staticmethod(lambda layer, x_: (layer(x_), x_))
        us_plain = event_time_us(block_step, 10, 3)
    finally:
        OPTBlock._linear_plus, OPTBlock._norm_fork = fused_plus, fused_fork
    us_again = event_time_us(block_step, 10, 3)
    # the same step recorded into a HIP graph and replayed: what the launch gaps of the eager step cost (the entry
    # points neither allocate nor synchronise, so forward + autograd backward capture whole)
    us_graph = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                block_step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        blk.zero_grad(set_to_none=True)
        xb.grad = None
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            blk(xb).backward(dyb)
        us_graph = event_time_us(graph.replay, 10, 3)
        del graph
    except RuntimeError as exc:  # a torch build that cannot capture: the eager figures stand
        sys.stderr.write("bench.py: the block step was not captured (%s)\n" % exc)
    lin_flop = 3 * 2.0 * 8192 * 2048 * (6144 + 2048 + 8192 + 8192)
    out["opt_block_fwd_bwd"] = {"ms": round(us / 1e3, 3), "linear_flop": lin_flop,
                                "linear_TFLOPs_if_all_time_were_linears": round(lin_flop / us / 1e6, 1),
                                "note": "four Linear2D, two LayerNorm2D and the fused attention core (cw_attn_fwd / cw_attn_bwd), tp=1",
                                "same_run_ab": {"residual_additions_as_separate_passes_ms": round(us_plain / 1e3, 3),
                                                "in_epilogue_and_ln_backward_again_ms": round(us_again / 1e3, 3),
                                                "replayed_from_a_hip_graph_ms": None if us_graph is None else round(us_graph / 1e3, 3)},
                                "per_kernel": per_kernel,
                                "per_kernel_source": "events around every C-ABI call during %d instrumented passes of the same "
                                                     "step in this run; the last row is the step's time minus their sum" % passes}
    return out


def _gloo_world_of_one():
    """torch.distributed on gloo with one rank, as cubework/initialize.py:33-35 sets it up. Returns True when
    the group exists (the raw all_reduce calls of the reference's CPU path then run on it)."""
    import torch.distributed as dist
    try:
        if dist.is_initialized():
            return True
        import socket
        s = socket.socket()
        s.bind(("127.0.0.1", 0))
        port = s.getsockname()[1]
        s.close()
        # gloo announces its connections on stdout; keep stdout for the one JSON line
        sys.stdout.flush()
        saved = os.dup(1)
        os.dup2(2, 1)
        try:
            dist.init_process_group("gloo", init_method="tcp://127.0.0.1:%d" % port, rank=0, world_size=1)
        finally:
            sys.stdout.flush()
            os.dup2(saved, 1)
            os.close(saved)
        return True
    except Exception:  # the baseline still runs; the collectives are identities at world size 1
        return False


def _timed_passes(fn, budget_s, max_iters=300):
    """One untimed call, one timed call to size the loop, then as many passes as fit the budget."""
    fn()
    t0 = time.perf_counter()
    fn()
    one = max(time.perf_counter() - t0, 1e-6)
    iters = max(2, min(max_iters, int(budget_s / one)))
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    return (time.perf_counter() - t0) / iters, iters


def cpu_baseline():
    """The reference's CPU path (torch on gloo, world size 1) on the GPU host's cores, restated by oracle/:
    the headline workload (config 2: _SUMMA_AB.forward + _SUMMAbias.forward + GeLU in the tensors' own dtype)
    and, under "other_configs", config 1 (fp32 F.linear forward + autograd backward), config 3 (LayerNorm2D
    forward + backward) and config 4 (vocab-parallel cross-entropy forward + backward) with the all-reduce
    calls the reference makes at world size 1. Each leg runs on a bounded sample: about 5-8 s of CPU work."""
    import torch
    import torch.distributed as dist
    import oracle
    from oracle import cpu_path

    group_ok = _gloo_world_of_one()
    threads = torch.get_num_threads()
    note = "os.cpu_count()=%d, torch threads=%d, gloo world of one %s" % (
        os.cpu_count(), threads, "initialised" if group_ok else "NOT initialised (collectives skipped)")

    # ---- config 2 (headline)
    def run2(rows):
        A = [_seeded((rows, K), i, 1.0, torch.bfloat16) for i in range(STEPS_K)]
        B = [_seeded((K, N), 10 + i, 0.02, torch.bfloat16) for i in range(STEPS_K)]
        bias = _seeded((N,), 7, 0.02, torch.bfloat16)
        return lambda: torch.nn.functional.gelu(oracle.summa_ab_reference_dtype(A, B, bias), approximate="tanh")
    f = run2(1024)
    f()
    t0 = time.perf_counter()
    f()
    per_row = (time.perf_counter() - t0) / 1024
    rows = M if per_row * M * 3 <= 8.0 else max(256, min(M, int(8.0 / (3 * per_row)) // 256 * 256))
    t, iters = _timed_passes(run2(rows), 6.0)
    flop = 2.0 * rows * N * K * STEPS_K
    head = {"value": round(flop / t / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": "%d of %d rows, full K=%dx%d steps and N=%d, bf16 addmm per k-step + bias + GeLU(tanh) as "
                      "parallel_2d/_operation.py:41-47,273 runs it on CPU tensors; %d timed passes, %.3f s each; %s"
                      % (rows, M, K, STEPS_K, N, iters, t, note)}
    other = {}

    # ---- config 1: Linear1D column-parallel, fp32, seed 0, forward + backward at full size
    g = torch.Generator().manual_seed(0)
    x1 = torch.randn((8, 512, 1024), generator=g)
    w1 = (torch.rand((4096, 1024), generator=g) * 2 - 1) * (6.0 / 5120) ** 0.5   # xavier_uniform_, module/init.py:88-99
    b1 = torch.zeros(4096)
    dy1 = torch.randn((8, 512, 4096), generator=g)
    t, iters = _timed_passes(lambda: cpu_path.linear1d_col_fwd_bwd(x1, w1, b1, dy1), 6.0)
    flop1 = 3 * 2.0 * 4096 * 1024 * 4096
    other["config1_linear1d_fp32_fwd_bwd"] = {
        "value": round(flop1 / t / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": "full size: x [8,512,1024], W [4096,1024], F.linear forward + autograd backward "
                  "(parallel_1d/module.py:263-278); %d timed passes, %.3f s each; %s" % (iters, t, note)}
    del x1, w1, dy1

    # ---- config 3: LayerNorm2D shard, bf16, forward + backward, H = 2048 (the peer's half is not there: the
    # reference's arithmetic on the local shard is the same, its row sums would be all-reduced)
    R3, C3 = 16384, 1024
    x3 = _seeded((R3, C3), 100, 1.0, torch.bfloat16)
    dy3 = _seeded((R3, C3), 200, 1.0, torch.bfloat16)
    g3 = (torch.rand(C3, generator=torch.Generator().manual_seed(3)) * 0.2 + 0.9).to(torch.bfloat16)
    b3 = _seeded((C3,), 4, 0.02, torch.bfloat16)
    t, iters = _timed_passes(lambda: cpu_path.layernorm2d_fwd_bwd(x3, g3, b3, dy3, 2048, 1e-5, group_ok), 5.0)
    bytes3 = (2 + 3) * R3 * C3 * 2   # forward reads x writes y; backward reads dy, x writes dx
    other["config3_layernorm2d_bf16_fwd_bwd"] = {
        "value": round(bytes3 / t / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": "%d of 16384 rows x 1024 columns, forward + backward in bf16 as parallel_2d/module.py:142-171 and "
                  "_operation.py:330-347 run on CPU tensors, the two backward all_reduce calls on the gloo group "
                  "included; algorithmic bytes 5 x rows x 1024 x 2; %d timed passes, %.3f s each; %s"
                  % (R3, iters, t, note)}
    del x3, dy3

    # ---- config 4: vocab-parallel cross-entropy, rank 1 of 4, forward + backward
    T4, V4 = 8192, 12568
    lg = _seeded((T4, V4), 300, 2.0, torch.bfloat16)
    tg = torch.randint(0, 50272, (T4,), generator=torch.Generator().manual_seed(9))
    dl = torch.full((T4,), 1.0 / 8192)
    t, iters = _timed_passes(lambda: cpu_path.vpce1d_fwd_bwd(lg, tg, V4, dl, group_ok), 5.0)
    bytes4 = T4 * V4 * 2 + T4 * V4 * 2 + T4 * V4 * 4   # forward reads the logits; backward reads them, writes fp32 grad
    other["config4_vocab_parallel_ce_fwd_bwd"] = {
        "value": round(bytes4 / t / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": "%d of 8192 tokens x 12568 classes (rank 1 of 4), forward + backward as loss/loss_1d.py:14-79 runs "
                  "on CPU tensors (fp32 copy of the bf16 logits, in place), the MAX / SUM / SUM all_reduce calls on "
                  "the gloo group included; algorithmic bytes tokens x 12568 x (2 + 2 + 4); %d timed passes, %.3f s "
                  "each; %s" % (T4, iters, t, note)}
    if group_ok and dist.is_initialized():
        dist.destroy_process_group()
    head["other_configs"] = other
    return head


def mfma_rate_ceiling(device, seconds=0.4):
    """cw_diag_mfma_rate (measurement library): the GEMM's matrix instruction issued back to back from registers,
    random operands of the workload's magnitudes, all-zero operands, and random operands read from LDS at the ring
    kernel's rate, each for `seconds`, with clock and power (and, for runs of 3 s and more, the energy counter)."""
    import ctypes
    import torch
    from cubework_amd import _diag
    lib = _diag.load()
    iters = 20000
    flop = lib.cw_diag_mfma_rate_flop(iters)
    sink = torch.empty(65536, dtype=torch.float32, device=device)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {}
    for name, mode in (("random_operands", 0), ("zero_operands", 1), ("random_operands_read_from_lds", 2),
                       ("random_operands_16x16x32_instruction", 3)):
        def call():
            rc = lib.cw_diag_mfma_rate(iters, mode, sink.data_ptr(), stream)
            if rc != 0:
                raise RuntimeError(lib.cw_last_error().decode())
        us, smi = sustained_us(call, max(10, int(seconds * 1e6 / 6000)))
        out[name] = {"TFLOPs": round(flop / us / 1e6, 1), "frac_of_peak": round(flop / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
        if smi:
            out[name].update({k: smi[k] for k in ("shader_clock_MHz", "socket_power_W", "gpu_metrics") if k in smi})
            gm = out[name].get("gpu_metrics")
            if gm and "socket_power_W_from_energy_counter" in gm:
                gm.pop("energy_mJ_per_launch", None)
                gm["pJ_per_FLOP"] = round(gm["socket_power_W_from_energy_counter"] / (flop / us / 1e6), 4)
    out["note"] = ("register-only loop of v_mfma_f32_32x32x16_bf16 on all 1024 SIMDs: what the board's power management "
                   "leaves of the data-sheet rate for operands that toggle like the workload's; read_from_lds: the same "
                   "loop with the ring kernel's fragment reads from LDS (8 KB per 16 MFMAs), no global loads; "
                   "16x16x32_instruction: the register-only loop with the other bf16 matrix instruction, same FLOP per trip")
    return out


def hw_probes(device):
    """Two facts about the hardware that the attention kernels are priced against. (1) A SIMD with two wavefronts, one
    issuing 4 independent 32x32x16 MFMAs per trip (128 cycles of the matrix pipe), the other 32 vector instructions
    per trip (v_fma_f32, or the transcendental v_exp_f32): time of each alone and of both together. (2) The rate at
    which a compute unit reads LDS with ds_read_b128 and with ds_read_b64_tr_b16 (8 wavefronts, no bank conflicts)."""
    import ctypes
    import torch
    from cubework_amd import _diag
    lib = _diag.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    sink = torch.empty(256 * 512, dtype=torch.float32, device=device)
    isink = torch.empty(256 * 512, dtype=torch.int32, device=device)
    iters = 20000
    out = {"matrix_and_vector_instructions_of_two_wavefronts_on_one_simd": {}, "lds_read_rate_per_compute_unit": {}}

    def check(rc):
        if rc != 0:
            raise RuntimeError(lib.cw_last_error().decode())
    for vop, name in ((0, "v_fma_f32"), (1, "v_exp_f32")):
        t = {}
        for roles, key in ((1, "mfma_only"), (2, "vector_only"), (3, "both")):
            us = event_time_us(lambda: check(lib.cw_diag_overlap(iters, roles, vop, sink.data_ptr(), stream)), 10, 3, min_ms=300)
            t[key] = us / iters * 1e3  # ns per trip
        row = {"ns_per_trip_" + k: round(v, 2) for k, v in t.items()}
        # both = vector_only + x * mfma_only: x = 0 would be complete overlap, 1 none
        row["share_of_the_mfma_time_not_hidden_under_the_vector_wavefront"] = round((t["both"] - t["vector_only"]) / t["mfma_only"], 3)
        row["vector_ns_per_instruction_alone"] = round(t["vector_only"] / 32, 3)
        row["mfma_ns_per_instruction_alone"] = round(t["mfma_only"] / 4, 3)
        out["matrix_and_vector_instructions_of_two_wavefronts_on_one_simd"][name] = row
    li = 4000
    nbytes = lib.cw_diag_lds_rate_bytes(li)
    for tr, name in ((0, "ds_read_b128"), (1, "ds_read_b64_tr_b16")):
        us = event_time_us(lambda: check(lib.cw_diag_lds_rate(li, tr, isink.data_ptr(), stream)), 10, 3, min_ms=300)
        out["lds_read_rate_per_compute_unit"][name] = {"us_per_call": round(us, 1), "GB_per_s": round(nbytes / us / 1e3, 1)}
    a = out["lds_read_rate_per_compute_unit"]
    a["b128_over_transposing"] = round(a["ds_read_b128"]["GB_per_s"] / a["ds_read_b64_tr_b16"]["GB_per_s"], 2)
    return out


def gemm_k_sweep(device):
    """Time of one launch of the block GEMM against its reduction length, at an output of one tile per compute
    unit (8192 x 2048 = 256 tiles of 256 x 256): slope = the k loop, intercept = what every round of tiles costs
    besides (the gap between launches, the first tiles' way from HBM into the ring, the epilogue and the write of
    C, during which no matrix instruction runs). Operands rotate through more than the Infinity Cache holds."""
    import torch
    from cubework_amd import ops
    m_, n_ = 8192, 2048
    out = {"M": m_, "N": n_, "tiles_256": (m_ // 256) * (n_ // 256), "rows": []}
    for layout in ("NT", "NN"):
        for epi in (None, "relu"):
            pts = []
            for k_ in (512, 1024, 2048, 4096, 8192):
                nrot = min(6, max(2, int(600e6 // ((m_ + n_) * k_ * 2))))
                a_ = [_seeded((m_, k_), 10 + i, 1.0, torch.bfloat16).to(device) for i in range(nrot)]
                b_ = [_seeded((n_, k_) if layout == "NT" else (k_, n_), 20 + i, 0.02, torch.bfloat16).to(device)
                      for i in range(nrot)]
                bias = _seeded((n_,), 5, 0.02, torch.bfloat16).to(device) if epi else None
                c_ = torch.empty((m_, n_), dtype=torch.bfloat16, device=device)
                j = [0]

                def fn():
                    j[0] += 1
                    ops.gemm_ksteps(layout, [a_[j[0] % nrot]], [b_[j[0] % nrot]], bias, epi, out=c_)
                pts.append((k_, event_time_us(fn, 30, 5, min_ms=400)))
                del a_, b_
            (k1, t1), (k2, t2) = pts[2], pts[4]
            slope = (t2 - t1) / (k2 - k1)
            flop_per_k = 2.0 * m_ * n_
            out["rows"].append({"layout": layout, "epilogue": epi or "none",
                                "us_by_k": {str(k_): round(t, 2) for k_, t in pts},
                                "us_per_1024_k": round(slope * 1024, 2),
                                "k_loop_frac_of_mfma_peak": round(flop_per_k / slope / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
                                "us_per_launch_beyond_the_k_loop": round(t1 - slope * k1, 2)})
    out["note"] = ("slope and intercept from K = 2048 and 8192; the intercept holds the launch-to-launch gap of back-to-back "
                   "launches, the ring's fill from HBM and the epilogue with the write of the 32 MiB of C")
    return out


def energy_table(device, sets, bias, outs, seconds):
    """Where a launch of the headline GEMM spends its energy: the ring kernel whole and with one part taken out
    (cw_diag_gemm_part of the measurement library: the same kernel source, parts 1-3 not computing anything
    meaningful), each run back to back for `seconds`, priced by the socket's energy counter (average power over
    whole refresh periods of the firmware's table inside the run x the event-timed launch duration). At the power
    cap time = energy / power, so the joules are what the microseconds are made of."""
    import ctypes
    import torch
    from cubework_amd import _diag
    lib = _diag.load()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    tabs = []
    for A, B in sets:
        tabs.append(((ctypes.c_void_p * STEPS_K)(*[t.data_ptr() for t in A]),
                     (ctypes.c_void_p * STEPS_K)(*[t.data_ptr() for t in B])))
    it = [0]

    def make(part, rotate):
        def call():
            k = it[0] % len(sets) if rotate else 0
            it[0] += 1
            ta, tb = tabs[k]
            rc = lib.cw_diag_gemm_part(part, M, N, K, STEPS_K, ta, K, tb, N, bias.data_ptr(), outs[k].data_ptr(), N, stream)
            if rc != 0:
                raise RuntimeError(lib.cw_last_error().decode())
        return call

    runs = {}
    for name, part, rotate in (("whole_kernel_operands_from_hbm", 0, True), ("whole_kernel_operands_cache_resident", 0, False),
                               ("no_operand_loads_in_the_k_loop", 1, False), ("no_lds_fragment_reads_in_the_k_loop", 3, False),
                               ("no_epilogue", 2, False)):
        fn = make(part, rotate)
        pilot, _ = sustained_us(fn, 2000)
        us, smi = sustained_us(fn, int(seconds * 1e6 / pilot) + 1)
        row = {"us_per_launch": round(us, 2)}
        if smi:
            row.update({k: smi[k] for k in ("shader_clock_MHz", "socket_power_W") if k in smi})
            gm = smi.get("gpu_metrics") or {}
            for k in ("socket_power_W_from_energy_counter", "energy_mJ_per_launch", "limiter_residency", "window_s"):
                if k in gm:
                    row[k] = gm[k]
        runs[name] = row
    ceil = mfma_rate_ceiling(device, seconds)
    out = {"runs": runs, "matrix_instruction_loops": ceil, "flop_per_launch": GEMM_FLOP}

    def mj(name):
        return runs[name].get("energy_mJ_per_launch")
    pj = {k: (ceil[k].get("gpu_metrics") or {}).get("pJ_per_FLOP") for k in ("random_operands", "random_operands_read_from_lds", "zero_operands")}
    if all(mj(k) is not None for k in runs) and pj["random_operands"]:
        whole, cached = mj("whole_kernel_operands_from_hbm"), mj("whole_kernel_operands_cache_resident")
        parts = {
            "matrix_instructions": round(pj["random_operands"] * GEMM_FLOP * 1e-9, 2),
            "lds_fragment_reads": round(cached - mj("no_lds_fragment_reads_in_the_k_loop"), 2),
            "operand_loads_l2_to_lds": round(cached - mj("no_operand_loads_in_the_k_loop"), 2),
            "hbm_and_fabric_instead_of_cache": round(whole - cached, 2),
            "epilogue_bias_gelu_store": round(cached - mj("no_epilogue"), 2),
        }
        parts["rest_launch_gap_prologue_barriers_waits"] = round(whole - sum(parts.values()), 2)
        out["energy_mJ_per_launch"] = {"whole_kernel": whole, **parts}
        if pj["zero_operands"]:
            # the matrix instructions' energy in two parts: what the same instructions cost on all-zero operands
            # (clocks, control, leakage: there whether or not the data toggle) and what the operands' switching adds
            idle = round(pj["zero_operands"] * GEMM_FLOP * 1e-9, 2)
            out["energy_mJ_per_launch"]["matrix_instructions_on_zero_operands"] = idle
            out["energy_mJ_per_launch"]["matrix_instructions_operand_switching"] = round(parts["matrix_instructions"] - idle, 2)
        if pj["random_operands_read_from_lds"]:
            out["energy_mJ_per_launch"]["cross_check_lds_reads_from_the_matrix_loops"] = round(
                (pj["random_operands_read_from_lds"] - pj["random_operands"]) * GEMM_FLOP * 1e-9, 2)
        out["note"] = ("each part = whole kernel minus the kernel without that part (cache-resident operands), the matrix "
                       "instructions priced by the register-only loop on random operands; the parts overlap in time, so "
                       "the differences are attributions, and the rest is what no ablation removes")
    return out


def stream_ceiling(device):
    """torch's own copy and fill kernels over the sizes of the LayerNorm / cross-entropy /
    embedding workloads, buffers rotated through more than 512 MiB, replayed from a HIP graph like the aux figures:
    what plain streaming kernels of these sizes reach on this GPU."""
    import torch
    out = {}
    for mib, nbuf in ((32, 18), (64, 10), (196, 4)):
        n = mib * (1 << 20) // 2
        src = [torch.empty(n, device=device, dtype=torch.bfloat16).normal_() for _ in range(nbuf)]
        dst = [torch.empty_like(src[0]) for _ in range(2)]
        i = [0]

        def copy():
            i[0] += 1
            dst[i[0] % 2].copy_(src[i[0] % nbuf])
        us = graph_time_us(copy, 2 * nbuf)
        out["copy_%dMiB" % mib] = {"us": round(us, 2), "bytes": 4 * n, "GBps": round(4 * n / us / 1e3, 1),
                                   "frac": round(4 * n / us / 1e3 / HBM_PEAK_GBPS, 3)}

        def fill():
            i[0] += 1
            src[i[0] % nbuf].zero_()
        us = graph_time_us(fill, 2 * nbuf)
        out["fill_%dMiB" % mib] = {"us": round(us, 2), "bytes": 2 * n, "GBps": round(2 * n / us / 1e3, 1),
                                   "frac": round(2 * n / us / 1e3 / HBM_PEAK_GBPS, 3)}
        # read-only: torch's row reductions over the same buffers viewed as rows of 1024 (what a statistics kernel
        # does: read everything, write one value per row)
        rows = [t.view(-1, 1024) for t in src]
        red = torch.empty(rows[0].shape[0], device=device, dtype=torch.float32)
        redb = torch.empty(rows[0].shape[0], device=device, dtype=torch.bfloat16)

        def row_sum():
            i[0] += 1
            torch.sum(rows[i[0] % nbuf], dim=1, dtype=torch.float32, out=red)

        def row_amax():
            i[0] += 1
            torch.amax(rows[i[0] % nbuf], dim=1, out=redb)
        for name, fn in (("row_sum", row_sum), ("row_amax", row_amax)):
            if mib > 64:
                continue
            us = graph_time_us(fn, 2 * nbuf)
            out["%s_%dMiB" % (name, mib)] = {"us": round(us, 2), "bytes": 2 * n, "GBps": round(2 * n / us / 1e3, 1),
                                            "frac": round(2 * n / us / 1e3 / HBM_PEAK_GBPS, 3)}
        del src, dst, rows
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--sustained", type=int, default=30000,
                    help="launches of the sustained run that roofline.achieved is taken from (0 = use the timed steps); "
                         "the default runs for about 3.5 s: past the window over which the board averages its power, "
                         "and long enough for the firmware's metrics table (energy counter, limiter residencies: one "
                         "refresh a second) to refresh at least twice inside the run")
    ap.add_argument("--no-aux", action="store_true", help="skip the LayerNorm / CE kernels")
    ap.add_argument("--stream-ceiling", action="store_true",
                    help="instead of the benchmark: plain torch copies and fills of 32, 64 and 196 MiB buffers, "
                         "rotated through more than 512 MiB, for a kernel trace of what streaming kernels of the "
                         "LayerNorm / cross-entropy sizes reach on this GPU")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--energy-table", type=float, default=0.0, metavar="SECONDS",
                    help="instead of the benchmark: run the headline GEMM kernel whole and with one part taken out "
                         "(operand loads, LDS fragment reads, epilogue), and the register-only matrix instruction "
                         "loops, each for SECONDS (4 or more, for the firmware's energy counter), and print where a "
                         "launch's energy goes")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy three times (the known-size kernel that hardware "
                         "counter runs of this script are scaled by)")
    ap.add_argument("--gemm-counter-run", action="store_true",
                    help="instead of the benchmark: launch the fp32 ring kernels (config 1 forward and input "
                         "gradient) and the small-tile 16-bit ring kernel (2048^3) six times each, interleaved with "
                         "torch.matmul on the same operands - the program of the hardware-counter comparison")
    ap.add_argument("--attention-counter-run", action="store_true",
                    help="instead of the benchmark: launch the attention core's forward and backward kernels four "
                         "times at config 5's shape (batch 4, 32 heads of 64, 2048 tokens, causal) - the program of "
                         "the hardware-counter passes over those kernels")
    ap.add_argument("--hw-probes", action="store_true",
                    help="instead of the benchmark: two probes of the measurement library that bound the attention "
                         "kernels - how far matrix instructions of one wavefront and vector instructions of another "
                         "overlap on a SIMD, and the LDS read rate of a compute unit with 16-byte reads and with the "
                         "transposing 8-byte reads")
    ap.add_argument("--gemm-k-sweep", action="store_true",
                    help="instead of the benchmark: the 16-bit block GEMM at 8192 x 2048 outputs (256 tiles, one round "
                         "of the chip) for reduction lengths 512 ... 8192, NT and NN, plain and bias + ReLU: the time "
                         "per 1024 of k and what a launch costs beyond its k loop (launch gap, filling the ring from "
                         "HBM, writing the 32 MiB of C)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.stderr.write("bench.py measures one rank's share on ONE GPU; --gpus N with N > 1 is not part of this "
                         "build (no collectives, no sharding across GPUs).\n")
        sys.exit(2)

    import torch
    from cubework_amd import _lib, ops

    if not torch.cuda.is_available():
        sys.stderr.write("bench.py needs an MI355X; there is no CPU fallback of the product path.\n")
        sys.exit(3)
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)
    lib = _lib.load()
    arch = lib.cw_device_arch().decode()
    if args.gemm_counter_run:
        x1 = _seeded((4096, 1024), 1, 1.0, torch.float32).to(device)
        w1 = _seeded((4096, 1024), 2, 0.03, torch.float32).to(device)
        dy1 = _seeded((4096, 4096), 3, 1.0, torch.float32).to(device)
        o1 = torch.empty((4096, 4096), dtype=torch.float32, device=device)
        a2 = _seeded((2048, 2048), 4, 1.0, torch.bfloat16).to(device)
        b2 = _seeded((2048, 2048), 5, 0.03, torch.bfloat16).to(device)
        o2 = torch.empty((2048, 2048), dtype=torch.bfloat16, device=device)
        for _ in range(6):
            ops.gemm_ksteps("NT", [x1], [w1], out=o1)
            torch.matmul(x1, w1.t(), out=o1)
            ops.gemm_ksteps("NN", [dy1], [w1])
            ops.gemm_ksteps("NN", [a2], [b2], out=o2)
            torch.matmul(a2, b2, out=o2)
        torch.cuda.synchronize()
        return

    if args.attention_counter_run:
        b_, s_, h_, d_ = 4, 2048, 32, 64
        t4 = _seeded((b_, s_, h_ * 3 * d_), 21, 1.0, torch.bfloat16).to(device).view(b_, s_, h_, 3 * d_)
        q_, k_, v_ = t4[..., :d_], t4[..., d_:2 * d_], t4[..., 2 * d_:]
        do_ = _seeded((b_, s_, h_ * d_), 22, 1.0, torch.bfloat16).to(device)
        g_ = torch.empty_like(t4)
        for _ in range(4):
            o_, lse_ = ops.attn_fwd(q_, k_, v_, want_lse=True)
            ops.attn_bwd(q_, k_, v_, o_, do_, lse_, g_[..., :d_], g_[..., d_:2 * d_], g_[..., 2 * d_:])
        torch.cuda.synchronize()
        return

    if args.stream_ceiling:
        print(json.dumps({"stream_ceiling": stream_ceiling(device)}))
        return

    if args.gemm_k_sweep:
        print(json.dumps({"gemm_k_sweep": gemm_k_sweep(device)}))
        return

    if args.hw_probes:
        print(json.dumps({"hw_probes": hw_probes(device)}))
        return

    # The bandwidth-bound kernels of the same path run first: the headline's warm-up and timed steps then find the
    # chip as a training loop would, busy and at its working clock, not waking up from idle.
    # (The headline's operands are made before them: seconds of host work during which the GPU would fall asleep.)
    # 5 x 80 MiB of operands and 5 x 32 MiB of outputs rotate (560 MiB against 256 MiB of Infinity Cache), so that no
    # step finds its inputs there; with 3 sets (336 MiB) a launch was 1 % faster
    n_sets = 5
    sets, bias = make_gemm_inputs(n_sets, device)
    outs = [torch.empty((M, N), dtype=torch.bfloat16, device=device) for _ in range(n_sets)]
    if args.energy_table > 0:
        print(json.dumps({"energy_table": energy_table(device, sets, bias, outs, args.energy_table)}))
        return
    aux = None if args.no_aux else bench_bandwidth_kernels(device)
    it = [0]

    def step():
        A, B = sets[it[0] % n_sets]
        ops.gemm_ksteps("NN", A, B, bias, "gelu_tanh", out=outs[it[0] % n_sets])
        it[0] += 1

    # The sustained run comes first: 10,000 launches (more than a second) bring the board to the clock and power it
    # holds under this load, and roofline.achieved is taken from them. The W warm-up steps and the K timed steps
    # follow at once, so `value` is measured on a chip in that steady state, not on the transient after the
    # bandwidth kernels (which leave the clock high and the power controller about to overshoot).
    smi = None
    kernel_us = None
    if args.sustained > 0:
        kernel_us, smi = sustained_us(step, args.sustained)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    steps_us = e0.elapsed_time(e1) * 1e3 / args.steps
    if kernel_us is None:
        kernel_us = steps_us
    achieved = GEMM_FLOP / kernel_us / 1e6

    result = {
        "metric": "Linear2D per-rank TFLOP/s (%bf16 MFMA peak); LN/CE HBM GB/s (%peak)",
        "value": round(GEMM_FLOP / ms_per_step / 1e9, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "Linear2D one rank of a q=2 grid: X blocks [8192,2048] bf16, W blocks [2048,2048] bf16, "
                               "2 SUMMA k-steps accumulated in fp32, fused bias+GeLU(tanh), out [8192,2048] bf16",
                   "layout": "NN", "flop_per_step": GEMM_FLOP, "operand_sets_rotated": n_sets, "device_arch": arch},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": measured_traffic(),
                     "traffic_source": "profiles/gemm_bf16_dma_kernel_linear2d_q2_counters.txt (committed counter runs of "
                                       "this script, not measured in this run)",
                     "kernel": "the launch cw_gemm_ksteps makes for this shape (gemm_bf16_dma_kernel, 256x256 tiles; "
                               "name as the kernel trace of this command shows it)",
                     "avg_launch_us": round(kernel_us, 2), "launches": args.sustained if args.sustained > 0 else args.steps,
                     "timed_steps": {"avg_launch_us": round(steps_us, 2),
                                     "frac": round(GEMM_FLOP / steps_us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
                                     "note": "HIP events around the K timed steps only, which follow the sustained run"}},
    }
    if smi is not None and smi.get("shader_clock_MHz"):
        # 4096 matrix instructions of 32 cycles per SIMD and launch: the share of the launch's shader cycles in which
        # the matrix pipe is busy, at the clock the driver reports
        cycles = kernel_us * smi["shader_clock_MHz"]
        smi["mfma_busy_frac"] = round(GEMM_FLOP / (256 * 4 * 1024.0) / cycles, 4) if cycles > 0 else None
        smi["clock_x_busy_vs_2400MHz"] = round(smi["shader_clock_MHz"] / 2400.0 * smi["mfma_busy_frac"], 4)
    if smi is not None:
        result["roofline"]["sustained_clock_power"] = smi
    result["roofline"]["mfma_rate_ceiling"] = mfma_rate_ceiling(device)
    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=device).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if aux is not None:
        result["aux"] = aux
        result["aux"]["hbm_peak_GBps"] = HBM_PEAK_GBPS
    if not args.no_aux:
        result["other_configs"] = bench_other_configs(device, sets)
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
