#!/usr/bin/env python3
"""Benchmark of the forward-mode attention hot path on one MI355X.

A "step" is one launch of the fused forward+JVP kernel over one synthetic batch
of the headline workload (SiT/DMFT-XL/2 at 512px: B=64, H=16, N=1024, D=72,
bf16, q/k RMS-normalised), inputs resident in HBM.  Prints ONE JSON line:

  metric/value   attention fwd+JVP TFLOP/s on the algorithmic FLOP count
                 12*B*H*N^2*D (unpadded head dim)
  roofline       the same figure against MI355X's dense bf16 MFMA peak
  cpu_baseline   the CPU oracle ('base' attention under torch.func.jvp, fp32)
                 timed on this box's host cores on a bounded slice of the
                 same workload
  extra          the other kernel-level figures (N=256 shape, backward,
                 primal-only forward, the HBM-bound block-glue kernels), board
                 power and shader clock while the attention kernels run, and
                 end-to-end images/s of the DMFT / SiT steps and the sampler

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extra]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16
HBM_PEAK_GBS = 8000.0
# Counter figures measured offline with rocprofv3 --pmc over `bench.py --workload W --kernel K` (summaries with the
# commands in profiles/attn_<kernel>_bf16_d72_<workload>.txt): HBM bytes per step from FETCH_SIZE / WRITE_SIZE, each scaled
# by what the counter reads for a plain 1 GiB copy in the same run, and the share of the clocked cycles in which the MFMA
# pipe was busy (SQ_VALU_MFMA_BUSY_CYCLES / (4 SQ_BUSY_CU_CYCLES)).  Each row names the kernel it was taken on and the
# hash of that kernel's source files at the time (source_hash()); a row whose kernel or hash no longer matches what
# this tree launches is reported as stale and its figures are withheld.  The two-kernel backward at N=1024 reads
# q, k, v, dout twice.
OFFLINE_COUNTERS = {
    ("fwd_jvp", "xl2_512px"): {"traffic": 1.2124e+09, "mfma_busy": 0.596, "kernel": "dmf::attn_fwd_bf16_kernel<72, true, 8, false, false>",
                               "src": ("attn_fwd_bf16.hip", "8b80f746688ed301")},
    ("fwd_jvp", "xl2_256px"): {"traffic": 1.2124e+09, "mfma_busy": 0.351, "kernel": "dmf::attn_fwd_bf16_kernel<72, true, 8, false, false>",
                               "src": ("attn_fwd_bf16.hip", "8b80f746688ed301")},
    ("fwd", "xl2_512px"): {"traffic": 6.0848e+08, "mfma_busy": 0.529, "kernel": "dmf::attn_fwd_bf16_kernel<72, false, 8, false, false>",
                           "src": ("attn_fwd_bf16.hip", "8b80f746688ed301")},
    ("fwd", "xl2_256px"): {"traffic": 6.0900e+08, "mfma_busy": 0.299, "kernel": "dmf::attn_fwd_bf16_kernel<72, false, 8, false, false>",
                           "src": ("attn_fwd_bf16.hip", "8b80f746688ed301")},
    ("bwd", "xl2_512px"): {"traffic": 1.8709e+09, "mfma_busy": 0.515,
                           "kernel": "dmf::attn_bwd_dq_bf16_kernel<72, 2> + dmf::attn_bwd_dkv_bf16_kernel<72, 4>", "src": ("attn_bwd_bf16.hip", "0baa6add1e385c9d")},
    ("bwd", "xl2_256px"): {"traffic": 1.2167e+09, "mfma_busy": 0.231, "kernel": "dmf::attn_bwd_fused_bf16_kernel<72>",
                           "src": ("attn_bwd_bf16.hip", "0baa6add1e385c9d")},
}


def source_hash(name):
    """First 16 hex digits of the SHA-256 of a kernel source file together with the shared device header."""
    import hashlib
    h = hashlib.sha256()
    for f in (name, "attn_common.h"):
        with open(os.path.join(ROOT, "dmf_amd", "csrc", f), "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()[:16]


DEVICE_WAKE_SECONDS = 0.3        # untimed launches of the measured kernel before the --warmup steps (clock ramp from idle)

WORKLOADS = {
    # name: (B, H, N, D, qk_norm)
    "xl2_512px": (64, 16, 1024, 72, True),    # SiT/DMFT-XL/2 at 512px with qk-norm (headline)
    "xl2_256px": (256, 16, 256, 72, False),   # SiT/DMFT-XL/2 at 256px
}


_T0 = time.perf_counter()


def progress(text):
    """One line per finished measurement on stderr (stdout carries only the final JSON line)."""
    print(f"[bench {time.perf_counter() - _T0:6.1f}s] {text}", file=sys.stderr, flush=True)


def make_inputs(name, device, dtype, seed):
    import torch
    from dmf_amd.layers import RMSNorm

    B, H, N, D, qk_norm = WORKLOADS[name]
    g = torch.Generator(device=device).manual_seed(seed)
    q, k, v, tq, tk, tv, do = (torch.randn(B, N, H, D, generator=g, device=device, dtype=torch.float32) for _ in range(7))
    if qk_norm:
        norm = RMSNorm(D).to(device)
        with torch.no_grad():
            q, k = norm(q), norm(k)
    return [t.to(dtype).contiguous() for t in (q, k, v, tq, tk, tv, do)]


def time_gpu(fn, steps, warmup):
    """Average duration (ms) of `fn` over `steps` back-to-back launches on the
    current stream, HIP events bracketing the timed region."""
    import torch

    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return start.elapsed_time(stop) / steps, wall_ms / steps


def attn_flops(B, H, N, D, kind):
    mult = {"fwd_jvp": 12, "fwd": 4, "bwd": 10}[kind]
    return mult * B * H * N * N * D


def attn_bytes(B, H, N, D, kind, elem=2):
    if kind == "fwd_jvp":
        return 8 * B * N * H * D * elem + 4 * B * H * N
    if kind == "fwd":
        return 4 * B * N * H * D * elem + 4 * B * H * N
    return 8 * B * N * H * D * elem + 2 * 4 * B * H * N


def cpu_baseline(name, budget_s=15.0):
    """Oracle ('base' attention under torch.func.jvp, fp32) on the host cores,
    on a slice of `name`: one batch element, all heads."""
    import torch
    from oracle import attn_oracle as ao

    B, H, N, D, qk_norm = WORKLOADS[name]
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    q, k, v, tq, tk, tv, _ = ao.make_inputs(1, N, H, D, seed=4)
    if qk_norm:
        q, k = ao.rms_norm(q), ao.rms_norm(k)
    ao.base_attn_jvp(q, k, v, tq, tk, tv)  # warm-up
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 50):
        t0 = time.perf_counter()
        ao.base_attn_jvp(q, k, v, tq, tk, tv)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    flops = attn_flops(1, H, N, D, "fwd_jvp")
    return {
        "value": flops / med / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"{name} slice B=1 H={H} N={N} D={D} fp32, naive attention under torch.func.jvp, "
                  f"median of {len(times)} calls ({med * 1e3:.1f} ms/call)",
    }


def cpu_baseline_config1():
    """The CPU-runnable case (B2 H12 N256 D64 fp32) at all cores and at the 4
    intra-op threads the reference pins (train_dmf.py:33-34)."""
    import torch
    from oracle import attn_oracle as ao

    out = {}
    q, k, v, tq, tk, tv, _ = ao.make_inputs(2, 256, 12, 64, seed=1)
    flops = attn_flops(2, 12, 256, 64, "fwd_jvp")
    for label, nthr in (("all_cores", os.cpu_count() or 1), ("threads_4", 4)):
        torch.set_num_threads(nthr)
        for _ in range(3):
            ao.base_attn_jvp(q, k, v, tq, tk, tv)
        ts = []
        for _ in range(15):
            t0 = time.perf_counter()
            ao.base_attn_jvp(q, k, v, tq, tk, tv)
            ts.append(time.perf_counter() - t0)
        ts.sort()
        out[label] = {"threads": nthr, "ms_median": ts[len(ts) // 2] * 1e3, "ms_min": ts[0] * 1e3,
                      "gflops": flops / ts[len(ts) // 2] / 1e9}
    torch.set_num_threads(os.cpu_count() or 1)
    return out


PROFILE_FILES = {(k, w): f"profiles/attn_{k}_bf16_d72_{w}.txt" for k in ("fwd_jvp", "fwd", "bwd") for w in ("xl2_512px", "xl2_256px")}


def roofline(name, ms, kind="fwd_jvp"):
    """Roofline entry for one kernel-level measurement: the MFMA roof when the workload's arithmetic intensity is above
    the machine balance (2.5 PFLOP/s / 8 TB/s = 312 FLOP/B), the HBM roof otherwise (fwd+JVP at N=256: 191 FLOP/B)."""
    from dmf_amd import _lib
    B, H, N, D, _ = WORKLOADS[name]
    flops, nbytes = attn_flops(B, H, N, D, kind), attn_bytes(B, H, N, D, kind)
    kernel = _lib.plan(kind, B, H, N, N, D)       # what the library launches for this shape on this device
    off = OFFLINE_COUNTERS.get((kind, name))
    fresh = off is not None and off["kernel"] == kernel and off["src"][1] == source_hash(off["src"][0])
    common = {"traffic": off["traffic"] if fresh else None,
              "traffic_source": (PROFILE_FILES[(kind, name)] + " (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, offline)") if fresh
                                else "withheld: the committed counter run was taken on another kernel or kernel source",
              "mfma_busy": off["mfma_busy"] if fresh else None, "kernel": kernel}
    if flops / nbytes >= MFMA_BF16_PEAK_TFLOPS * 1e12 / (HBM_PEAK_GBS * 1e9):
        a = flops / (ms * 1e-3) / 1e12
        return {"bound": "mfma", "achieved": a, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": a / MFMA_BF16_PEAK_TFLOPS,
                **common, "hbm_gbs_algorithmic": nbytes / (ms * 1e-3) / 1e9}
    a = nbytes / (ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": a, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": a / HBM_PEAK_GBS,
            **common, "tflops_algorithmic": flops / (ms * 1e-3) / 1e12}


def device_probes():
    """Practical ceilings of this device (bench_probes.hip): sustained bf16 MFMA rate from a register-only
    loop with constant and with random operand bits (power-limited clocks), and the bandwidth of a math-free kernel
    with the operator's row access pattern at the N=256 workload."""
    import ctypes
    path = os.path.join(ROOT, "libbench_probes.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    lib.dmf_probe_mfma_tflops.restype = ctypes.c_float
    lib.dmf_probe_mfma_tflops.argtypes = [ctypes.c_int, ctypes.c_int]
    out = {}
    for label, rnd in (("mfma_constant_operands_tflops", 0), ("mfma_random_operands_tflops", 1)):
        out[label] = max(lib.dmf_probe_mfma_tflops(rnd, 100000) for _ in range(2))
    # memory-system ceiling for the operator's access pattern (6 reads + 2 writes of D-wide rows per head, no math)
    lib.dmf_probe_rows_stream_tbps.restype = ctypes.c_float
    lib.dmf_probe_rows_stream_tbps.argtypes = [ctypes.c_int] * 5
    B, H, N, D, _ = WORKLOADS["xl2_256px"]
    out["rows_stream_BNHD_tbps"] = lib.dmf_probe_rows_stream_tbps(B, H, N, D, 0)
    out["rows_stream_head_contiguous_tbps"] = lib.dmf_probe_rows_stream_tbps(B, H, N, D, 1)
    return out


class _Telemetry:
    """Samples the board's power draw and shader clock from sysfs (hwmon ``power1_input`` in microwatts, the
    starred line of ``pp_dpm_sclk``) every few milliseconds on a thread while a block of GPU work runs."""

    def __init__(self):
        import glob
        pw = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input"))
        self.power_file = pw[0] if pw else None
        dev = os.path.dirname(os.path.dirname(os.path.dirname(pw[0]))) if pw else None
        self.sclk_file = os.path.join(dev, "pp_dpm_sclk") if dev and os.path.exists(os.path.join(dev, "pp_dpm_sclk")) else None
        cap = pw[0].replace("power1_input", "power1_cap") if pw else None
        self.cap_w = int(open(cap).read()) / 1e6 if cap and os.path.exists(cap) else None
        # The SMU's throttler residency counters (amdsmi): one tick per controller iteration (about 1 kHz) in which
        # the package-power (PPT), socket / VR / HBM thermal or PROCHOT controller was holding the clocks down.
        self.smi = None
        try:
            import amdsmi
            amdsmi.amdsmi_init()
            self.smi = (amdsmi, amdsmi.amdsmi_get_processor_handles()[0])
            self._violations()
        except Exception:   # not installed, no permission, or a driver that does not export the counters
            self.smi = None

    def _violations(self):
        amdsmi, h = self.smi
        v = amdsmi.amdsmi_get_violation_status(h)
        keys = ("acc_counter", "acc_ppt_pwr", "acc_socket_thrm", "acc_vr_thrm", "acc_hbm_thrm", "acc_prochot_thrm")
        return {k: v[k] for k in keys if isinstance(v.get(k), int)}

    def _metrics(self):
        amdsmi, h = self.smi
        m = amdsmi.amdsmi_get_gpu_metrics_info(h)
        out = {k: m[k] for k in ("temperature_hotspot", "temperature_mem", "current_socket_power") if isinstance(m.get(k), (int, float))}
        clk = [c for c in m.get("current_gfxclks", []) if isinstance(c, (int, float))]
        if clk:
            out["gfxclk_mhz_per_xcd"] = clk
        return out

    def available(self):
        return self.power_file is not None

    def _sample(self):
        p = int(open(self.power_file).read()) / 1e6
        f = None
        if self.sclk_file:
            for line in open(self.sclk_file).read().splitlines():
                if line.rstrip().endswith("*"):
                    f = float(line.split(":")[1].strip().rstrip("*").strip().lower().replace("mhz", ""))
        return p, f

    def measure(self, fn, seconds=2.0, burst=20):
        """Run ``fn`` (which enqueues GPU work) repeatedly for about ``seconds`` and return mean / max power in watts
        and the mean shader clock in MHz over the samples taken after the first quarter of the interval."""
        import threading
        import torch
        samples, stop = [], threading.Event()

        def sampler():
            while not stop.is_set():
                try:
                    samples.append((time.perf_counter(),) + self._sample())
                except (OSError, ValueError, IndexError):
                    pass
                time.sleep(0.005)

        th = threading.Thread(target=sampler, daemon=True)
        t0 = time.perf_counter()
        th.start()
        v0 = v1 = smu = None
        while time.perf_counter() - t0 < seconds:
            for _ in range(burst):
                fn()
            torch.cuda.synchronize()
            if self.smi is not None and v0 is None and time.perf_counter() - t0 > 0.3 * seconds:
                v0 = self._violations()     # both readings are taken while the load runs: the counters lag by a fraction of a second
        if self.smi is not None and v0 is not None:
            try:
                v1, smu = self._violations(), self._metrics()
            except Exception:
                v1 = None
        stop.set()
        th.join()
        t1 = time.perf_counter()
        keep = [x for x in samples if x[0] >= t0 + 0.25 * (t1 - t0)]
        if not keep:
            return None
        clocks = [x[2] for x in keep if x[2] is not None]
        out = {"power_w_mean": sum(x[1] for x in keep) / len(keep), "power_w_max": max(x[1] for x in keep),
               "sclk_mhz_mean": sum(clocks) / len(clocks) if clocks else None, "samples": len(keep)}
        if v1 is not None and v1.get("acc_counter", 0) > v0.get("acc_counter", 0):
            ticks = v1["acc_counter"] - v0["acc_counter"]
            out["throttler_residency_pct"] = {k[4:]: 100.0 * (v1[k] - v0[k]) / ticks for k in v1 if k != "acc_counter" and k in v0}
            out["smu"] = smu
        return out


def power_probes(fns, seconds=2.0):
    """Board power, shader clock and the SMU's throttler residencies while each of the named GPU workloads runs for
    ``seconds`` (None without sysfs access)."""
    tel = _Telemetry()
    if not tel.available():
        return None
    out = {"power_cap_w": tel.cap_w}
    for label, fn in fns:
        out[label] = tel.measure(fn, seconds=seconds)
    probe = os.path.join(ROOT, "libbench_probes.so")
    if os.path.exists(probe):   # the register-only MFMA loop of device_probes(): what pure matrix work draws (each call is synchronous)
        import ctypes
        lib = ctypes.CDLL(probe)
        lib.dmf_probe_mfma_tflops.restype = ctypes.c_float
        lib.dmf_probe_mfma_tflops.argtypes = [ctypes.c_int, ctypes.c_int]
        for label, rnd in (("mfma_loop_random_operands", 1), ("mfma_loop_constant_operands", 0)):
            rates = []
            out[label] = tel.measure(lambda: rates.append(lib.dmf_probe_mfma_tflops(rnd, 20000)), seconds=seconds, burst=1)
            if out[label] is not None and rates:
                out[label]["tflops_mean"] = sum(rates) / len(rates)
    return out


def per_launch_stats(fn, iters=50):
    """Median and minimum duration (ms) of single launches, one HIP event pair per launch."""
    import torch

    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    torch.cuda.synchronize()
    for a, b in ev:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    ts = sorted(a.elapsed_time(b) for a, b in ev)
    return ts[len(ts) // 2], ts[0]


def block_kernel_rows(device, steps=50, warmup=10):
    """HBM-bound block-glue kernels at the two end-to-end shapes: algorithmic
    bytes (each operand read once, each result written once) / launch time."""
    import torch
    from dmf_amd import _lib

    out = {}
    f32, bf16 = torch.float32, torch.bfloat16
    for tag, (B, L, C) in {"dmft_b2_b64": (64, 256, 768), "dmft_xl2_b32": (32, 256, 1152)}.items():
        n = B * L * C
        x, tx, gyf = (torch.randn(B, L, C, device=device) for _ in range(3))
        h, th, gyb = (torch.randn(B, L, C, device=device, dtype=bf16) for _ in range(3))
        mods = torch.randn(B, 1, 6 * C, device=device, dtype=bf16) * 0.3
        tmods = torch.randn(B, 1, 6 * C, device=device, dtype=bf16) * 0.3
        sh, sc, gt = mods[..., :C], mods[..., C:2 * C], mods[..., 2 * C:3 * C]
        tsh, tsc, tgt = tmods[..., :C], tmods[..., C:2 * C], tmods[..., 2 * C:3 * C]
        u, tu = (torch.randn(B, L, 4 * C, device=device, dtype=bf16) for _ in range(2))
        cases = {
            # name: (callable, algorithmic bytes)
            "ln_modulate_fwd_jvp": (lambda: _lib.ln_modulate_fwd(x, sh, sc, tx, tsh, tsc, 1e-6, bf16, True), n * (4 + 4 + 2 + 2)),
            "ln_modulate_bwd": (lambda: _lib.ln_modulate_bwd(gyb, x, sc), n * (2 + 4 + 4)),
            "gate_residual_fwd_jvp": (lambda: _lib.gate_residual_fwd(x, gt, h, tx, tgt, th, True), n * (4 + 4 + 2 + 2 + 4 + 4)),
            "gate_residual_bwd": (lambda: _lib.gate_residual_bwd(gyf, gt, h), n * (4 + 2 + 2)),
            "residual_ln_modulate_fwd_jvp": (lambda: _lib.residual_ln_modulate_fwd(x, gt, h, sh, sc, tx, tgt, th, tsh, tsc, 1e-6, bf16, True),
                                             n * (4 + 4 + 2 + 2 + 4 + 4 + 2 + 2)),
            "gelu_tanh_fwd_jvp": (lambda: _lib.gelu_tanh_fwd(u, tu), 4 * n * 2 * 4),
            "gelu_tanh_bwd": (lambda: _lib.gelu_tanh_bwd(tu, u), 4 * n * 2 * 3),
            "colsum_4C": (lambda: _lib.colsum(u.view(B * L, 4 * C), f32), 4 * n * 2),
        }
        row = {}
        for kname, (fn, nbytes) in cases.items():
            ms, _ = time_gpu(fn, steps, warmup)
            row[kname] = {"ms": ms, "hbm_gbs_algorithmic": nbytes / ms / 1e6, "pct_hbm_peak": 100 * nbytes / ms / 1e6 / HBM_PEAK_GBS}
        out[tag] = row
    return out


def main():
    from dmf_amd.layers import ATTN_FUNCS

    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="xl2_512px", choices=list(WORKLOADS))
    ap.add_argument("--kernel", default="fwd_jvp", choices=["fwd_jvp", "fwd", "bwd"],
                    help="the entry point one step launches (default: the fused forward+JVP, the headline); "
                         "'fwd' = primal-only forward, 'bwd' = backward on the primal output -- for per-kernel profiles")
    ap.add_argument("--attn-func", default="hip", choices=ATTN_FUNCS,
                    help="attention operator of the model built by --dmft-graph (the reference's --attn-func switch, "
                         "train_dmf.py:427, with the new value 'hip')")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary measurements")
    ap.add_argument("--all-cases", action="store_true",
                    help="also run the end-to-end cases outside the two BASELINE model configurations (no-grad forward, 512px training "
                         "step, whole DMF loss step, SiT flow-matching step, sampling loop) and every variant of each case")
    ap.add_argument("--copy-calib", action="store_true",
                    help="also launch one plain 1 GiB device copy (reads 1 GiB, writes 1 GiB): the known-size kernel "
                         "that HBM traffic counters are scaled by when this command runs under rocprofv3 --pmc")
    ap.add_argument("--dmft-graph", default=None, metavar="CASE",
                    help="profiling aid: run only the HIP-graph replay of one fused end-to-end case of extra.dmft (its key, e.g. "
                         "'DMFT-B/2', 'DMFT-XL/2', 'SiT-XL/2 FM train step') for --steps replays and print its images/s")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the attention units (b, h) are independent and shard "
                 "over GPUs by batch without any collective); run with --gpus 1")

    import torch
    from dmf_amd import _lib

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP kernels are the only implementation")
    _lib.load()
    dev, dtype = "cuda:0", torch.bfloat16
    if args.dmft_graph:
        from dmf_amd import harness
        # 'hip': the fused model replayed as a HIP graph; 'base' / 'torch_sdpa': the reference's expressions around that operator, eager
        variant = "hip_fused_graph" if args.attn_func == "hip" else args.attn_func
        rows = harness.bench_dmft(steps=max(1, args.steps // 4), only=args.dmft_graph, variants=(variant,))
        if args.dmft_graph not in rows:
            sys.exit(f"bench.py: unknown --dmft-graph case {args.dmft_graph!r}")
        row = rows[args.dmft_graph]
        how = "hip attention + fused block glue, HIP-graph replay" if args.attn_func == "hip" else f"{args.attn_func} attention, eager"
        print(json.dumps({"metric": "dmft_images_per_s", "value": row[f"{variant}_images_per_s"], "unit": "images/s",
                          "n_gpus": 1, "steps": args.steps, "ms_per_step": row[f"{variant}_ms_per_step"],
                          "config": {"workload": f"{args.dmft_graph}: {row['tokens']} tokens, {row['mode']}, batch {row['batch']}, "
                                                 f"{row['dtype']}, {how}", "attn_func": args.attn_func}}))
        return
    name = args.workload
    B, H, N, D, _ = WORKLOADS[name]
    q, k, v, tq, tk, tv, do = make_inputs(name, dev, dtype, seed=4)
    scale = D ** -0.5

    if args.copy_calib:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # an idle device sits at its lowest clock level (157 MHz shader clock) and takes tens of milliseconds of load to leave
    # it: bring it up with untimed launches first, so that a short --warmup measures the same steady state as a long one
    kind = args.kernel
    if kind == "fwd_jvp":
        step = lambda: _lib.fwd_jvp(q, k, v, tq, tk, tv, scale)
    elif kind == "fwd":
        step = lambda: _lib.fwd(q, k, v, scale)
    else:
        o0, lse0 = _lib.fwd(q, k, v, scale)[:2]
        step = lambda: _lib.bwd(do, q, k, v, o0, lse0, scale)
    label = {"fwd_jvp": "fwd+JVP", "fwd": "primal forward", "bwd": "backward (dQ, dK, dV)"}[kind]
    wake_until = time.perf_counter() + DEVICE_WAKE_SECONDS
    while time.perf_counter() < wake_until:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
    ms, wall_ms = time_gpu(step, args.steps, args.warmup)
    flops = attn_flops(B, H, N, D, kind)
    tflops = flops / (ms * 1e-3) / 1e12
    ms_median, ms_min = per_launch_stats(step)
    progress(f"{name} attention {label}: {ms:.4f} ms/step, {tflops:.1f} TFLOP/s")
    result = {
        "metric": f"attn_{kind}_tflops", "value": tflops, "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{name}: attention {label} B={B} H={H} N={N} D={D} bf16"
                               + (" q,k RMS-normalised" if WORKLOADS[name][4] else ""),
                   "flops_per_step": flops, "hbm_bytes_per_step": attn_bytes(B, H, N, D, kind),
                   "wall_ms_per_step": wall_ms, "single_launch_ms_median": ms_median, "single_launch_ms_min": ms_min,
                   "untimed_device_wake_seconds": DEVICE_WAKE_SECONDS},
        "roofline": roofline(name, ms, kind),
    }

    if not args.no_extra:
        extra = {}
        rows = []
        o, to, lse = _lib.fwd_jvp(q, k, v, tq, tk, tv, scale)
        for wname in WORKLOADS:
            Bw, Hw, Nw, Dw, _ = WORKLOADS[wname]
            if wname == name:
                ins, ow, lsew = (q, k, v, tq, tk, tv, do), o, lse
            else:
                ins = make_inputs(wname, dev, dtype, seed=3)
                ow, _, lsew = _lib.fwd_jvp(*ins[:6], scale)
            qw, kw, vw, tqw, tkw, tvw, dow = ins
            row = {}
            for kind, fn in (("fwd_jvp", lambda: _lib.fwd_jvp(qw, kw, vw, tqw, tkw, tvw, scale)),
                             ("fwd", lambda: _lib.fwd(qw, kw, vw, scale)),
                             ("bwd", lambda: _lib.bwd(dow, qw, kw, vw, ow, lsew, scale))):
                t_ms, _ = time_gpu(fn, max(10, args.steps // 2), max(5, args.warmup // 2))
                fl, by = attn_flops(Bw, Hw, Nw, Dw, kind), attn_bytes(Bw, Hw, Nw, Dw, kind)
                rl = roofline(wname, t_ms, kind)
                row[kind] = {"ms": t_ms, "tflops": fl / t_ms / 1e9, "pct_bf16_mfma_peak": 100 * fl / t_ms / 1e9 / MFMA_BF16_PEAK_TFLOPS,
                             "hbm_gbs_algorithmic": by / t_ms / 1e6, "pct_hbm_peak": 100 * by / t_ms / 1e6 / HBM_PEAK_GBS,
                             "roofline": rl}
                rows.append({"workload": f"{wname} B{Bw} H{Hw} N{Nw} D{Dw}", "entry": kind, "kernel": rl["kernel"], "ms": round(t_ms, 4),
                             "bound": rl["bound"], "frac": round(rl["frac"], 4), "tflops": round(fl / t_ms / 1e9, 1),
                             "hbm_gbs": round(by / t_ms / 1e6, 1),
                             "traffic_ratio": None if rl["traffic"] is None else round(rl["traffic"] / by, 3),
                             "mfma_busy": rl["mfma_busy"]})
            extra[wname] = row
            progress(f"{wname}: fwd_jvp / fwd / bwd = " + " / ".join(f"{row[kd]['ms']:.4f}" for kd in ("fwd_jvp", "fwd", "bwd")) + " ms")
            del ins
        # every kernel-level figure of the path in one compact list (the bulky detail stays under "extra")
        result["roofline_rows"] = rows
        extra["device_probes"] = device_probes()
        zq = [torch.zeros_like(q) for _ in range(6)]
        other = "xl2_256px" if name == "xl2_512px" else "xl2_512px"
        q2, k2, v2, tq2, tk2, tv2, do2 = make_inputs(other, dev, dtype, seed=3)
        o2, _, lse2 = _lib.fwd_jvp(q2, k2, v2, tq2, tk2, tv2, scale)
        zq2 = [torch.zeros_like(q2) for _ in range(6)]
        # (all-zero inputs: six separate tensors, so that the memory footprint -- and with it what the caches hold --
        #  is that of the real call and only the operand toggling differs)
        extra["power"] = power_probes([
            (f"attn_fwd_jvp_{name}", lambda: _lib.fwd_jvp(q, k, v, tq, tk, tv, scale)),
            (f"attn_fwd_jvp_{name}_all_zero_inputs", lambda: _lib.fwd_jvp(*zq, scale)),
            (f"attn_bwd_{name}", lambda: _lib.bwd(do, q, k, v, o, lse, scale)),
            (f"attn_fwd_jvp_{other}", lambda: _lib.fwd_jvp(q2, k2, v2, tq2, tk2, tv2, scale)),
            (f"attn_fwd_jvp_{other}_all_zero_inputs", lambda: _lib.fwd_jvp(*zq2, scale)),
            (f"attn_bwd_{other}", lambda: _lib.bwd(do2, q2, k2, v2, o2, lse2, scale)),
        ] if args.all_cases else [
            (f"attn_fwd_jvp_{name}", lambda: _lib.fwd_jvp(q, k, v, tq, tk, tv, scale)),
            (f"attn_fwd_jvp_{name}_all_zero_inputs", lambda: _lib.fwd_jvp(*zq, scale)),
        ], seconds=2.0 if args.all_cases else 1.0)
        if extra["power"] is not None:
            pw = extra["power"].get(f"attn_fwd_jvp_{name}") or {}
            result["power"] = {"cap_w": extra["power"].get("power_cap_w"), "fwd_jvp_w_mean": pw.get("power_w_mean"),
                               "fwd_jvp_sclk_mhz_mean": pw.get("sclk_mhz_mean"),
                               "fwd_jvp_ppt_residency_pct": (pw.get("throttler_residency_pct") or {}).get("ppt_pwr")}
        del zq, zq2, q2, k2, v2, tq2, tk2, tv2, do2, o2, lse2
        progress("device probes done" + ("" if extra["power"] is None else f"; power {json.dumps(extra['power'])}"))
        if args.all_cases:
            extra["block_kernels"] = block_kernel_rows(dev)
            progress("block kernels done")
        try:
            from dmf_amd import harness
            # default: the two model configurations BASELINE names (DMFT-B/2 forward+JVP at batch 64, DMFT-XL/2 training step at
            # batch 32) and the caller of the headline attention shape, fused graph replay against the naive operator
            only = None if args.all_cases else ("DMFT-B/2", "DMFT-XL/2", "DMFT-XL/2 512px qk-norm")
            variants = None if args.all_cases else ("hip_fused_graph", "hip", "base")
            extra["dmft"] = harness.bench_dmft(steps=max(3, args.steps // 10), log=progress, only=only, variants=variants)
            result["images_per_s"] = {
                key: {v: round(extra["dmft"][key][f"{v}_images_per_s"], 1) for v in ("hip_fused_graph", "hip", "base")
                      if f"{v}_images_per_s" in extra["dmft"][key]}
                for key in ("DMFT-B/2", "DMFT-XL/2", "DMFT-XL/2 512px qk-norm") if key in extra["dmft"]}
            result["images_per_s"]["cases"] = {"DMFT-B/2": "forward+JVP, batch 64, 256px, bf16 autocast (BASELINE config 2)",
                                               "DMFT-XL/2": "forward+JVP+backward, batch 32, 256px, bf16 autocast (BASELINE config 5)",
                                               "DMFT-XL/2 512px qk-norm": "forward+JVP, batch 16, 1024 tokens, qk-norm (caller of the headline shape)"}
        except ImportError:
            pass

    if not args.no_cpu:
        progress("CPU baseline (bounded sample) ...")
        result["cpu_baseline"] = cpu_baseline(name)
        if not args.no_extra:
            result["cpu_config1"] = cpu_baseline_config1()

    if not args.no_extra:
        result["extra"] = extra     # last: the bulky detail behind the compact keys above
    print(json.dumps(result))


if __name__ == "__main__":
    main()
