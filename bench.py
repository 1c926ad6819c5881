#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload config3] [--no-secondary] [--no-cpu]

A step is one call of the hot path (ttsdpa_forward through the C ABI) over one batch of synthetic input already
resident in HBM.  The headline workload is "config3" (bf16 causal GQA prefill, B2 32q/8kv S4096 D128: the shape the
prefill throughput target is quoted on); the decode workload "config4" (bf16, B64 32q/8kv KV 8192) is measured in the
same run and reported under "secondary" and, in short, as "roofline"."decode" of the headline (the metric is prefill
TFLOP/s + decode GB/s: both halves sit in the one object), config 3's shape in fp32 (the reference's default dtype,
on the fp32 MFMA kernel, against the 157.3 TFLOP/s fp32 peak) under "fp32", and the row-wise neighbour ops (rmsNorm,
fusedAddRmsNorm, siluMul, softmax; HBM-bound) under "fused_ops" and the linear layer (QKV projection of the same
token batch; MFMA-bound) under "linear", and the attention backward (dq, dk, dv at config 3's shape; MFMA-bound) under
"backward" (bf16, and the same shape in fp32 on the fp32 matrix cores under "backward"."fp32").  One JSON line is printed.

Timing.  After the --warmup launches comes a declared, untimed settle phase (about SETTLE_SECONDS of back-to-back
launches, its length reported as "settle_launches"): the core clock of this chip takes that long to reach its level under
a kernel, and without it the first timed launches measure the ramp.  Then --steps launches are timed, each between its own
pair of HIP events on the launch stream; "kernel_ms" is the median of the launches ("kernel_ms_mean" beside it), and
"ms_per_step" / "value" come from the host clock around the same --steps launches (synchronised on both sides).
Inputs are drawn by tinytorch_amd.synth (counter-based normal generator, seed 0x5EED0000 + config number, one stream
per tensor), rounded to the workload's element type.
The other configurations of the baseline (1, 2, 5) and config 3's shape at head_dim 64 are measured the same way and
reported under "other_configs".

"roofline"."zero_operands" is the headline launch repeated on all-zero Q, K, V: the same instruction stream without operand
toggling, i.e. what the kernel's schedule reaches when the chip's power management leaves the clock alone (the prefill
kernel is power-bound on N(0,1) data: "roofline"."power" and "zero_operands"."power" hold the socket power and the
core clock the driver's sysfs files report while each of the two runs back to back, after its timed launches).
The linear and backward lines carry the same repeat as "roofline"."zero_operands_frac".
"roofline"."summary" lists the fraction of every other line of the run, and the line's last key, "in_short", repeats
the headline, decode and summary figures in a few hundred characters.

Algorithmic work per launch (what "achieved" divides by the measured launch time):
  prefill, causal:  4 * B * Hq * D * S(S+1)/2 flop   (two GEMMs over the visible triangle)
  prefill, full:    4 * B * Hq * L * S * D flop
  decode:           2 * B*Hkv*S*D*2 bytes (K and V once) + 2 * B*Hq*D*2 bytes (q in, out)
  backward, causal: 2.5 x the causal prefill's flop (five matrix products; the kernels execute seven)
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "f32": 157.3}  # MI355X dense MFMA peaks
PEAK_HBM_GBS = 8000.0
SETTLE_SECONDS = 0.4   # untimed launches after the warm-up, until the core clock has settled under the kernel
TRAFFIC_SOURCE = ("profiles/traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an earlier run of the same "
                  "command, scaled by a 1 GiB copy; not measured in this run")  # said once per line, under "traffic_source"
PROBE_LIB = os.path.join(ROOT, "bench_probes", "libttbench_probes.so")
_probe_lib = None


def probe_lib():
    """The measurement probes (bench_probes/probes.hip): a shared object of their own, not part of the product library."""
    global _probe_lib
    if _probe_lib is None:
        import torch  # noqa: F401  (one HIP runtime per process: torch's)
        if not os.path.exists(PROBE_LIB):
            raise ImportError("bench.py: %s is missing; build it with `make -C bench_probes`" % PROBE_LIB)
        L = ctypes.CDLL(PROBE_LIB)
        L.ttbench_probe.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p,
                                    ctypes.POINTER(ctypes.c_double)]
        L.ttbench_probe.restype = ctypes.c_int
        _probe_lib = L
    return _probe_lib

WORKLOADS = {
    # name: (B, Hq, Hkv, L, S, D, dtype, causal, input multiplier, bound)
    "config1": (1, 4, 4, 128, 128, 64, "f32", True, 1.0, "mfma"),
    "config2": (4, 32, 32, 2048, 2048, 128, "f16", True, 0.5, "mfma"),
    "config3": (2, 32, 8, 4096, 4096, 128, "bf16", True, 1.0, "mfma"),
    "config4": (64, 32, 8, 1, 8192, 128, "bf16", False, 1.0, "hbm"),
    "config5": (1, 28, 4, 16384, 16384, 128, "bf16", True, 1.0, "mfma"),
    "config3_f32": (2, 32, 8, 4096, 4096, 128, "f32", True, 1.0, "mfma"),  # config 3's shape in the reference's default dtype
    "config3_d64": (2, 32, 8, 4096, 4096, 64, "bf16", True, 1.0, "mfma"),   # config 3's shape at head_dim 64
    # one GPU's share of config 3 when its 8 KV heads are dealt out to 8 GPUs (no exchange between them): 128 row tiles
    "config3_share8": (2, 4, 1, 4096, 4096, 128, "bf16", True, 1.0, "mfma"),
    # config 3's shape with a Bool attnMask [L, S] instead of the causal flag (the reference's masked fill; every product is executed)
    "config3_boolmask": (2, 32, 8, 4096, 4096, 128, "bf16", False, 1.0, "mfma"),
}
MASKED = {"config3_boolmask"}  # workloads that pass an attnMask: [L, S] Bool, about 70 % of the entries set, the first key always
SEEDS = {"config1": 0x5EED0001, "config2": 0x5EED0002, "config3": 0x5EED0003, "config4": 0x5EED0004, "config5": 0x5EED0005,
         "config3_f32": 0x5EED0003, "config3_d64": 0x5EED0006, "config3_share8": 0x5EED0007, "config3_boolmask": 0x5EED0008}
DESCR = {
    "config1": "fp32 causal SDPA B1 H4 S128 D64",
    "config2": "fp16 causal MHA prefill B4 H32 S2048 D128",
    "config3": "bf16 causal GQA prefill B2 32q/8kv S4096 D128",
    "config4": "bf16 decode B64 32q/8kv L1 KV8192 D128 (isCausal=false)",
    "config5": "bf16 causal GQA prefill B1 28q/4kv S16384 D128",
    "config3_f32": "fp32 causal GQA prefill B2 32q/8kv S4096 D128",
    "config3_d64": "bf16 causal GQA prefill B2 32q/8kv S4096 D64",
    "config3_share8": "bf16 causal GQA prefill B2 4q/1kv S4096 D128 (one KV head of config 3: an 8-GPU head-sharded share)",
    "config3_boolmask": "bf16 GQA prefill B2 32q/8kv S4096 D128 with a Bool attnMask [L,S] (not causal)",
}


def algorithmic_work(B, Hq, Hkv, L, S, D, dtype, causal):
    esz = 4 if dtype == "f32" else 2
    if causal:
        vis = sum(min(i + 1, S) for i in range(L)) if L != S else S * (S + 1) // 2
        flops = 4 * B * Hq * D * vis
    else:
        flops = 4 * B * Hq * L * S * D
    nbytes = 2 * B * Hkv * S * D * esz + 2 * B * Hq * L * D * esz
    return flops, nbytes


def measured_traffic(name):
    """HBM bytes per launch of the workload's dominant kernel, as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
    (profiles/traffic.json holds the figures and the commands that produced them); None when not measured."""
    path = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        return json.load(f).get(name, {}).get("hbm_bytes_per_launch")


def time_launches(step, stream, steps, warmup, settle_seconds=None):
    """warmup untimed launches, a declared untimed settle phase, then `steps` launches each between its own pair of HIP
    events on `stream`.  Returns per-launch device times (median, mean, min; ms), the host-clock time per step around
    the timed launches, and the number of settle launches."""
    import torch

    if settle_seconds is None:
        settle_seconds = SETTLE_SECONDS
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    settle = 0
    if settle_seconds > 0:
        t_end = time.perf_counter() + settle_seconds
        while time.perf_counter() < t_end:
            for _ in range(16):
                step()
            settle += 16
            if settle % 256 == 0:
                torch.cuda.synchronize()  # keeps the launch queue (and the phase's length) bounded
        torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for e0, e1 in events:
        e0.record(stream)
        step()
        e1.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    ms = sorted(e0.elapsed_time(e1) for e0, e1 in events)
    return {"median_ms": ms[len(ms) // 2], "mean_ms": sum(ms) / len(ms), "min_ms": ms[0], "wall_ms": wall_ms,
            "settle_launches": settle}


def power_under(step, seconds=2.0):
    """Socket power and core clock while `step` is launched back to back for `seconds`, read from the driver's sysfs
    files (hwmon power1_input in microwatts, the current entry of pp_dpm_sclk; None where they are missing).  Untimed: it
    runs after the timed launches."""
    import glob
    import re
    import threading
    import torch

    pfiles = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input"))
    if not pfiles:
        return None
    pfile = pfiles[0]
    dev = pfile.split("/hwmon/")[0]
    samples, stop = [], threading.Event()

    def read(path):
        with open(path) as f:
            return f.read()

    def sampler():
        while not stop.is_set():
            try:
                watts = int(read(pfile).strip()) / 1e6
                mhz = None
                for ln in read(os.path.join(dev, "pp_dpm_sclk")).splitlines():
                    m = re.match(r"\s*\S+:\s*(\d+)\s*Mhz\s*\*", ln, re.I)
                    if m:
                        mhz = int(m.group(1))
                samples.append((watts, mhz))
            except Exception:
                pass
            time.sleep(0.05)

    th = threading.Thread(target=sampler)
    th.start()
    t_end = time.perf_counter() + seconds
    n = 0
    while time.perf_counter() < t_end:
        for _ in range(256):
            step()
        n += 256
        torch.cuda.synchronize()
    stop.set()
    th.join()
    samples = samples[len(samples) // 4:]  # the first ones see the ramp
    if not samples:
        return None
    watts = sorted(w for w, _ in samples)
    clocks = sorted(c for _, c in samples if c is not None)
    cap = None
    try:
        cap = int(read(os.path.join(os.path.dirname(pfile), "power1_cap")).strip()) / 1e6
    except Exception:
        pass
    return {"socket_power_w": round(watts[len(watts) // 2], 1), "power_cap_w": cap,
            "gfx_clock_mhz": clocks[len(clocks) // 2] if clocks else None, "samples": len(samples), "launches": n,
            "source": "sysfs hwmon power1_input and pp_dpm_sclk during back-to-back launches (medians)"}


def synth_qkv(name):
    """The workload's Q, K, V on the device: N(0,1) * multiplier from the repository's generator, rounded to its dtype."""
    import torch
    from tinytorch_amd import synth

    B, Hq, Hkv, L, S, D, dtype, causal, mul, bound = WORKLOADS[name]
    td = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype]
    seed = SEEDS[name]
    q = synth.randn(seed, 0, (B, Hq, L, D), mul).to(td)
    k = synth.randn(seed, 1, (B, Hkv, S, D), mul).to(td)
    v = synth.randn(seed, 2, (B, Hkv, S, D), mul).to(td)
    return q, k, v


def synth_mask(name):
    """The workload's attnMask on the device (None unless it has one): uniform numbers from the same generator, set where
    below 0.7 of the unit normal's range; key 0 visible to every row."""
    if name not in MASKED:
        return None
    from tinytorch_amd import synth
    B, Hq, Hkv, L, S, D, dtype, causal, mul, bound = WORKLOADS[name]
    m = synth.randn(SEEDS[name], 7, (L, S)) < 0.5244  # P(N(0,1) < 0.5244) = 0.70
    m[:, 0] = True
    return m


def run_gpu(name, steps, warmup, zero_inputs=False, power=False):
    import torch
    from tinytorch_amd import _capi, build_params

    B, Hq, Hkv, L, S, D, dtype, causal, mul, bound = WORKLOADS[name]
    q, k, v = synth_qkv(name)
    if zero_inputs:  # the same launch without operand toggling
        q.zero_(), k.zero_(), v.zero_()
    out = torch.empty_like(q)
    mask = synth_mask(name)
    p = build_params(q, k, v, out, causal, mask)
    lib = _capi.lib()
    rc, route = _capi.plan(p)
    assert rc == 0, _capi.status_string(rc)
    nbytes = lib.ttsdpa_workspace_bytes(ctypes.byref(p))
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream()

    def step():
        rc = lib.ttsdpa_forward(ctypes.byref(p), ws.data_ptr(), nbytes, stream.cuda_stream)
        if rc != 0:
            raise RuntimeError("ttsdpa_forward: %s" % _capi.status_string(rc))

    t = time_launches(step, stream, steps, warmup)
    wall_ms, dev_ms = t["wall_ms"], t["median_ms"]  # HIP events on the launch stream, one pair per launch: the median

    flops, abytes = algorithmic_work(B, Hq, Hkv, L, S, D, dtype, causal)
    if bound == "mfma":
        achieved, peak, unit = flops / (dev_ms * 1e-3) / 1e12, PEAK_TFLOPS[dtype], "TFLOP/s"
        value = flops / (wall_ms * 1e-3) / 1e12
    else:
        achieved, peak, unit = abytes / (dev_ms * 1e-3) / 1e9, PEAK_HBM_GBS, "GB/s"
        value = abytes / (wall_ms * 1e-3) / 1e9
    res = {
        "workload": name, "description": DESCR[name], "route": _capi.ROUTE_NAMES[route], "dtype": dtype,
        "value": round(value, 3), "unit": unit, "ms_per_step": round(wall_ms, 5),
        "roofline": {"bound": bound, "achieved": round(achieved, 3), "peak": peak, "unit": unit,
                     "frac": round(achieved / peak, 4), "traffic": measured_traffic(name),
                     "kernel_ms": round(dev_ms, 5), "kernel_ms_mean": round(t["mean_ms"], 5),
                     "kernel_ms_min": round(t["min_ms"], 5), "timing": "median of %d launches, one HIP event pair each" % steps,
                     "settle_launches": t["settle_launches"], "algorithmic_flops": flops, "algorithmic_bytes": abytes},
    }
    if power:  # what the chip's power management does under this launch (after the timed region)
        res["roofline"]["power"] = power_under(step)
    return res, (q, k, v, out, mask)


def run_probes():
    """What this GPU sustains on the two bounding resources, measured with the probe kernels of bench_probes/ (a shared
    object of their own): a register-only MFMA loop on constant and on random operands, and a streaming read of 1 GiB,
    plain and nontemporal.  HIP events on the launch stream."""
    import torch

    lib = probe_lib()
    stream = torch.cuda.current_stream()
    buf = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
    out = {}
    for key, kind, iters, reps, unit in (("mfma_loop", 0, 20000, 300, 1e12), ("mfma_loop_random", 3, 20000, 300, 1e12),
                                         ("read_plain", 1, 1, 300, 1e9), ("read_nontemporal", 2, 1, 300, 1e9)):
        work = ctypes.c_double(0.0)

        def go():
            rc = lib.ttbench_probe(kind, buf.data_ptr(), buf.numel(), iters, stream.cuda_stream, ctypes.byref(work))
            if rc != 0:
                raise RuntimeError("ttbench_probe: status %d" % rc)
        for _ in range(reps):
            go()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(reps):
            go()
        e1.record(stream)
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        out[key] = round(work.value / (ms * 1e-3) / unit, 1)
    del buf
    torch.cuda.empty_cache()
    return {"mfma_loop_tflops": out["mfma_loop"], "mfma_loop_random_operands_tflops": out["mfma_loop_random"],
            "read_plain_gbs": out["read_plain"], "read_nontemporal_gbs": out["read_nontemporal"],
            "note": "sustained by the bench_probes kernels in this run: register-only bf16 32x32x16 MFMA loop on constant and on "
                    "random operands (the chip lowers its clock under the latter), 1 GiB streaming reads"}


FUSED_WORKLOADS = {
    # name: (op, rows, dim) — bf16, sized well beyond the 256 MB last-level cache so that the figure is HBM traffic
    "rms_norm": ("rms_norm", 65536, 4096),            # [B16 x S4096 tokens, hidden 4096]
    "fused_add_rms_norm": ("add_rms_norm", 65536, 4096),
    "silu_mul": ("silu_mul", 32768, 14336),           # gate/up rows of 2 x 14336
    "softmax": ("softmax", 8192, 32000),              # logits rows
}


def run_fused(name, steps, warmup, cpu=True):
    """One row-wise neighbour op (include/ttfused.h) on bf16 rows resident in HBM: algorithmic bytes per launch / HIP-event
    time per launch against the 8 TB/s HBM peak, with the compiled reference (one core) on the first rows beside it.
    Algorithmic bytes: rms_norm and softmax read and write every element once (2 n e), fused_add_rms_norm reads and
    writes two tensors (4 n e), silu_mul reads two halves and writes one (3 n e); e = 2 bytes."""
    import numpy as np
    import torch
    from tinytorch_amd import _capi

    op, rows, dim = FUSED_WORKLOADS[name]
    lib = _capi.lib()
    stream = torch.cuda.current_stream()
    st = stream.cuda_stream
    gen = torch.Generator(device="cuda").manual_seed(0x5EED)
    cols = 2 * dim if op == "silu_mul" else dim
    x = torch.randn(rows, cols, device="cuda", generator=gen).bfloat16()
    w = torch.randn(dim, device="cuda", generator=gen).bfloat16()
    n = rows * dim
    if op == "rms_norm":
        out = torch.empty_like(x)
        step = lambda: lib.ttfused_rms_norm(_capi.BF16, x.data_ptr(), w.data_ptr(), out.data_ptr(), rows, dim, 1e-6, st)
        abytes = 2 * n * 2
    elif op == "add_rms_norm":
        res = torch.randn(rows, dim, device="cuda", generator=gen).bfloat16()
        x0, r0 = x[:64].clone(), res[:64].clone()
        step = lambda: lib.ttfused_add_rms_norm(_capi.BF16, x.data_ptr(), res.data_ptr(), w.data_ptr(), rows, dim, 1e-6, st)
        abytes = 4 * n * 2
    elif op == "silu_mul":
        out = torch.empty(rows, dim, device="cuda", dtype=torch.bfloat16)
        step = lambda: lib.ttfused_silu_mul(_capi.BF16, x.data_ptr(), out.data_ptr(), rows, dim, st)
        abytes = 3 * n * 2
    else:
        out = torch.empty_like(x)
        step = lambda: lib.ttfused_softmax(_capi.BF16, x.data_ptr(), out.data_ptr(), rows, dim, 1, 0, st)
        abytes = 2 * n * 2
    rc = step()
    if rc != 0:
        raise RuntimeError("%s: %s" % (name, _capi.status_string(rc)))
    torch.cuda.synchronize()
    first = None
    if op == "add_rms_norm":
        first = (x[:64].float().cpu().numpy(), res[:64].float().cpu().numpy())  # before further in-place passes
    t = time_launches(step, stream, steps, warmup)
    ms = t["median_ms"]
    res_line = {"workload": "%s bf16 [%d, %d]" % (name, rows, cols), "dtype": "bf16", "ms_per_step": round(ms, 5),
                "kernel_ms_mean": round(t["mean_ms"], 5), "settle_launches": t["settle_launches"],
                "roofline": {"bound": "hbm", "achieved": round(abytes / (ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                             "unit": "GB/s", "frac": round(abytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                             "traffic": measured_traffic(name), "algorithmic_bytes": abytes}}
    if cpu:
        import oracle
        kind = "reference" if oracle.have_ref() else "port"
        take = 64
        xh = (x0 if op == "add_rms_norm" else x[:take]).float().cpu().numpy()
        wh = w.float().cpu().numpy()
        t0 = time.perf_counter()
        reps = 0
        while True:
            if op == "rms_norm":
                ref = (oracle.ref_rms_norm if kind == "reference" else oracle.rms_norm)(xh, wh, 1e-6)
                got = out[:take].float().cpu().numpy()
            elif op == "add_rms_norm":
                rh = r0.float().cpu().numpy()
                ref = (oracle.ref_fused_add_rms_norm if kind == "reference" else oracle.fused_add_rms_norm)(xh, rh, wh, 1e-6)[0]
                got = first[0]
            elif op == "silu_mul":
                ref = (oracle.ref_silu_mul if kind == "reference" else oracle.silu_mul)(xh)
                got = out[:take].float().cpu().numpy()
            else:
                ref = (oracle.ref_softmax if kind == "reference" else oracle.softmax)(xh, -1)
                got = out[:take].float().cpu().numpy()
            reps += 1
            spent = time.perf_counter() - t0
            if spent > 1.0:
                break
        frac_bytes = abytes * take / rows
        res_line["cpu_baseline"] = {"value": float("%.4g" % (frac_bytes * reps / spent / 1e9)), "unit": "GB/s", "cores": 1,
                                    "kind": kind, "sample": "the first %d rows, %d passes in %.1f s, one thread (fp32 on the bf16 values)"
                                    % (take, reps, spent),
                                    "max_abs_err_gpu_vs_cpu": float("%.3g" % float(np.abs(ref - got).max()))}
    return res_line


LINEAR_WORKLOAD = (8192, 6144, 4096)  # config 3's token batch through the fused QKV projection: [B2 x S4096, 4096] -> 6144


def run_linear(steps, warmup, cpu=True):
    """The linear layer (include/ttlinear.h) at the QKV projection of config 3's token batch, bf16: 2*M*N*K flop per
    launch / HIP-event time per launch against the bf16 MFMA peak, the compiled reference (one core) on a slice beside it."""
    import numpy as np
    import torch
    from tinytorch_amd import _capi

    M, N, K = LINEAR_WORKLOAD
    lib = _capi.lib()
    stream = torch.cuda.current_stream()
    gen = torch.Generator(device="cuda").manual_seed(0x5EED)
    x = torch.randn(M, K, device="cuda", generator=gen).bfloat16()
    w = (torch.randn(N, K, device="cuda", generator=gen) * K ** -0.5).bfloat16()
    b = torch.randn(N, device="cuda", generator=gen).bfloat16()
    out = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)

    def step():
        rc = lib.ttlinear_forward(_capi.BF16, x.data_ptr(), w.data_ptr(), b.data_ptr(), out.data_ptr(), M, N, K, K, K, N,
                                  stream.cuda_stream)
        if rc != 0:
            raise RuntimeError("ttlinear_forward: %s" % _capi.status_string(rc))
    t = time_launches(step, stream, steps, warmup)
    ms = t["median_ms"]
    flops = 2 * M * N * K
    res = {"workload": "linear bf16 x[%d,%d] . w[%d,%d]^T + bias" % (M, K, N, K), "dtype": "bf16", "ms_per_step": round(ms, 5),
           "kernel_ms_mean": round(t["mean_ms"], 5), "settle_launches": t["settle_launches"],
           "roofline": {"bound": "mfma", "achieved": round(flops / (ms * 1e-3) / 1e12, 1), "peak": PEAK_TFLOPS["bf16"],
                        "unit": "TFLOP/s", "frac": round(flops / (ms * 1e-3) / 1e12 / PEAK_TFLOPS["bf16"], 4),
                        "traffic": measured_traffic("linear"), "algorithmic_flops": flops,
                        "algorithmic_bytes": 2 * (M * K + N * K + M * N + N)}}
    if cpu:
        import oracle
        kind = "reference" if oracle.have_ref() else "port"
        rows, cols = 16, 256
        xh = x[:rows].float().cpu().numpy()
        wh = w[:cols].float().cpu().numpy()
        bh = b[:cols].float().cpu().numpy()
        fn = oracle.ref_linear if kind == "reference" else oracle.linear
        fn(xh[:1], wh[:1], bh[:1])  # the library's one-time set-up stays out of the timing
        t0 = time.perf_counter()
        reps = 0
        while True:
            ref = fn(xh, wh, bh)
            reps += 1
            spent = time.perf_counter() - t0
            if spent > 1.0:
                break
        got = out[:rows, :cols].float().cpu().numpy()
        res["cpu_baseline"] = {"value": float("%.4g" % (2.0 * rows * cols * K * reps / spent / 1e12)), "unit": "TFLOP/s", "cores": 1,
                               "kind": kind, "sample": "a [%d, %d] corner of the output, %d passes in %.1f s, one thread (fp32 on the bf16 values)"
                               % (rows, cols, reps, spent),
                               "max_abs_err_gpu_vs_cpu": float("%.3g" % float(np.abs(ref - got).max()))}
    # the same launch on all-zero operands: what the kernel's schedule reaches without the power its data draws
    x.zero_(), w.zero_(), b.zero_()
    tz = time_launches(step, stream, steps, warmup)
    res["roofline"]["zero_operands_frac"] = round(flops / (tz["median_ms"] * 1e-3) / 1e12 / PEAK_TFLOPS["bf16"], 4)
    return res


def run_backward(steps, warmup, cpu=True, dtype="bf16"):
    """Attention backward (ttsdpa_backward) at config 3's shape, causal, bf16 or fp32 (the reference's default dtype, on
    the fp32 matrix cores): dq, dk, dv per launch pair.  Flop count: the textbook five matrix products (2.5 x the
    forward's), halved by the causal mask; the two kernels execute seven."""
    import ctypes
    import numpy as np
    import torch
    from tinytorch_amd import _capi, build_backward_params, sdpAttention

    B, Hq, Hkv, L, S, D = 2, 32, 8, 4096, 4096, 128
    lib = _capi.lib()
    stream = torch.cuda.current_stream()
    from tinytorch_amd import synth
    td = torch.bfloat16 if dtype == "bf16" else torch.float32
    q = synth.randn(0x5EED0003, 0, (B, Hq, L, D)).to(td)
    k = synth.randn(0x5EED0003, 1, (B, Hkv, S, D)).to(td)
    v = synth.randn(0x5EED0003, 2, (B, Hkv, S, D)).to(td)
    go = synth.randn(0x5EED0003, 3, (B, Hq, L, D)).to(td)
    out = sdpAttention(q, k, v, isCausal=True)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    bp = build_backward_params(q, k, v, out, go, dq, dk, dv, True)
    nbytes = lib.ttsdpa_backward_workspace_bytes(ctypes.byref(bp))
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device="cuda")
    route = ctypes.c_int(-1)
    lib.ttsdpa_backward_plan(ctypes.byref(bp), ctypes.byref(route))

    def step():
        rc = lib.ttsdpa_backward(ctypes.byref(bp), ws.data_ptr(), nbytes, stream.cuda_stream)
        if rc != 0:
            raise RuntimeError("ttsdpa_backward: %s" % _capi.status_string(rc))
    t = time_launches(step, stream, steps, warmup)
    ms = t["median_ms"]
    flops = 2.5 * 4.0 * B * Hq * L * S * D * 0.5
    tf = flops / (ms * 1e-3) / 1e12
    kernels = "backward_dq128_kernel + backward_dkv128_kernel" if dtype == "bf16" else "backward_dq_f32_kernel + backward_dkv_f32_kernel"
    res = {"workload": "attention backward %s B%d %dq/%dkv L=S=%d D%d causal" % (dtype, B, Hq, Hkv, L, D), "dtype": dtype,
           "route": _capi.ROUTE_NAMES[route.value], "ms_per_step": round(ms, 5), "kernel_ms_mean": round(t["mean_ms"], 5),
           "settle_launches": t["settle_launches"], "value": round(tf, 1), "unit": "TFLOP/s",
           "roofline": {"bound": "mfma", "achieved": round(tf, 1), "peak": PEAK_TFLOPS[dtype], "unit": "TFLOP/s",
                        "frac": round(tf / PEAK_TFLOPS[dtype], 4),
                        "traffic": measured_traffic("backward" if dtype == "bf16" else "backward_f32"),
                        "algorithmic_flops": flops, "kernels": kernels + " per step"}}
    if cpu:
        import oracle
        # the causal top-left corner is a problem of its own for dq: rows below n see keys below n only
        n = 2048
        qh, kh, vh, gh = (t[:1, :h, :n].float().cpu().numpy() for t, h in ((q, Hq // Hkv), (k, 1), (v, 1), (go, Hq // Hkv)))
        t0 = time.perf_counter()
        rq, _, _ = oracle.sdpa_backward_f32(qh, kh, vh, gh, causal=True, nthreads=1)
        spent = time.perf_counter() - t0
        got = dq[:1, :Hq // Hkv, :n].float().cpu().numpy()
        res["cpu_baseline"] = {"value": float("%.4g" % (2.5 * 4.0 * (Hq // Hkv) * n * n * D * 0.5 / spent / 1e12)), "unit": "TFLOP/s",
                               "cores": 1, "kind": "port",
                               "sample": "the first %d queries x %d keys of one KV head (its %d query heads), %.1f s, one thread, double accumulation"
                               % (n, n, Hq // Hkv, spent),
                               "max_abs_err_gpu_vs_cpu_dq": float("%.3g" % float(np.abs(rq - got).max()))}
    if dtype == "bf16":  # the same launches on all-zero tensors (as for the forward: the share of the power limit)
        for t_ in (q, k, v, go, out):
            t_.zero_()
        tz = time_launches(step, stream, steps, warmup)
        res["roofline"]["zero_operands_frac"] = round(flops / (tz["median_ms"] * 1e-3) / 1e12 / PEAK_TFLOPS[dtype], 4)
    return res


def run_cpu_baseline(name, tensors, budget_s=20.0, corner=None):
    """The reference CPU path (compiled reference if oracle/_ref is present, else this repository's C restatement)
    on one host core, over as many (batch, head) slices of the same inputs as fit the time budget.  corner=n (causal
    workloads with L == S): only the first n queries against the first n keys of a slice, which under the top-left
    aligned mask is an attention problem of its own (rows below n see keys below n only)."""
    import numpy as np
    import oracle

    B, Hq, Hkv, L, S, D, dtype, causal, mul, bound = WORKLOADS[name]
    q, k, v, out, mask = tensors
    mask_h = None if mask is None else mask.cpu().numpy().astype(np.uint8)
    kind = "reference" if oracle.have_ref() else "port"
    fn = oracle.ref_sdpa_f32 if kind == "reference" else (lambda *a, **kw: oracle.sdpa_f32(*a, nthreads=1, **kw))
    G = Hq // Hkv
    if corner is not None:
        assert causal and L == S
        L = S = min(corner, L)
    flops_slice, _ = algorithmic_work(1, 1, 1, L, S, D, dtype, causal)
    done, spent, worst = 0, 0.0, 0.0
    slices = [(b, h) for b in range(B) for h in range(Hq)]
    for (b, h) in slices:
        qs = q[b:b + 1, h:h + 1, :L].float().cpu().numpy()
        ks = k[b:b + 1, h // G:h // G + 1, :S].float().cpu().numpy()
        vs = v[b:b + 1, h // G:h // G + 1, :S].float().cpu().numpy()
        t0 = time.perf_counter()
        ref = fn(qs, ks, vs, causal=causal) if mask_h is None else fn(qs, ks, vs, causal=causal, mask=mask_h)
        dt = time.perf_counter() - t0
        err = float(np.abs(ref - out[b:b + 1, h:h + 1, :L].float().cpu().numpy()).max())
        worst = max(worst, err)
        done += 1
        spent += dt
        if spent + dt > budget_s:
            break
    if bound == "mfma":
        val, unit = flops_slice * done / spent / 1e12, "TFLOP/s"
    else:
        esz = 4 if dtype == "f32" else 2
        slice_bytes = (2 * S * D * esz) / G + 2 * L * D * esz  # a query head's share of its KV head + q + out
        val, unit = slice_bytes * done / spent / 1e9, "GB/s"
    return {"value": float("%.4g" % val), "unit": unit, "cores": 1, "host_cores": os.cpu_count(), "kind": kind,
            "sample": "%d of %d (batch, head) slices of the same inputs%s, %.1f s, one thread%s"
                      % (done, len(slices), "" if corner is None else " (their first %d queries x %d keys)" % (L, S), spent,
                         "; whole-job estimate %.1f s" % (spent / done * len(slices)) if corner is None else ""),
            "max_abs_err_gpu_vs_cpu": float("%.3g" % worst)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="config3", choices=sorted(WORKLOADS))
    ap.add_argument("--secondary", default="config4", choices=sorted(WORKLOADS))
    ap.add_argument("--no-secondary", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--no-probes", action="store_true", help="skip the hardware ceiling probes")
    ap.add_argument("--no-zero", action="store_true", help="skip the repeat of the headline launch on all-zero operands")
    ap.add_argument("--no-power", action="store_true", help="skip the socket power / core clock samples of the headline launch")
    ap.add_argument("--zero-inputs", action="store_true",
                    help="run the workload on all-zero Q, K, V only (for profiling the same instruction stream without operand toggling)")
    ap.add_argument("--settle", type=float, default=None,
                    help="seconds of untimed launches after the warm-up (default %.1f; 0 for counter runs that only need a few dispatches)" % SETTLE_SECONDS)
    ap.add_argument("--no-other", action="store_true", help="skip the baseline's other configurations (1, 2, 5) and head_dim 64")
    ap.add_argument("--no-fused", action="store_true", help="skip the row-wise neighbour ops (rmsNorm, siluMul, ...)")
    ap.add_argument("--fused-only", default=None, choices=sorted(FUSED_WORKLOADS),
                    help="measure one row-wise op only and print its line (for profiling)")
    ap.add_argument("--linear-only", action="store_true", help="measure the linear layer only and print its line (for profiling)")
    ap.add_argument("--backward-only", action="store_true", help="measure the attention backward only and print its line (for profiling)")
    ap.add_argument("--backward-dtype", choices=["bf16", "f32"], default="bf16", help="element type for --backward-only")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run one device-to-device copy of 1 GiB (a kernel of known traffic that calibrates "
                         "FETCH_SIZE / WRITE_SIZE when this command runs under rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.settle is not None:
        globals()["SETTLE_SECONDS"] = max(0.0, args.settle)
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the attention path shards by batch / KV head with no "
                 "exchange; no multi-GPU figure is produced). Run with --gpus 1.")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback.")

    if args.copy_probe:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.fused_only:
        print(json.dumps(run_fused(args.fused_only, args.steps, args.warmup, cpu=not args.no_cpu)), flush=True)
        return
    if args.linear_only:
        print(json.dumps(run_linear(args.steps, args.warmup, cpu=not args.no_cpu)), flush=True)
        return
    if args.backward_only:
        print(json.dumps(run_backward(args.steps, args.warmup, cpu=not args.no_cpu and args.backward_dtype == "bf16",
                                      dtype=args.backward_dtype)), flush=True)
        return
    main_res, tensors = run_gpu(args.workload, args.steps, args.warmup, zero_inputs=args.zero_inputs, power=not args.no_power)
    ceilings = None if args.no_probes else run_probes()
    cpu = None if args.no_cpu else run_cpu_baseline(args.workload, tensors, args.cpu_seconds)
    del tensors
    torch.cuda.empty_cache()
    main_res["roofline"]["traffic_source"] = TRAFFIC_SOURCE  # for every "traffic" figure of this line
    if not args.no_zero and not args.zero_inputs and WORKLOADS[args.workload][9] == "mfma":
        # the same launch on all-zero operands: the instruction stream without operand toggling (the kernel is power-bound
        # on N(0,1) data: the chip lowers its clock under it)
        z, tensors = run_gpu(args.workload, args.steps, args.warmup, zero_inputs=True, power=not args.no_power)
        del tensors
        torch.cuda.empty_cache()
        main_res["roofline"]["zero_operands"] = {
            "kernel_ms": z["roofline"]["kernel_ms"], "achieved": z["roofline"]["achieved"], "frac": z["roofline"]["frac"],
            "power": z["roofline"].get("power"),
            "note": "the same launch with Q = K = V = 0: identical instruction stream, no operand toggling; not a result, "
                    "the clock the power management grants is the difference"}
    summary = {}
    line = {
        "metric": "attn prefill TFLOP/s + decode KV GB/s on 1 MI355X (% of roofline)",
        "value": main_res["value"], "unit": main_res["unit"], "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": main_res["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": main_res["dtype"], "data": "synthetic (tinytorch_amd.synth: counter-based N(0,1), seed 0x5EED0000 + config number, a stream per tensor)",
        "config": {"workload": "%s: %s" % (args.workload, main_res["description"]), "route": main_res["route"]},
        "roofline": main_res["roofline"], "cpu_baseline": cpu,
    }
    if ceilings:
        line["measured_ceilings"] = ceilings
    if not args.no_secondary and args.secondary != args.workload:
        sec, tensors = run_gpu(args.secondary, args.steps, args.warmup)
        sec["cpu_baseline"] = None if args.no_cpu else run_cpu_baseline(args.secondary, tensors, args.cpu_seconds)
        del tensors
        line["secondary"] = sec
        if args.secondary == "config4":  # the metric's second half, inside the object that is kept whole
            r = sec["roofline"]
            line["roofline"]["decode"] = {
                "workload": "config4: " + sec["description"], "bound": r["bound"], "achieved": r["achieved"], "peak": r["peak"],
                "unit": r["unit"], "frac": r["frac"], "kernel_ms": r["kernel_ms"], "traffic": r["traffic"],
                "algorithmic_bytes": r["algorithmic_bytes"], "settle_launches": r["settle_launches"],
                "cpu_baseline": sec["cpu_baseline"]}
        if args.workload == "config3":  # the same shape in fp32, against the fp32 MFMA peak (no CPU leg: same arithmetic as config 3's)
            f32, tensors = run_gpu("config3_f32", max(1, min(args.steps, 100)), min(args.warmup, 20))
            del tensors
            line["fp32"] = f32
            summary["config3_f32"] = f32["roofline"]["frac"]
    if not args.no_other and args.workload == "config3":
        # the baseline's other configurations (config 1: launch-sized, its time is the figure) and head_dim 64
        line["other_configs"] = []
        for name, corner, budget in (("config1", None, 2.0), ("config2", None, 4.0), ("config5", 4096, 4.0),
                                     ("config3_d64", 2048, 3.0), ("config3_share8", 2048, 2.0), ("config3_boolmask", None, 3.0)):
            torch.cuda.empty_cache()
            res, tensors = run_gpu(name, max(1, min(args.steps, 50)), min(args.warmup, 20))
            if not args.no_cpu:
                res["cpu_baseline"] = run_cpu_baseline(name, tensors, budget, corner)
            del tensors
            line["other_configs"].append(res)
            summary[name] = res["roofline"]["kernel_ms"] if name == "config1" else res["roofline"]["frac"]
    if not args.no_fused:
        torch.cuda.empty_cache()
        line["fused_ops"] = [run_fused(n, max(1, min(args.steps, 100)), min(args.warmup, 20), cpu=not args.no_cpu)
                             for n in ("rms_norm", "fused_add_rms_norm", "silu_mul", "softmax")]
        torch.cuda.empty_cache()
        line["linear"] = run_linear(max(1, min(args.steps, 100)), min(args.warmup, 50), cpu=not args.no_cpu)
        torch.cuda.empty_cache()
        line["backward"] = run_backward(max(1, min(args.steps, 50)), min(args.warmup, 20), cpu=not args.no_cpu)
        line["backward"]["fp32"] = run_backward(max(1, min(args.steps, 10)), min(args.warmup, 3), cpu=False, dtype="f32")
        for r in line["fused_ops"]:
            summary[r["workload"].split()[0]] = r["roofline"]["frac"]
        summary["linear"] = line["linear"]["roofline"]["frac"]
        summary["linear_zero_operands"] = line["linear"]["roofline"]["zero_operands_frac"]
        summary["backward_bf16"] = line["backward"]["roofline"]["frac"]
        summary["backward_bf16_zero_operands"] = line["backward"]["roofline"]["zero_operands_frac"]
        summary["backward_f32"] = line["backward"]["fp32"]["roofline"]["frac"]
    if summary:  # fraction of its own roofline for every other line of this run (config1: launch-sized, its kernel ms)
        line["roofline"]["summary"] = summary
    # said once, in the headline's roofline object: how every line is timed; the secondary line's figures sit in roofline.decode
    for other in [line.get("secondary"), line.get("fp32")] + list(line.get("other_configs", [])):
        if other:
            for key in ("timing", "kernel_ms_mean", "kernel_ms_min"):
                other["roofline"].pop(key, None)
    if "decode" in line["roofline"] and "secondary" in line:
        line["secondary"] = {"workload": line["secondary"]["workload"], "route": line["secondary"]["route"],
                             "ms_per_step": line["secondary"]["ms_per_step"], "value": line["secondary"]["value"],
                             "unit": line["secondary"]["unit"], "roofline": "see roofline.decode of the headline"}
    # the figures the metric is quoted on once more as the line's last key: a record that keeps only the end of a
    # long line still holds them
    r = line["roofline"]
    line["in_short"] = {"prefill_%s" % args.workload: {"frac": r["frac"], "kernel_ms": r["kernel_ms"], "achieved": r["achieved"], "unit": r["unit"]}}
    if "zero_operands" in r:
        line["in_short"]["prefill_%s_zero_operands_frac" % args.workload] = r["zero_operands"]["frac"]
    pw, zpw = r.get("power"), r.get("zero_operands", {}).get("power")
    if pw and zpw:
        line["in_short"]["socket_power_w_and_gfx_mhz"] = {
            "n01_operands": [pw["socket_power_w"], pw["gfx_clock_mhz"]],
            "zero_operands": [zpw["socket_power_w"], zpw["gfx_clock_mhz"]], "power_cap_w": pw["power_cap_w"]}
    if "decode" in r:
        d = r["decode"]
        line["in_short"]["decode_config4"] = {"frac": d["frac"], "kernel_ms": d["kernel_ms"], "achieved": d["achieved"], "unit": d["unit"]}
    if summary:
        line["in_short"]["frac_of_other_lines"] = summary
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
