"""Benchmark of the fused MoE-layer forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]
                    [--power-seconds S] [--zero-expert-weights] [--calib-gemm M,N,K] [--calib-mfma]

A step is one forward of the layer (one persistent kernel launch) over one batch of synthetic
tokens already resident in HBM. The per-phase figures are measured first, with launch counts of
their own (72 phased forwards, 1568 persistent ones: about half a second of sustained load, after
which the device holds the clocks it keeps in a serving loop; it takes some 0.4 s to get there and
loses them within milliseconds of idling); then come the timed region proper: `warmup`
forwards and exactly `steps` forwards between two readings of the wall clock. Prints one JSON line: latency per forward, the roofline of the
launch (the workload's arithmetic intensity decides which roof binds: algorithmic bytes / event-timed
duration against HBM peak, with the matrix-core fraction beside it), per-phase figures from the
phased mode, and the CPU oracle timed on this box's host cores as a baseline. After the timed region
the forwards keep running for `--power-seconds` while a thread reads the socket power (`power`): all
of these workloads hold the package at its 1400 W cap, and so does the vendor's GEMM (`--calib-gemm`).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA
PEAK_FP32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0


def source_fingerprint() -> str:
    """First 16 hex digits of the SHA-256 over the library's device and host sources: what a
    committed counter summary was measured on."""
    import hashlib
    csrc = os.path.join(ROOT, "aristos_amd", "csrc")
    h = hashlib.sha256()
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".hpp", ".cpp")):
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload: str):
    """HBM bytes per launch of the persistent kernel as the committed rocprofv3 summary of this
    workload states them (FETCH_SIZE and WRITE_SIZE passes, each scaled by what the counter reads
    for a copy of known size): counters cannot be read inside a timed run. Returns (bytes or None,
    whether the summary was made from the sources this run uses)."""
    import re
    path = os.path.join(ROOT, "profiles", f"fused_kernel_{workload}_hbm_traffic.txt")
    if not os.path.exists(path):
        return None, None
    text = open(path).read()
    m = re.search(r"=\s*([0-9.]+) GB of HBM traffic per launch", text)
    if not m:
        return None, None
    fp = re.search(r"source fingerprint:\s*([0-9a-f]{16})", text)
    return float(m.group(1)) * 1e9, bool(fp and fp.group(1) == source_fingerprint())


class PowerSampler:
    """Socket power while a load runs, read from the amdgpu hwmon node (power1_input, microwatts)
    every 0.2 s by a thread. MI355X caps the package at power1_cap (1400 W); a load that sits at the
    cap runs at whatever clocks that power buys, so its duration follows the energy it needs."""

    def __init__(self):
        import glob
        nodes = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input"))
        self.path = nodes[0] if nodes else None
        self.samples, self._stop, self._thread = [], False, None

    @staticmethod
    def _read(path):
        try:
            with open(path) as f:
                return int(f.read().strip()) / 1e6
        except (OSError, ValueError):
            return None

    def cap_w(self):
        return self._read(self.path.replace("power1_input", "power1_cap")) if self.path else None

    def start(self):
        import threading
        if not self.path:
            return

        def run():
            while not self._stop:
                v = self._read(self.path)
                if v is not None:
                    self.samples.append((time.perf_counter(), v))
                time.sleep(0.2)
        self._thread = threading.Thread(target=run, daemon=True)
        self._thread.start()

    def stop(self, since: float):
        """Mean and maximum of the samples taken after `since` (perf_counter seconds)."""
        self._stop = True
        if self._thread:
            self._thread.join()
        vals = [v for t, v in self.samples if t >= since]
        if not vals:
            return None
        return {"mean_w": round(sum(vals) / len(vals), 1), "max_w": round(max(vals), 1), "samples": len(vals),
                "cap_w": self.cap_w(), "source": self.path}


def sustained_power(seconds: float, launch_some) -> dict | None:
    """Runs `launch_some()` (a few dozen milliseconds of back-to-back work that ends synchronised)
    for `seconds` and returns the socket power over all but the first 1.5 s."""
    ps = PowerSampler()
    ps.start()
    t0 = time.perf_counter()
    n = 0
    while time.perf_counter() - t0 < seconds:
        launch_some()
        n += 1
    out = ps.stop(t0 + 1.5)
    if out is not None:
        out["seconds"] = round(time.perf_counter() - t0, 2)
    return out


def vendor_gemm_calibration(shape: str, seconds: float, zero_a: bool) -> int:
    """`--calib-gemm M,N,K`: the vendor's bf16 GEMM (torch `a @ b.T`, hipBLASLt) on random operands
    of one projection's shape, looped for `seconds`: TFLOP/s and socket power. What another kernel
    reaches on this box, this data and this power cap; not part of the library."""
    import torch
    M, N, K = (int(v) for v in shape.split(","))
    a = torch.randn(M, K, device="cuda", dtype=torch.bfloat16) * 0.5
    b = torch.randn(N, K, device="cuda", dtype=torch.bfloat16) * 0.02
    if zero_a:
        a.zero_()
    c = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
    torch.matmul(a, b.T, out=c)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = max(1, int(0.05 / (2.0 * M * N * K / 1.2e15)))
    rates = []

    def some():
        ev0.record()
        for _ in range(reps):
            torch.matmul(a, b.T, out=c)
        ev1.record()
        torch.cuda.synchronize()
        rates.append(2.0 * M * N * K * reps / (ev0.elapsed_time(ev1) * 1e-3) / 1e12)
    power = sustained_power(max(3.0, seconds), some)
    tail = rates[len(rates) // 2:]
    print(json.dumps({"calibration": "vendor bf16 GEMM (torch matmul, a @ b.T)", "M": M, "N": N, "K": K,
                      "a_zeroed": zero_a, "tflops": round(sum(tail) / len(tail), 1),
                      "mfma_frac": round(sum(tail) / len(tail) / PEAK_BF16_TFLOPS, 4), "power": power}))
    return 0


def mfma_calibration(seconds: float, zero: bool) -> int:
    """`--calib-mfma`: the library's matrix-instruction probe (bf16 operands held in registers, no
    memory traffic) looped for `seconds` per instruction: what the matrix cores sustain, at which
    socket power, with 32x32x16 and with 16x16x32 instructions. One JSON line per instruction."""
    import aristos_amd as ka
    for tile in (32, 16, 32, 16):
        rates = []
        power = sustained_power(max(3.0, seconds), lambda: rates.append(ka.moe.debug_mfma_probe(tile, 20000, zero)["tflops"]))
        tail = rates[len(rates) // 2:]
        tf = sum(tail) / len(tail)
        print(json.dumps({"calibration": "bf16 matrix instructions on register operands, all CUs",
                          "instruction": "v_mfma_f32_32x32x16_bf16" if tile == 32 else "v_mfma_f32_16x16x32_bf16",
                          "operands": "zeros" if zero else "random values of unit size", "tflops": round(tf, 1),
                          "mfma_frac": round(tf / PEAK_BF16_TFLOPS, 4), "power": power,
                          "joule_per_tflop": round(power["mean_w"] / tf, 4) if power else None}))
    return 0


PHASED_SKIP, FUSED_SKIP, REHEARSALS = 8, 32, 3


def prewarm_protocol(steps: int, warmup: int, pass_ms):
    """What runs before the timed region, spelled out for the JSON line: the launches of the
    per-phase measurements (phased and persistent), the rehearsal passes of the whole
    `warmup` + `steps` pattern, and the per-step latency every pass measured. The first pass is what
    a caller sees who runs `warmup` + `steps` from cold; the last one is `value`."""
    phased = PHASED_SKIP + max(64, steps)
    fused = FUSED_SKIP + max(1536, steps)
    return {
        "prewarm_launches": phased + fused + REHEARSALS * (warmup + steps),
        "prewarm_detail": {"phased_forwards": phased, "persistent_forwards": fused,
                           "rehearsal_passes": REHEARSALS, "forwards_per_pass": warmup + steps},
        "pass_ms_per_step": [round(v, 5) for v in pass_ms],
        "cold_ms_per_step": round(pass_ms[0], 5) if pass_ms else None,
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # 256 after 256 (0.2 s in all): with the 32 after 32 of the reference's driver the wall-clock figure
    # is still a few per cent high, the first launches of a process run before the clocks have settled
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=256)
    ap.add_argument("--workload", default="headline_e64_zipf")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--calib-copy-mib", type=int, default=0,
                    help="also run one device-to-device copy of this many MiB before the timed region "
                         "(a kernel of known traffic to scale rocprofv3 FETCH_SIZE / WRITE_SIZE by)")
    ap.add_argument("--power-seconds", type=float, default=4.0,
                    help="after the timed region, keep launching forwards for this long and report the socket "
                         "power over that time (0: skip)")
    ap.add_argument("--zero-expert-weights", action="store_true",
                    help="power probe, not the metric: the expert weights are zeroed, so that the same kernel "
                         "with the same schedule and memory traffic multiplies zeros")
    ap.add_argument("--calib-gemm", default="",
                    help="M,N,K: instead of the layer, loop the vendor's bf16 GEMM of that shape for "
                         "--power-seconds and report its TFLOP/s and socket power (add --zero-expert-weights "
                         "to zero its first operand)")
    ap.add_argument("--calib-mfma", action="store_true",
                    help="instead of the layer, loop the library's matrix-instruction probe for --power-seconds per "
                         "instruction and report TFLOP/s and socket power (--zero-expert-weights: zero operands)")
    ap.add_argument("--print-fingerprint", action="store_true",
                    help="print the fingerprint of the library sources (recorded in the counter summaries) and exit")
    args = ap.parse_args()
    if args.print_fingerprint:
        print(source_fingerprint())
        return 0
    traffic_bytes, traffic_current = measured_traffic(args.workload)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures the single-GPU path (expert-parallel degree 1) only; run it with --gpus 1",
              file=sys.stderr)
        return 2

    import numpy as np
    import torch

    import aristos_amd as ka
    from aristos_amd import _capi, synth

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)
    if args.calib_gemm:
        return vendor_gemm_calibration(args.calib_gemm, args.power_seconds, args.zero_expert_weights)
    if args.calib_mfma:
        return mfma_calibration(args.power_seconds, args.zero_expert_weights)
    w = synth.WORKLOADS[args.workload]
    iP, d = synth.make_inputs(w, seed=args.seed, device="cuda")
    if args.zero_expert_weights:
        iP.view(-1)[d.off_w_up:d.off_w_up + 2 * d.E * d.I * d.H].zero_()
    torch.cuda.synchronize()
    bf16 = d.elem_bytes == 2

    if args.calib_copy_mib > 0:
        n = args.calib_copy_mib * (1 << 20)
        src = torch.ones(n, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    ka.initialize(w.config)
    try:
        oP = synth.alloc_outputs(d)
        lib_stream = torch.cuda.ExternalStream(_capi.lib().kleos_stream())
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        # ---- phased mode first: the same device code, one launch per phase, for per-phase figures
        ka.moe.set_mode(ka.MODE_PHASED)
        ph_total = ka.moe.forward_host_bench(iP, oP, skip=PHASED_SKIP, trials=max(64, args.steps))
        ph = ka.moe.phase_times()
        # ---- fused mode: the product path. Event-timed on the library stream (the reference's protocol,
        # moe.cuh:160-181: skip launches, then trials launches between two events) ...
        ka.moe.set_mode(ka.MODE_FUSED)
        ka.moe.forward_host_bench(iP, oP, skip=FUSED_SKIP, trials=max(1536, args.steps))
        # ... then, with nothing in between (the device drops its clocks within milliseconds of idling),
        # the timed region: `warmup` forwards, then exactly `steps` forwards, timed by the wall clock (the
        # reported value) and, the same launches, by HIP events on the stream the kernel runs on
        # The protocol runs four times back to back and only the last pass counts: whatever ran before
        # (nothing, 256 or 1536 launches), the first passes of this launch pattern measure high (at 20
        # steps the first pass reads some 8 % above the fourth). Every pass is reported in the JSON line
        # (`pass_ms_per_step`; the first as `cold_ms_per_step`), with the count of launches before the
        # timed region (`prewarm_launches`).
        pass_ms = []
        for _ in range(REHEARSALS + 1):
            for _ in range(args.warmup):
                ka.moe.forward_host(iP, oP)
            ka.moe.stream_synchronize()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            ev0.record(lib_stream)
            for _ in range(args.steps):
                ka.moe.forward_host(iP, oP)
            ev1.record(lib_stream)
            ka.moe.stream_synchronize()
            torch.cuda.synchronize()
            wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
            ev_ms = ev0.elapsed_time(ev1) / args.steps
            pass_ms.append(wall_ms)
        # per-phase figures of the persistent kernel: from the stamps of the last launch and an event-timed run
        ka.moe.forward_host_bench(iP, oP, skip=0, trials=8)
        fused_ph = ka.moe.phase_times()
        sched = ka.moe.scheduler_stats()
        # socket power under the same load, kept up for a few seconds, and what a forward takes then
        power = None
        if args.power_seconds > 0:
            per_call = max(8, int(0.05 / max(wall_ms * 1e-3, 1e-6)))
            seen = []
            power = sustained_power(args.power_seconds, lambda: seen.append(
                (time.perf_counter(), ka.moe.forward_host_bench(iP, oP, skip=0, trials=per_call))))
            if power is not None and seen:
                late = [ms for t, ms in seen if t >= seen[0][0] + 1.5] or [ms for _, ms in seen]
                power["sustained_ms_per_step"] = round(sum(late) / len(late), 5)
        schedule = "static" if ka.moe.schedule_taken() == ka.SCHEDULE_STATIC else "dynamic"
        views = ka.moe.debug_views(d)
        kept = int(np.minimum(views["expert_count"].astype(np.int64), d.kept_capacity).sum())
        dropped = int((views["topk_slot"] < 0).sum())
        hottest = float(views["expert_count"].max() / (d.S * d.k / d.E))
    finally:
        ka.finalize()

    flops_layer = synth.layer_flops(d, kept)
    flops_expert = synth.expert_flops(d, kept)
    eb = d.elem_bytes
    peak = PEAK_BF16_TFLOPS if bf16 else PEAK_FP32_TFLOPS
    # minimum HBM traffic of one forward: expert weights once + x (gate) + gathered rows + output + Wg
    n_active = int((views["expert_count"] > 0).sum())
    hbm_bytes = float(2 * n_active * d.H * d.I * eb + d.S * d.H * eb + kept * d.H * eb + d.S * d.H * eb + d.E * d.H * eb)
    up_dn_ms = ph["up"] + ph["down"]
    ex_ms = fused_ph["up"]
    fused_phases = {
        "gate_ms": round(fused_ph["gate"], 4), "slots_ms": round(fused_ph["slots"], 4),
        "experts_ms": round(ex_ms, 4), "combine_ms": round(fused_ph["combine"], 4),
        "expert_gemm_tflops": round(flops_expert / (ex_ms * 1e-3) / 1e12, 2) if ex_ms > 0 else None,
        "expert_gemm_mfma_frac": round(flops_expert / (ex_ms * 1e-3) / 1e12 / peak, 4) if ex_ms > 0 else None,
        "scheduler": {k: round(v, 5) for k, v in sched.items()},
    }
    phases = {
        "total_ms": round(ph_total, 4),
        "gate_ms": round(ph["gate"], 4), "slots_ms": round(ph["slots"], 4), "up_ms": round(ph["up"], 4),
        "down_ms": round(ph["down"], 4), "combine_ms": round(ph["combine"], 4),
        "expert_gemm_tflops": round(flops_expert / (up_dn_ms * 1e-3) / 1e12, 2) if up_dn_ms > 0 else None,
        "expert_gemm_mfma_frac": round(flops_expert / (up_dn_ms * 1e-3) / 1e12 / peak, 4) if up_dn_ms > 0 else None,
        # gate streams x once; combine reads T rows and writes S rows
        "gate_hbm_gbs": round((d.S * d.H * eb + d.E * d.H * eb) / (ph["gate"] * 1e-3) / 1e9, 1) if ph["gate"] > 0 else None,
        "combine_hbm_gbs": round((kept * d.H * eb + d.S * d.H * eb) / (ph["combine"] * 1e-3) / 1e9, 1) if ph["combine"] > 0 else None,
    }

    # the expert phase alone (both projections of every expert, inside the persistent launch):
    # weights once + the gathered activation rows, against both roofs
    ex_bytes = float(2 * n_active * d.H * d.I * eb + kept * d.H * eb)
    experts = None
    if ex_ms > 0:
        ex_gbs = ex_bytes / (ex_ms * 1e-3) / 1e9
        ex_tf = flops_expert / (ex_ms * 1e-3) / 1e12
        experts = {"ms": round(ex_ms, 4), "algorithmic_bytes": ex_bytes, "flops": flops_expert,
                   "hbm": {"achieved": round(ex_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(ex_gbs / PEAK_HBM_GBS, 4)},
                   "mfma": {"achieved": round(ex_tf, 2), "peak": peak, "unit": "TFLOP/s", "frac": round(ex_tf / peak, 4)}}

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(w, iP, d, kept)

    line = {
        "metric": "moe_layer_fwd_latency_us",
        "value": round(wall_ms * 1e3, 2),
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        **prewarm_protocol(args.steps, args.warmup, pass_ms),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16" if bf16 else "f32",
        "data": "synthetic" if not args.zero_expert_weights else "synthetic, expert weights zeroed (power probe: not the metric)",
        "config": {"workload": f"{w.name}: {w.note}", "S": d.S, "H": d.H, "I": d.I, "E": d.E, "top_k": d.k,
                   "capacity_factor": w.config.capacity_factor, "EC": d.EC, "kept_pairs": kept,
                   "dropped_pairs": dropped, "hottest_expert_vs_mean": round(hottest, 2),
                   "mode": "fused persistent kernel, 1 launch per forward",
                   "expert_schedule": schedule + " (KLEOS_SCHEDULE_AUTO)"},
        "tokens_per_s": round(d.S / (wall_ms * 1e-3), 1),
        "event_ms_per_step": round(ev_ms, 5),
        "roofline": roofline(flops_layer, hbm_bytes, ev_ms, peak, traffic_bytes, traffic_current, experts),
        "power": power,
        "fused_phases": fused_phases,
        "phased_mode": phases,
        "cpu_baseline": cpu,
    }
    print(json.dumps(line))
    return 0


def roofline(flops, hbm_bytes, ev_ms, mfma_peak, traffic, traffic_current, experts):
    """The roof that binds the launch: below the ridge (peak FLOP/s / peak B/s) the algorithmic
    bytes cannot move faster than HBM, above it the FLOPs cannot run faster than the matrix cores.
    Both fractions are reported; `bound`, `achieved`, `peak`, `frac` describe the binding one."""
    sec = ev_ms * 1e-3
    gbs = hbm_bytes / sec / 1e9
    tflops = flops / sec / 1e12
    intensity = flops / hbm_bytes
    ridge = mfma_peak * 1e12 / (PEAK_HBM_GBS * 1e9)
    common = {"traffic": traffic, "traffic_measured_on_these_sources": traffic_current, "experts": experts, "kernel": "fused_kernel (whole layer: gate + slots + expert GEMMs + combine)",
              "flops_per_launch": flops, "algorithmic_bytes_per_launch": hbm_bytes,
              "intensity_flop_per_byte": round(intensity, 1), "ridge_flop_per_byte": round(ridge, 1),
              "hbm": {"achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(gbs / PEAK_HBM_GBS, 4)},
              "mfma": {"achieved": round(tflops, 2), "peak": mfma_peak, "unit": "TFLOP/s", "frac": round(tflops / mfma_peak, 4)}}
    if intensity < ridge:
        return {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "frac": round(gbs / PEAK_HBM_GBS, 4), **common}
    return {"bound": "mfma", "achieved": round(tflops, 2), "peak": mfma_peak, "unit": "TFLOP/s",
            "frac": round(tflops / mfma_peak, 4), **common}


def cpu_baseline(w, iP, d, kept):
    """The CPU oracle (a port of the reference semantics, OpenMP) on this box's host cores. The
    sample is a prefix of the tokens sized to a few seconds of CPU work; its time is scaled to the
    whole layer by kept (token, expert) pairs, the gate being evaluated in full."""
    import numpy as np
    import torch
    from oracle import moe_ref

    c = moe_ref.cfg_from_keys(w.config)
    if d.elem_bytes == 2:
        iP_np = iP.view(torch.int16).cpu().numpy().view(np.uint16)
    else:
        iP_np = iP.cpu().numpy()
    # routing pass (cheap) to pick the sample: a prefix of the tokens worth ~150 GFLOP of expert work
    t0 = time.perf_counter()
    route = moe_ref.forward(c, iP_np, token_mask=np.zeros(c.S, np.uint8))
    gate_s = time.perf_counter() - t0
    # a sample of about 10 s of CPU work at the ~0.5 TFLOP/s the oracle reaches on 16 cores
    target_pairs = max(64, min(kept, int(5e12 / (4.0 * d.H * d.I))))
    frac = min(1.0, target_pairs / max(kept, 1))
    mask = np.zeros(c.S, np.uint8)
    n_tok = max(1, int(round(c.S * frac)))
    mask[:n_tok] = 1
    sampled_pairs = int(((route["topk_slot"] >= 0) & (mask[:, None] == 1)).sum())
    # median of several passes when one pass is short
    times = []
    budget = time.perf_counter() + 12.0
    while len(times) < 3 or (time.perf_counter() < budget and len(times) < 25):
        t0 = time.perf_counter()
        moe_ref.forward(c, iP_np, logits=route["logits"], token_mask=mask)
        times.append(time.perf_counter() - t0)
    ffn_s = sorted(times)[len(times) // 2]
    scale = kept / max(sampled_pairs, 1)
    total_s = gate_s + ffn_s * scale
    return {"value": round(total_s * 1e6, 1), "unit": "us", "cores": moe_ref.threads(), "kind": "port",
            "sample": f"gate+routing on all {c.S} tokens ({gate_s:.2f} s) + expert FFN and combine on "
                      f"the first {int(mask.sum())} tokens = {sampled_pairs} of {kept} kept (token, expert) pairs "
                      f"(median of {len(times)} passes, {ffn_s:.2f} s each), scaled by {scale:.2f}",
            "gflops": round((2.0 * d.S * d.H * d.E + 4.0 * kept * d.H * d.I) / total_s / 1e9, 1)}


if __name__ == "__main__":
    sys.exit(main())
