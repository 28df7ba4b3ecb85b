"""Host API of the MoE forward, named after the reference's kleos::moe functions
(csrc/include/kleos/moe/moe.cuh:146-205). Buffers are device pointers (ints) or objects with a
``data_ptr()`` method (torch tensors); nothing here touches their contents on the host."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _capi


def _ptr(buf) -> int:
    if isinstance(buf, int):
        return buf
    if hasattr(buf, "data_ptr"):
        return int(buf.data_ptr())
    raise TypeError(f"expected a device pointer or tensor, got {type(buf)!r}")


def forward_host(iP, oP) -> None:
    """kleos::moe::forwardHost(iP, oP) (moe.cuh:186-205): enqueue one forward on the library stream."""
    _capi.check(_capi.lib().kleos_moe_forward(_ptr(iP), _ptr(oP)))


def forward_host_dense(iP, oP) -> None:
    """kleos_moe_forward_dense: num_experts == 1 on the packing of the reference's fffn kernel
    (fffn.cuh:43-49): iP = x | Wup | Wdown | bup | bdown, oP = moeOut."""
    _capi.check(_capi.lib().kleos_moe_forward_dense(_ptr(iP), _ptr(oP)))


def forward_host_bench(iP, oP, skip: int = 32, trials: int = 32) -> float:
    """kleos::moe::forwardHostBench<skip, trials>(iP, oP, ms) (moe.cuh:146-184): mean milliseconds per
    launch over `trials` launches after `skip` warm-ups. The defaults are the reference driver's
    (csrc/main.cu:68)."""
    ms = C.c_float(0.0)
    _capi.check(_capi.lib().kleos_moe_forward_bench(_ptr(iP), _ptr(oP), skip, trials, C.byref(ms)))
    return float(ms.value)


def forward_static_scratch(config, iP, oP, stream: int = 0) -> None:
    """kleos_moe_forward_static_scratch: one forward of the layer `config` (a KleosConfig) that allocates
    nothing, on `stream` (a hipStream_t as an integer; 0 = the default stream). Asynchronous."""
    st = config.to_struct()
    _capi.check(_capi.lib().kleos_moe_forward_static_scratch(C.byref(st), _ptr(iP), _ptr(oP), stream or None))


def static_scratch_prepare(config) -> None:
    """kleos_static_scratch_prepare: the per-device set-up and the launch plan of `config`, so that a
    first forward_static_scratch of that layer may be recorded under stream capture."""
    st = config.to_struct()
    _capi.check(_capi.lib().kleos_static_scratch_prepare(C.byref(st)))


def static_scratch_status(stream: int = 0) -> None:
    """kleos_static_scratch_status: drains `stream`, raises KleosError (KLEOS_EHIP) if a wait inside a
    static-scratch forward expired since the last status call."""
    _capi.check(_capi.lib().kleos_static_scratch_status(stream or None))


def debug_static_scratch_expiry(ticks: int, skip_launch_numbers: int) -> None:
    """Test hook: tick limit and launch-number offset of later static-scratch forwards ((0, 0): normal)."""
    _capi.check(_capi.lib().kleos_debug_static_scratch_expiry(int(ticks), int(skip_launch_numbers)))


def stream_synchronize() -> None:
    _capi.check(_capi.lib().kleos_stream_synchronize())


def set_mode(mode: int) -> None:
    """MODE_FUSED (one persistent launch, default) or MODE_PHASED (one launch per phase)."""
    _capi.check(_capi.lib().kleos_set_mode(int(mode)))


def debug_mfma_probe(tile: int, iterations: int = 20000, zero_operands: bool = False) -> dict:
    """One launch of the matrix-instruction probe (tile 32: 32x32x16 bf16 instructions, tile 16:
    16x16x32) on every CU: its duration and the rate it ran at. Needs no initialised context."""
    ms = C.c_float(0.0)
    flop = C.c_double(0.0)
    _capi.check(_capi.lib().kleos_debug_mfma_probe(int(tile), int(iterations), int(bool(zero_operands)), C.byref(ms), C.byref(flop)))
    return {"ms": float(ms.value), "tflops": float(flop.value) / (float(ms.value) * 1e-3) / 1e12}


def set_schedule(schedule: int) -> None:
    """SCHEDULE_AUTO (default), SCHEDULE_DYNAMIC or SCHEDULE_STATIC: how the persistent launch hands
    out expert tiles."""
    _capi.check(_capi.lib().kleos_set_schedule(int(schedule)))


def set_cooperative_launch(on: bool) -> None:
    """Launch the persistent kernel through hipLaunchCooperativeKernel (the runtime then verifies per launch
    that the whole grid is resident together; about 14 us more per launch)."""
    _capi.check(_capi.lib().kleos_set_cooperative_launch(1 if on else 0))


def schedule_taken() -> int:
    """SCHEDULE_DYNAMIC or SCHEDULE_STATIC: what the most recent persistent launch did."""
    out = C.c_int(-1)
    _capi.check(_capi.lib().kleos_schedule_taken(C.byref(out)))
    return int(out.value)


def phase_times() -> dict:
    """Per-phase milliseconds of the last phased forward_host_bench."""
    arr = (C.c_float * 5)()
    _capi.check(_capi.lib().kleos_phase_times(arr))
    return dict(zip(("gate", "slots", "up", "down", "combine"), (float(v) for v in arr)))


def scheduler_stats() -> dict:
    """Tile-scheduler statistics of the last fused forward_host_bench launch."""
    arr = (C.c_double * 6)()
    _capi.check(_capi.lib().kleos_scheduler_stats(arr))
    keys = ("fetch_ms", "wait_ms", "publish_ms", "tiles", "late_tiles", "foreign_tiles")
    return dict(zip(keys, (float(v) for v in arr)))


def measure_throughput(trials: int = 16) -> dict:
    """One expert at full padded capacity through both projections (the reference's mT probe,
    throughput.cuh:104-170): median latency in ms and its reciprocal."""
    ms = C.c_float(0.0)
    thr = C.c_float(0.0)
    _capi.check(_capi.lib().kleos_measure_throughput(int(trials), C.byref(ms), C.byref(thr)))
    return {"median_ms": float(ms.value), "throughput": float(thr.value)}


def measure_throughput_output(derived, trials: int = 4) -> dict:
    """The same probe, with its result y[pEC, H] copied back as raw Element words (uint16 for the
    16-bit Elements, float32 otherwise)."""
    ms = C.c_float(0.0)
    thr = C.c_float(0.0)
    y = np.empty((derived.pEC, derived.H), dtype=np.float32 if derived.elem_bytes == 4 else np.uint16)
    _capi.check(_capi.lib().kleos_measure_throughput_output(int(trials), C.byref(ms), C.byref(thr), y.ctypes.data,
                                                            y.nbytes))
    return {"median_ms": float(ms.value), "throughput": float(thr.value), "y": y}


def debug_set_wait_ticks(ticks: int) -> None:
    """Bound of every wait inside the persistent kernel, in ticks of the 100 MHz device clock (0: default, 3 s)."""
    _capi.check(_capi.lib().kleos_debug_set_wait_ticks(int(ticks)))


def debug_skip_launch_number() -> None:
    """Counts a persistent launch that never ran, so that the next one runs into its wait limit."""
    _capi.check(_capi.lib().kleos_debug_skip_launch_number())


def gate_loss(n_experts: int) -> dict:
    """Training mode: loss, mean probability [E] and mean routed count [E] of the last forward."""
    loss = C.c_float(0.0)
    mp = (C.c_float * n_experts)()
    mc = (C.c_float * n_experts)()
    _capi.check(_capi.lib().kleos_gate_loss(C.byref(loss), mp, mc))
    return {"loss": float(loss.value), "mean_prob": np.array(mp[:], np.float32),
            "mean_count": np.array(mc[:], np.float32)}


def phase_stamps(max_workgroups: int = 4096) -> np.ndarray:
    """Raw 100 MHz wall-clock stamps [workgroups, 8] of the last persistent launch. Synchronises."""
    buf = (C.c_ulonglong * (max_workgroups * 8))()
    n = C.c_uint32(0)
    _capi.check(_capi.lib().kleos_phase_stamps(buf, max_workgroups, C.byref(n)))
    rows = min(int(n.value), max_workgroups)
    return np.ctypeslib.as_array(buf)[: rows * 8].reshape(rows, 8).copy()


def debug_views(derived) -> dict:
    """Copies the routing state of the most recent forward to host numpy arrays. Synchronises."""
    lib = _capi.lib()
    v = _capi.DebugViewsStruct()
    _capi.check(lib.kleos_moe_debug_views(C.byref(v)))
    S, E, k, R = derived.S, derived.E, derived.k, derived.cap_rows
    spec = {
        "logits": (v.logits, (S, E), np.float32),
        "topk_expert": (v.topk_expert, (S, k), np.int32),
        "topk_prob": (v.topk_prob, (S, k), np.float32),
        "combine_den": (v.combine_den, (S,), np.float32),
        "topk_slot": (v.topk_slot, (S, k), np.int32),
        "expert_count": (v.expert_count, (E,), np.uint32),
        "slot_token": (v.slot_token, (E, R), np.int32),
    }
    out = {}
    for name, (ptr, shape, dt) in spec.items():
        host = np.empty(shape, dtype=dt)
        _capi.check(lib.kleos_debug_copy_to_host(host.ctypes.data, ptr, host.nbytes))
        out[name] = host
    return out
