"""kleos_moe_forward_static_scratch: the forward that allocates nothing (its library-owned arrays live
in a fixed array in device memory) gives the bits of kleos_moe_forward, on calls in a row that share
the array: a layer, then a smaller one of a different shape, then the first again."""
import ctypes

import numpy as np
import pytest
import torch

import aristos_amd as ka
from aristos_amd import _capi, synth
from helpers import pack_inputs, random_layer
from oracle import moe_ref

pytestmark = pytest.mark.gpu


def _keys(S, H, I, E, k, dt=2, cf=1.0):
    return ka.KleosConfig(capacity_factor=cf, drop_tokens=1, expert_top_k=k, hidden_act=0, hidden_size=H,
                          intermediate_size=I, num_experts=E, sequence_len=S, mini_batch=1, torch_dtype=dt)


def _device_inputs(keys, seed):
    c = moe_ref.cfg_from_keys(keys)
    x, wg, w_up, w_down, b_up, b_down = random_layer(c, seed=seed, w_std=0.08, bias_std=0.1)
    wg[0] *= 2.5                                   # an expert that overflows: dropped tokens
    if c.dtype == 2:
        from np_restatement import round_bf16
        wg = round_bf16(wg)
    iP_np = pack_inputs(c, x, wg, w_up, w_down, b_up, b_down)
    if c.dtype in (2, 3):
        iP = torch.from_numpy(iP_np.view(np.int16)).cuda().view(torch.bfloat16 if c.dtype == 2 else torch.float16)
    else:
        iP = torch.from_numpy(iP_np).cuda()
    return c, iP


def _bits(c, oP):
    return oP.view(torch.int16).cpu().numpy().copy() if c.dtype in (2, 3) else oP.cpu().numpy().copy()


def _existing_entry_point(keys, iP):
    d = ka.initialize(keys)
    try:
        oP = synth.alloc_outputs(d)
        oP.fill_(float("nan"))
        torch.cuda.synchronize()
        ka.moe.forward_host(iP, oP)
        ka.moe.stream_synchronize()
        return d, oP
    finally:
        ka.finalize()


def test_static_scratch_forward_matches_the_allocating_one():
    big = _keys(1024, 256, 512, 16, 2)
    small = _keys(256, 128, 128, 8, 2, cf=2.0)
    small_f32 = _keys(128, 64, 64, 4, 1, dt=0)
    cases = []
    for keys, seed in ((big, 71), (small, 72), (small_f32, 73)):
        c, iP = _device_inputs(keys, seed)
        d, ref = _existing_entry_point(keys, iP)
        cases.append((keys, c, d, iP, _bits(c, ref)))
    assert not ka.is_initialized()
    # calls in a row on the default stream, no context: big, small, smaller still (fp32), big again
    for keys, c, d, iP, ref in (cases[0], cases[1], cases[2], cases[0], cases[1]):
        oP = synth.alloc_outputs(d)
        oP.fill_(float("nan"))
        torch.cuda.synchronize()
        ka.moe.forward_static_scratch(keys, iP, oP)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(_bits(c, oP), ref)
    # two calls queued back to back without a synchronisation in between share the array in order
    (k0, c0, d0, i0, r0), (k1, c1, d1, i1, r1) = cases[0], cases[1]
    o0, o1 = synth.alloc_outputs(d0), synth.alloc_outputs(d1)
    torch.cuda.synchronize()
    ka.moe.forward_static_scratch(k0, i0, o0)
    ka.moe.forward_static_scratch(k1, i1, o1)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(_bits(c0, o0), r0)
    np.testing.assert_array_equal(_bits(c1, o1), r1)
    # an initialised context is left alone, and works beside it
    d = ka.initialize(k1)
    try:
        oa, ob = synth.alloc_outputs(d1), synth.alloc_outputs(d0)
        ka.moe.forward_host(i1, oa)
        ka.moe.stream_synchronize()
        ka.moe.forward_static_scratch(k0, i0, ob)
        torch.cuda.synchronize()
        ka.moe.forward_host(i1, oa)
        ka.moe.stream_synchronize()
        np.testing.assert_array_equal(_bits(c1, oa), r1)
        np.testing.assert_array_equal(_bits(c0, ob), r0)
    finally:
        ka.finalize()


def test_static_scratch_refuses_what_does_not_fit():
    """The headline layer needs about 137 MB of library arrays: beyond what the 32 MiB scratch holds
    (all of it but the 256 bytes at its end that keep the record of expired waits)."""
    keys = synth.WORKLOADS["headline_e64_zipf"].config
    dummy = torch.zeros(64, dtype=torch.bfloat16, device="cuda")
    st = keys.to_struct()
    rc = _capi.lib().kleos_moe_forward_static_scratch(ctypes.byref(st), dummy.data_ptr(), dummy.data_ptr(), None)
    assert rc == _capi.KLEOS_EUNSUPPORTED
    msg = _capi.lib().kleos_last_error().decode()
    assert f"static scratch holds {(32 << 20) - 256}" in msg, msg
    torch.cuda.synchronize()


def test_static_scratch_forward_replays_from_a_graph():
    """The entry point exists for callers under stream capture: recorded once into a HIP graph, every
    replay gives the bits of kleos_moe_forward, with eager calls on the same array between the replays
    (the counters are cleared by a fill kernel, which a graph replays faithfully)."""
    keys = _keys(1024, 256, 512, 16, 2)
    c, iP = _device_inputs(keys, 71)
    d, ref = _existing_entry_point(keys, iP)
    ref = _bits(c, ref)
    oP = synth.alloc_outputs(d)
    side = torch.cuda.Stream()
    ka.moe.forward_static_scratch(keys, iP, oP, stream=side.cuda_stream)   # the per-device set-up happens eagerly
    side.synchronize()
    np.testing.assert_array_equal(_bits(c, oP), ref)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ka.moe.forward_static_scratch(keys, iP, oP, stream=torch.cuda.current_stream().cuda_stream)
    other = _keys(256, 128, 128, 8, 2, cf=2.0)
    c2, iP2 = _device_inputs(other, 72)
    oP2 = synth.alloc_outputs(other.derive())
    for _ in range(4):
        oP.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(_bits(c, oP), ref)
        # eager work on the same array, of another shape, between the replays
        ka.moe.forward_static_scratch(other, iP2, oP2)
        torch.cuda.synchronize()


def test_static_scratch_status_reports_an_expired_wait():
    """An expired in-kernel wait of a static-scratch forward is on record until the status call has
    reported it. The expiry is provoked from the host (a 0.2 ms limit on every wait, and counters that
    lag the launch number by one launch, so that no barrier is ever complete); every kernel exits
    normally, and the next forward gives the right bits again."""
    keys = _keys(1024, 256, 512, 16, 2)
    c, iP = _device_inputs(keys, 71)
    d, ref = _existing_entry_point(keys, iP)
    ref = _bits(c, ref)
    oP = synth.alloc_outputs(d)
    ka.moe.forward_static_scratch(keys, iP, oP)
    ka.moe.static_scratch_status()            # nothing expired
    try:
        ka.moe.debug_static_scratch_expiry(20000, 1)
        ka.moe.forward_static_scratch(keys, iP, oP)
        with pytest.raises(ka.KleosError) as ei:
            ka.moe.static_scratch_status()
        assert ei.value.code == _capi.KLEOS_EHIP and "the most recent call" in ei.value.message, ei.value.message
        ka.moe.static_scratch_status()        # the record was cleared
        # a failed call followed by a good one: the fill kernel of the good call keeps the record
        ka.moe.forward_static_scratch(keys, iP, oP)
        ka.moe.debug_static_scratch_expiry(0, 0)
        oP.fill_(float("nan"))
        ka.moe.forward_static_scratch(keys, iP, oP)
        with pytest.raises(ka.KleosError) as ei:
            ka.moe.static_scratch_status()
        assert ei.value.code == _capi.KLEOS_EHIP and "an earlier call" in ei.value.message, ei.value.message
        np.testing.assert_array_equal(_bits(c, oP), ref)   # the good call itself was fine
    finally:
        ka.moe.debug_static_scratch_expiry(0, 0)
    ka.moe.static_scratch_status()
    oP.fill_(float("nan"))
    ka.moe.forward_static_scratch(keys, iP, oP)
    ka.moe.static_scratch_status()
    np.testing.assert_array_equal(_bits(c, oP), ref)


def test_static_scratch_first_call_of_a_layer_under_capture():
    """After kleos_static_scratch_prepare the first forward of a layer may be recorded under stream
    capture: the launch plan is looked up, nothing queries the runtime."""
    keys = _keys(512, 192, 320, 12, 3)       # a layer no other test of this file runs
    c, iP = _device_inputs(keys, 74)
    d, ref = _existing_entry_point(keys, iP)
    ref = _bits(c, ref)
    oP = synth.alloc_outputs(d)
    ka.moe.static_scratch_prepare(keys)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ka.moe.forward_static_scratch(keys, iP, oP, stream=torch.cuda.current_stream().cuda_stream)
    for _ in range(3):
        oP.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(_bits(c, oP), ref)
    ka.moe.static_scratch_status()
