"""The C-ABI library loads and exports every function include/kleos_amd.h declares, and the host
API fails loudly (never falls back) when it cannot run."""
import ctypes
import os
import re

import pytest

import aristos_amd as ka
from aristos_amd import _capi

HEADER = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include", "kleos_amd.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kleos_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    names = declared_functions()
    assert len(names) >= 20
    lib = ctypes.CDLL(_capi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in kleos_amd.h but not exported"
    assert sorted(_capi.SYMBOLS) == names, "the ctypes table and the header disagree"


def test_struct_layout_matches_the_header():
    # 1 double + 14 + 10 uint32 + 10 uint64, naturally aligned
    assert ctypes.sizeof(_capi.KleosConfigStruct) == 8 + 4 * 24 + 8 * 10
    assert ctypes.sizeof(_capi.DebugViewsStruct) == 7 * ctypes.sizeof(ctypes.c_void_p)


def test_calls_before_initialize_fail_like_the_reference():
    """KLEOS_ASSERT(isInitialized, "Not initialized!") (moe.cuh:152,191; bootstrap.cuh:551,557,566)."""
    assert not ka.is_initialized()
    for fn in (ka.finalize, ka.set_device, ka.get_rank, ka.moe.stream_synchronize, lambda: ka.moe.forward_host(16, 16)):
        with pytest.raises(ka.KleosError) as ei:
            fn()
        assert ei.value.code == _capi.KLEOS_ESTATE and "Not initialized" in ei.value.message


def test_initialize_without_a_gpu_raises():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(ka.KleosError) as ei:
        ka.initialize(ka.KleosConfig(sequence_len=128, hidden_size=64, intermediate_size=64, num_experts=4))
    assert ei.value.code == _capi.KLEOS_EHIP
    assert not ka.is_initialized()


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU's share only: asked for more, it says so and exits (no GPU needed)."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode == 2
    assert "single-GPU" in proc.stderr and proc.stdout.strip() == ""


def test_a_refused_cooperative_launch_maps_to_kleos_ehip():
    """With kleos_set_cooperative_launch(1) a grid that cannot be resident is refused by the runtime at
    launch (hipErrorCooperativeLaunchTooLarge, 720) and kleos_moe_forward itself returns KLEOS_EHIP with
    the runtime's name of the error; hipSuccess maps to KLEOS_OK. The mapping touches no device."""
    lib = _capi.lib()
    assert lib.kleos_debug_map_hip_error(0) == _capi.KLEOS_OK
    assert lib.kleos_debug_map_hip_error(720) == _capi.KLEOS_EHIP
    assert "hipErrorCooperativeLaunchTooLarge" in lib.kleos_last_error().decode()
    assert lib.kleos_debug_map_hip_error(2) == _capi.KLEOS_EHIP
    assert "hipErrorOutOfMemory" in lib.kleos_last_error().decode()
