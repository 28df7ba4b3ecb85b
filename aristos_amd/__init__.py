"""aristos_amd — MI355X-native fused MoE-layer forward behind the Kleos host API.

The product is the HIP library ``libkleos_amd.so`` (C ABI in ``include/kleos_amd.h``). This package
is the Python mirror of the reference's host interface for that path:

    kleos::initialize()              -> aristos_amd.initialize(config)
    kleos::finalize()                -> aristos_amd.finalize()
    kleos::getRank()                 -> aristos_amd.get_rank()
    kleos::setDevice()               -> aristos_amd.set_device()
    kleos::moe::forwardHost          -> aristos_amd.moe.forward_host(iP, oP)
    kleos::moe::forwardHostBench     -> aristos_amd.moe.forward_host_bench(iP, oP, skip, trials)

There is no CPU or PyTorch implementation behind these calls: if the library is not built they raise.
"""
from __future__ import annotations

import ctypes as _C
import os as _os

from . import _capi, moe
from ._capi import KleosError, MODE_FUSED, MODE_PHASED, SCHEDULE_AUTO, SCHEDULE_DYNAMIC, SCHEDULE_STATIC, DTYPE_FP32, DTYPE_BF16, ACT_RELU, ACT_GELU
from .config import KleosConfig, DerivedConfig

__all__ = ["initialize", "finalize", "is_initialized", "get_rank", "set_device", "active_config", "moe",
           "KleosConfig", "DerivedConfig", "KleosError", "MODE_FUSED", "MODE_PHASED",
           "SCHEDULE_AUTO", "SCHEDULE_DYNAMIC", "SCHEDULE_STATIC"]


def initialize(config) -> DerivedConfig:
    """kleos::initialize() (csrc/include/kleos/bootstrap.cuh:533-547). `config` is a path to a
    kleos_config.json, a KleosConfig, or a dict of its keys. Returns the derived constants."""
    lib = _capi.lib()
    if isinstance(config, (str, _os.PathLike)):
        _capi.check(lib.kleos_initialize(str(config).encode()))
    else:
        if isinstance(config, dict):
            config = KleosConfig(**config)
        st = config.to_struct()
        _capi.check(lib.kleos_initialize_cfg(_C.byref(st)))
    return active_config()


def finalize() -> None:
    """kleos::finalize() (bootstrap.cuh:562-588)."""
    _capi.check(_capi.lib().kleos_finalize())


def is_initialized() -> bool:
    return bool(_capi.lib().kleos_is_initialized())


def get_rank() -> int:
    """kleos::getRank() (bootstrap.cuh:556-559); 0 on the single-GPU path."""
    r = _capi.lib().kleos_get_rank()
    if r < 0:
        _capi.check(_capi.KLEOS_ESTATE)
    return r


def set_device() -> None:
    """kleos::setDevice() (bootstrap.cuh:550-553)."""
    _capi.check(_capi.lib().kleos_set_device())


def active_config() -> DerivedConfig:
    st = _capi.KleosConfigStruct()
    _capi.check(_capi.lib().kleos_get_config(_C.byref(st)))
    from .config import DERIVED
    return DerivedConfig(KleosConfig.from_struct(st), **{n: getattr(st, n) for n in DERIVED})
