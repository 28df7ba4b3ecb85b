"""kleos_config.json handling: the same keys and enumerations as the reference's schema
(csrc/kleos_config.schema.json:5-72), parsed and validated by the C library at run time."""
from __future__ import annotations

import ctypes as C
import json
from dataclasses import dataclass, fields, asdict

from . import _capi

# keys of kleos_config.json, in schema order
JSON_KEYS = ("capacity_factor", "drop_tokens", "expert_top_k", "global_batch", "is_training", "hidden_act",
             "hidden_size", "intermediate_size", "mini_batch", "moe_frequency", "num_experts", "num_layers",
             "sequence_len", "torch_dtype", "vocab_size")
DERIVED = ("S", "H", "I", "E", "k", "PX", "EC", "pEC", "cap_rows", "elem_bytes", "off_x", "off_gate_w", "off_w_up",
           "off_w_down", "off_b_up", "off_b_down", "in_elems", "off_gate_out", "off_moe_out", "out_elems")


@dataclass
class KleosConfig:
    """The JSON keys of the reference configuration. Defaults are the shipped kleos_config.json
    (csrc/kleos_config.json:1-17) with torch_dtype = 2 (bf16)."""
    capacity_factor: float = 1.0
    drop_tokens: int = 1
    expert_top_k: int = 2
    global_batch: int = 256
    is_training: int = 0
    hidden_act: int = 0
    hidden_size: int = 2048
    intermediate_size: int = 2048
    mini_batch: int = 1
    moe_frequency: int = 1
    num_experts: int = 64
    num_layers: int = 1
    sequence_len: int = 8192
    torch_dtype: int = 2
    vocab_size: int = 32000

    # ---- construction
    @classmethod
    def from_struct(cls, st: _capi.KleosConfigStruct) -> "KleosConfig":
        return cls(**{f.name: getattr(st, f.name) for f in fields(cls)})

    @classmethod
    def from_json_text(cls, text: str) -> "KleosConfig":
        st = _capi.KleosConfigStruct()
        _capi.check(_capi.lib().kleos_config_parse_string(text.encode(), C.byref(st)))
        return cls.from_struct(st)

    @classmethod
    def from_json_file(cls, path: str) -> "KleosConfig":
        st = _capi.KleosConfigStruct()
        _capi.check(_capi.lib().kleos_config_parse_file(str(path).encode(), C.byref(st)))
        return cls.from_struct(st)

    def to_json_text(self) -> str:
        d = asdict(self)
        if float(d["capacity_factor"]).is_integer():
            d["capacity_factor"] = int(d["capacity_factor"])
        return json.dumps(d, indent=2)

    def to_struct(self) -> _capi.KleosConfigStruct:
        st = _capi.KleosConfigStruct()
        for f in fields(self):
            setattr(st, f.name, getattr(self, f.name))
        return st

    # ---- derived constants (struct ACC of the reference, types.cuh:471-507)
    def derive(self) -> "DerivedConfig":
        st = self.to_struct()
        _capi.check(_capi.lib().kleos_config_derive(C.byref(st)))
        return DerivedConfig(self, **{n: getattr(st, n) for n in DERIVED})


@dataclass
class DerivedConfig:
    keys: KleosConfig
    S: int
    H: int
    I: int
    E: int
    k: int
    PX: int
    EC: int
    pEC: int
    cap_rows: int
    elem_bytes: int
    off_x: int
    off_gate_w: int
    off_w_up: int
    off_w_down: int
    off_b_up: int
    off_b_down: int
    in_elems: int
    off_gate_out: int
    off_moe_out: int
    out_elems: int

    @property
    def kept_capacity(self) -> int:
        """Rows an expert can hold: min(EC, cap_rows)."""
        return min(self.EC, self.cap_rows)
