"""TEST INFRASTRUCTURE: ctypes wrapper of the C oracle in moe_ref.c (built by oracle/Makefile).

Never imported by the product package. Inputs and outputs are numpy arrays holding the packed
Element buffers the GPU library takes: uint16 (bf16 bit patterns) or float32.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmoe_ref.so")


class RefCfg(C.Structure):
    _fields_ = [("S", C.c_uint32), ("H", C.c_uint32), ("I", C.c_uint32), ("E", C.c_uint32), ("k", C.c_uint32),
                ("capacity_factor", C.c_double), ("drop_tokens", C.c_uint32), ("hidden_act", C.c_uint32),
                ("dtype", C.c_uint32),
                ("PX", C.c_uint32), ("EC", C.c_uint32), ("pEC", C.c_uint32), ("cap_rows", C.c_uint32)]


class RefViews(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in
                ("logits", "probs", "topk_expert", "topk_prob", "combine_den", "topk_slot", "expert_count",
                 "slot_token")]


def build(force: bool = False) -> str:
    """Compiles the oracle with gcc (make -C oracle)."""
    if force and os.path.exists(LIB_PATH):
        os.remove(LIB_PATH)
    subprocess.run(["make", "-C", HERE, "libmoe_ref.so"], check=True, capture_output=True)
    return LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        h = C.CDLL(LIB_PATH)
        h.moe_ref_derive.restype = C.c_int
        h.moe_ref_derive.argtypes = [C.POINTER(RefCfg)]
        h.moe_ref_forward.restype = C.c_int
        h.moe_ref_forward.argtypes = [C.POINTER(RefCfg), C.c_void_p, C.c_void_p, C.POINTER(RefViews), C.c_int,
                                      C.c_void_p]
        h.moe_ref_threads.restype = C.c_int
        h.moe_ref_round_bf16.restype = C.c_float
        h.moe_ref_round_bf16.argtypes = [C.c_float]
        h.moe_ref_round_f16.restype = C.c_float
        h.moe_ref_round_f16.argtypes = [C.c_float]
        h.moe_ref_round_tf32.restype = C.c_float
        h.moe_ref_round_tf32.argtypes = [C.c_float]
        h.moe_ref_tf32_operand.restype = C.c_float
        h.moe_ref_tf32_operand.argtypes = [C.c_float]
        h.moe_ref_f32_to_f16_bits.restype = C.c_uint16
        h.moe_ref_f32_to_f16_bits.argtypes = [C.c_float]
        h.moe_ref_f16_bits_to_f32.restype = C.c_float
        h.moe_ref_f16_bits_to_f32.argtypes = [C.c_uint16]
        h.moe_ref_gate_logits.restype = None
        h.moe_ref_gate_logits.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p]
        h.moe_ref_softmax.restype = None
        h.moe_ref_softmax.argtypes = [C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p]
        h.moe_ref_topk.restype = None
        h.moe_ref_topk.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p,
                                   C.c_void_p, C.c_void_p]
        h.moe_ref_gate_loss.restype = None
        h.moe_ref_gate_loss.argtypes = [C.c_uint32, C.c_uint32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                        C.c_void_p]
        h.moe_ref_slots.restype = None
        h.moe_ref_slots.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p,
                                    C.c_void_p, C.c_void_p, C.c_void_p]
        _lib = h
    return _lib


def threads() -> int:
    return int(lib().moe_ref_threads())


def make_cfg(S, H, I, E, k, capacity_factor=1.0, drop_tokens=1, hidden_act=0, dtype=2) -> RefCfg:
    c = RefCfg(S=S, H=H, I=I, E=E, k=k, capacity_factor=float(capacity_factor), drop_tokens=drop_tokens,
               hidden_act=hidden_act, dtype=dtype)
    if lib().moe_ref_derive(C.byref(c)) != 0:
        raise ValueError("moe_ref_derive rejected the shape")
    return c


def cfg_from_keys(keys) -> RefCfg:
    """keys: an object with the kleos_config.json attributes (aristos_amd.KleosConfig) or a dict."""
    g = (lambda n: keys[n]) if isinstance(keys, dict) else (lambda n: getattr(keys, n))
    return make_cfg(g("sequence_len") * g("mini_batch"), g("hidden_size"), g("intermediate_size"),
                    g("num_experts"), g("expert_top_k"), g("capacity_factor"), g("drop_tokens"),
                    g("hidden_act"), g("torch_dtype"))


def in_elems(c: RefCfg) -> int:
    return c.S * c.H + c.PX * c.H + 2 * c.E * c.I * c.H + c.E * c.I + c.E * c.H


def out_elems(c: RefCfg) -> int:
    return c.S * c.PX + c.S * c.H


def elem_np_dtype(c: RefCfg):
    return np.uint16 if c.dtype in (2, 3) else np.float32


def bf16_bits_to_f32(a: np.ndarray) -> np.ndarray:
    return (a.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    rounded = u + 0x7FFF + ((u >> 16) & 1)
    return (rounded >> 16).astype(np.uint16)


def round_tf32(a: np.ndarray) -> np.ndarray:
    """fp32 -> tf32 held in 32 bits: 10 mantissa bits, ties to even, the lower 13 bits cleared."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    finite = (u & 0x7F800000) != 0x7F800000
    r = np.where(finite, u + 0x0FFF + ((u >> 13) & 1), u) & 0xFFFFE000
    return r.astype(np.uint32).view(np.float32).reshape(a.shape)


def f32_to_elem_bits(a: np.ndarray, c: RefCfg) -> np.ndarray:
    """fp32 values -> the packed Element representation of the configuration."""
    if c.dtype == 1:
        return round_tf32(a)
    if c.dtype == 2:
        return f32_to_bf16_bits(a)
    if c.dtype == 3:
        return np.ascontiguousarray(a, dtype=np.float32).astype(np.float16).view(np.uint16)
    return np.ascontiguousarray(a, dtype=np.float32)


def elems_to_f32(a: np.ndarray, c: RefCfg) -> np.ndarray:
    if c.dtype == 2:
        return bf16_bits_to_f32(a)
    if c.dtype == 3:
        return np.ascontiguousarray(a).view(np.float16).astype(np.float32)
    return a.astype(np.float32)


def forward(c: RefCfg, iP: np.ndarray, logits: np.ndarray | None = None,
            token_mask: np.ndarray | None = None) -> dict:
    """Runs the whole layer. Returns gate_out [S,PX], moe_out [S,H] (fp32 views of Element values),
    the raw packed output, and every routing view. `logits` (fp32 [S,E]) overrides the gate GEMM."""
    dt = elem_np_dtype(c)
    iP = np.ascontiguousarray(iP)
    assert iP.dtype == dt and iP.size == in_elems(c), (iP.dtype, iP.size, in_elems(c))
    oP = np.zeros(out_elems(c), dtype=dt)
    S, E, k, R = c.S, c.E, c.k, c.cap_rows
    arrs = {
        "logits": np.empty((S, E), np.float32),
        "probs": np.empty((S, E), np.float32),
        "topk_expert": np.empty((S, k), np.int32),
        "topk_prob": np.empty((S, k), np.float32),
        "combine_den": np.empty((S,), np.float32),
        "topk_slot": np.empty((S, k), np.int32),
        "expert_count": np.empty((E,), np.uint32),
        "slot_token": np.empty((E, R), np.int32),
    }
    given = 0
    if logits is not None:
        arrs["logits"][...] = np.asarray(logits, dtype=np.float32).reshape(S, E)
        given = 1
    views = RefViews(**{n: a.ctypes.data for n, a in arrs.items()})
    mask_ptr = None
    if token_mask is not None:
        token_mask = np.ascontiguousarray(token_mask, dtype=np.uint8)
        assert token_mask.size == S
        mask_ptr = token_mask.ctypes.data
    rc = lib().moe_ref_forward(C.byref(c), iP.ctypes.data, oP.ctypes.data, C.byref(views), given, mask_ptr)
    if rc != 0:
        raise RuntimeError("moe_ref_forward failed")
    out = dict(arrs)
    out["oP"] = oP
    out["gate_out"] = elems_to_f32(oP[:S * c.PX], c).reshape(S, c.PX)
    out["moe_out"] = elems_to_f32(oP[S * c.PX:], c).reshape(S, c.H)
    return out


def gate_loss(c: RefCfg, probs: np.ndarray, expert_count: np.ndarray) -> dict:
    """Training-mode gate loss from the fp32 softmax probabilities [S,E] and the routed counts [E]."""
    probs = np.ascontiguousarray(probs, dtype=np.float32).reshape(c.S, c.E)
    cnt = np.ascontiguousarray(expert_count, dtype=np.uint32).reshape(c.E)
    mp = np.empty(c.E, np.float32)
    mc = np.empty(c.E, np.float32)
    loss = np.empty(1, np.float32)
    lib().moe_ref_gate_loss(c.S, c.E, probs.ctypes.data, cnt.ctypes.data, mp.ctypes.data, mc.ctypes.data,
                            loss.ctypes.data)
    return {"mean_prob": mp, "mean_count": mc, "loss": float(loss[0])}


def route(c: RefCfg, logits: np.ndarray) -> dict:
    """Softmax + top-k + slots on given fp32 logits (the routing half of the layer)."""
    S, E, k, R = c.S, c.E, c.k, c.cap_rows
    logits = np.ascontiguousarray(logits, dtype=np.float32).reshape(S, E)
    probs = np.empty((S, E), np.float32)
    te = np.empty((S, k), np.int32)
    tp = np.empty((S, k), np.float32)
    den = np.empty((S,), np.float32)
    ts = np.empty((S, k), np.int32)
    cnt = np.empty((E,), np.uint32)
    st = np.empty((E, R), np.int32)
    h = lib()
    h.moe_ref_softmax(S, E, logits.ctypes.data, probs.ctypes.data)
    h.moe_ref_topk(S, E, k, logits.ctypes.data, probs.ctypes.data, te.ctypes.data, tp.ctypes.data, den.ctypes.data)
    h.moe_ref_slots(S, E, k, c.EC, R, te.ctypes.data, ts.ctypes.data, cnt.ctypes.data, st.ctypes.data)
    return {"probs": probs, "topk_expert": te, "topk_prob": tp, "combine_den": den, "topk_slot": ts,
            "expert_count": cnt, "slot_token": st}
