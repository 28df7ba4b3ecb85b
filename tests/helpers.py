"""Shared helpers of the tests: packing layer tensors into the reference's buffer layout
(csrc/include/kleos/moe/moe.cuh:92-98) and error measures."""
from __future__ import annotations

import numpy as np

from oracle import moe_ref


def pack_inputs(c, x, wg, w_up, w_down, b_up=None, b_down=None) -> np.ndarray:
    """fp32 arrays (Element-representable for bf16 configs) -> packed Element buffer for `c` (RefCfg)."""
    S, H, I, E, PX = c.S, c.H, c.I, c.E, c.PX
    buf = np.zeros(moe_ref.in_elems(c), dtype=np.float32)
    o = 0
    buf[o:o + S * H] = np.asarray(x, np.float32).ravel(); o += S * H
    buf[o:o + E * H] = np.asarray(wg, np.float32).ravel(); o += PX * H
    buf[o:o + E * I * H] = np.asarray(w_up, np.float32).ravel(); o += E * I * H
    buf[o:o + E * H * I] = np.asarray(w_down, np.float32).ravel(); o += E * H * I
    if b_up is not None:
        buf[o:o + E * I] = np.asarray(b_up, np.float32).ravel()
    o += E * I
    if b_down is not None:
        buf[o:o + E * H] = np.asarray(b_down, np.float32).ravel()
    return moe_ref.f32_to_elem_bits(buf, c)


def unpack_inputs(c, iP: np.ndarray):
    S, H, I, E, PX = c.S, c.H, c.I, c.E, c.PX
    f = moe_ref.elems_to_f32(iP, c)
    o = 0
    x = f[o:o + S * H].reshape(S, H); o += S * H
    wg = f[o:o + E * H].reshape(E, H); o += PX * H
    w_up = f[o:o + E * I * H].reshape(E, I, H); o += E * I * H
    w_down = f[o:o + E * H * I].reshape(E, H, I); o += E * H * I
    b_up = f[o:o + E * I].reshape(E, I); o += E * I
    b_down = f[o:o + E * H].reshape(E, H)
    return x, wg, w_up, w_down, b_up, b_down


def rel_fro(a: np.ndarray, b: np.ndarray) -> float:
    """||a - b||_F / ||b||_F (b is the checker's result)."""
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    den = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / den) if den > 0 else float(np.linalg.norm(a - b))


def random_layer(c, seed=0, x_std=1.0, w_std=0.02, bias_std=0.0):
    """Seeded random layer tensors, rounded to Element when the config is bf16."""
    rng = np.random.default_rng(seed)
    S, H, I, E = c.S, c.H, c.I, c.E
    x = rng.standard_normal((S, H)).astype(np.float32) * x_std
    wg = rng.standard_normal((E, H)).astype(np.float32) * w_std
    w_up = rng.standard_normal((E, I, H)).astype(np.float32) * w_std
    w_down = rng.standard_normal((E, H, I)).astype(np.float32) * w_std
    b_up = rng.standard_normal((E, I)).astype(np.float32) * bias_std
    b_down = rng.standard_normal((E, H)).astype(np.float32) * bias_std
    if c.dtype == 2:
        from np_restatement import round_bf16
        x, wg, w_up, w_down, b_up, b_down = (round_bf16(a) for a in (x, wg, w_up, w_down, b_up, b_down))
    if c.dtype == 1:
        x, wg, w_up, w_down, b_up, b_down = (moe_ref.round_tf32(a) for a in (x, wg, w_up, w_down, b_up, b_down))
    if c.dtype == 3:
        x, wg, w_up, w_down, b_up, b_down = (a.astype(np.float16).astype(np.float32)
                                             for a in (x, wg, w_up, w_down, b_up, b_down))
    return x, wg, w_up, w_down, b_up, b_down
