"""An independent restatement of the layer in numpy (float64 GEMMs, vectorised routing), written
from the semantics table rather than from oracle/moe_ref.c, used only to pin the C oracle.

Semantics restated (reference csrc/include/kleos/...):
  logits = x Wg^T over the E real experts                           moe/gate.cuh:526-534
  p = softmax(logits) in fp32                                       moe/gate.cuh:556-584
  top-k by descending value, equal values -> lower index            moe/gate.cuh:654-670
  den = sum of the k selected p                                     moe/gate.cuh:669
  slot = rank of the token among those routed to e, token order;
         kept iff slot < EC                                         moe/gate.cuh:678-718
  h1 = Elem(act(x Wup^T + bup)), y = Elem(h1 Wdown^T + bdown)       os/processor/processor.cuh:706-741
  out[t] = sum_kept Elem(Elem(p_e) * Elem(y / den)) in Element      os/processor/processor.cuh:110-168
  k == 1: out[t] = y (unscaled)                                     os/processor/processor.cuh:170-203
"""
from __future__ import annotations

import math

import numpy as np


def round_bf16(a: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 -> fp32, round to nearest even, by integer arithmetic on the bit patterns."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16) << 16
    return (r & 0xFFFFFFFF).astype(np.uint32).view(np.float32).reshape(a.shape)


def round_tf32(a: np.ndarray) -> np.ndarray:
    """fp32 -> tf32 (10 mantissa bits, round to nearest even) -> fp32, by decomposing the value: the
    mantissa scaled to an integer of 11 bits, rounded by numpy's rint (ties to even), scaled back."""
    a = np.asarray(a, dtype=np.float32)
    m, e = np.frexp(a.astype(np.float64))          # a = m * 2^e, 0.5 <= |m| < 1
    return np.ldexp(np.rint(m * 2048.0) / 2048.0, e).astype(np.float32)


def to_elem(a, bf16):
    """bf16: True / "bf16" -> bfloat16, "f16" -> IEEE half (numpy's conversion), "tf32" -> 10 mantissa
    bits in 32, False -> fp32."""
    a = np.asarray(a, dtype=np.float32)
    if bf16 == "f16":
        return a.astype(np.float16).astype(np.float32)
    if bf16 == "tf32":
        return round_tf32(a)
    return round_bf16(a) if bf16 else a


def derive(S, E, k, cf, drop):
    PX = -(-E // 64) * 64
    base = -(-S // E) if drop else S
    EC = int(math.ceil(base * cf * k - 1e-9))
    pEC = -(-EC // 128) * 128
    return PX, EC, pEC, min(pEC, S)


def topk_lowest_index_first(logits: np.ndarray, k: int) -> np.ndarray:
    """Brute force: stable sort of (-value, index)."""
    S, E = logits.shape
    idx = np.broadcast_to(np.arange(E), (S, E))
    order = np.lexsort((idx, -logits.astype(np.float64)), axis=1)   # last key is primary
    return order[:, :k].astype(np.int32)


def slots_bruteforce(topk_expert: np.ndarray, E: int, EC: int, cap_rows: int):
    S, k = topk_expert.shape
    count = np.zeros(E, dtype=np.uint32)
    slot = np.full((S, k), -1, dtype=np.int32)
    slot_token = np.full((E, cap_rows), -1, dtype=np.int32)
    for t in range(S):
        for r in range(k):
            e = topk_expert[t, r]
            rank = int(count[e])
            count[e] += 1
            if rank < EC and rank < cap_rows:
                slot[t, r] = rank
                slot_token[e, rank] = t
    return slot, count, slot_token


def gelu_erf(v):
    from scipy.special import erf
    return 0.5 * v * (1.0 + erf(v / math.sqrt(2.0)))


def forward(x, wg, w_up, w_down, b_up, b_down, k, cf=1.0, drop=1, act=0, bf16=True, logits=None, elem=None):
    """x [S,H], wg [E,H], w_up [E,I,H], w_down [E,H,I], b_up [E,I], b_down [E,H]; all fp32 arrays
    holding Element-representable values. Returns a dict like the C oracle's."""
    if elem is not None:
        bf16 = elem
    S, H = x.shape
    E = wg.shape[0]
    PX, EC, pEC, cap_rows = derive(S, E, k, cf, drop)
    if logits is None:
        logits = (x.astype(np.float64) @ wg.astype(np.float64).T).astype(np.float32)
    l64 = logits.astype(np.float64)
    p = np.exp(l64 - l64.max(axis=1, keepdims=True))
    p = (p / p.sum(axis=1, keepdims=True)).astype(np.float32)
    te = topk_lowest_index_first(logits, k)
    tp = np.take_along_axis(p, te, axis=1)
    den = np.zeros(S, dtype=np.float32)
    for r in range(k):
        den = (den + tp[:, r]).astype(np.float32)
    slot, count, slot_token = slots_bruteforce(te, E, EC, cap_rows)

    gate_out = np.zeros((S, PX), dtype=np.float32)
    gate_out[:, :E] = to_elem(p, bf16)
    out = np.zeros((S, H), dtype=np.float32)
    actf = (lambda v: np.maximum(v, 0.0)) if act == 0 else gelu_erf
    # per-expert dense evaluation of the kept rows
    y_pair = {}
    for e in range(E):
        kept = min(int(count[e]), EC, cap_rows)
        if kept == 0:
            continue
        toks = slot_token[e, :kept]
        xe = x[toks].astype(np.float64)
        h1 = to_elem(actf(xe @ w_up[e].astype(np.float64).T + b_up[e].astype(np.float64)).astype(np.float32), bf16)
        y = to_elem((h1.astype(np.float64) @ w_down[e].astype(np.float64).T + b_down[e].astype(np.float64)).astype(np.float32), bf16)
        for i, t in enumerate(toks):
            y_pair[(int(t), e)] = y[i]
    for t in range(S):
        if k == 1:
            e = int(te[t, 0])
            if slot[t, 0] >= 0:
                out[t] = y_pair[(t, e)]
            continue
        acc = np.zeros(H, dtype=np.float32)
        for e in sorted(int(v) for v in te[t]):
            r = list(te[t]).index(e)
            if slot[t, r] < 0:
                continue
            v = to_elem(y_pair[(t, e)] / den[t], bf16)
            prod = to_elem(gate_out[t, e] * v, bf16)
            acc = to_elem(acc + prod, bf16)
        out[t] = acc
    return {"logits": logits, "probs": p, "topk_expert": te, "topk_prob": tp, "combine_den": den,
            "topk_slot": slot, "expert_count": count, "slot_token": slot_token, "gate_out": gate_out,
            "moe_out": out, "EC": EC, "cap_rows": cap_rows, "PX": PX}
