"""Synthetic workloads: the five layer configurations the benchmark and the parity tests use, and
seeded input generation in the packed buffer layout of the reference driver (csrc/main.cu:23-66:
activations, gate weights for the E real experts, per-expert up and down weights, zero biases).

Two generators:
  * ``portable_normal`` — a counter-based generator (SplitMix64 hash + Box-Muller) written out in
    numpy, so that committed fixtures can be regenerated bit-for-bit anywhere;
  * torch's generator on the target device, for large tensors where only "same inputs for the GPU
    and for the checker in this process" matters.
torch is used here for device memory and bulk random numbers only.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np

from .config import KleosConfig, DerivedConfig

_MASK = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(x: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        z = (x + np.uint64(0x9E3779B97F4A7C15)) & _MASK
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _MASK
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _MASK
        return z ^ (z >> np.uint64(31))


def portable_normal(seed: int, stream: int, n: int, std: float = 1.0, mean: float = 0.0) -> np.ndarray:
    """n samples of N(mean, std) as float32; element i of (seed, stream) never depends on n."""
    out = np.empty(n, dtype=np.float32)
    key = _splitmix64(np.array([(seed * 0x1000193 + stream * 0x9E3779B1 + 12345) & 0xFFFFFFFFFFFFFFFF],
                               dtype=np.uint64))[0]
    step = 1 << 22
    for a in range(0, n, step):
        b = min(n, a + step)
        idx = np.arange(a, b, dtype=np.uint64)
        with np.errstate(over="ignore"):
            h1 = _splitmix64((key + np.uint64(2) * idx) & _MASK)
            h2 = _splitmix64((key + np.uint64(2) * idx + np.uint64(1)) & _MASK)
        u1 = ((h1 >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)   # (0, 1]
        u2 = (h2 >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)           # [0, 1)
        z = np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * math.pi * u2)
        out[a:b] = (mean + std * z).astype(np.float32)
    return out


def portable_permutation(seed: int, stream: int, n: int) -> np.ndarray:
    """A permutation of 0..n-1: argsort of hashed keys (ties impossible for n << 2^64)."""
    key = _splitmix64(np.array([(seed * 0x1000193 + stream * 0x9E3779B1 + 777) & 0xFFFFFFFFFFFFFFFF],
                               dtype=np.uint64))[0]
    with np.errstate(over="ignore"):
        h = _splitmix64((key + np.arange(n, dtype=np.uint64)) & _MASK)
    return np.argsort(h, kind="stable")


@dataclass(frozen=True)
class Workload:
    name: str
    config: KleosConfig
    x_std: float
    w_std: float
    zipf_s: float = 0.0          # > 0: per-expert logit bias from a Zipf ranking, injected through the data
    hot_ratio: float = 0.0       # target load of the hottest expert relative to the mean
    forced_rows: tuple = ()      # non-empty (top-1 only): expert e is routed exactly forced_rows[e] tokens
    note: str = ""


def _cfg(S, H, I, E, k, cf, dtype) -> KleosConfig:
    return KleosConfig(capacity_factor=cf, drop_tokens=1, expert_top_k=k, hidden_act=0, hidden_size=H,
                       intermediate_size=I, mini_batch=1, num_experts=E, sequence_len=S, torch_dtype=dtype)


WORKLOADS = {
    "tiny_fp32": Workload("tiny_fp32", _cfg(128, 256, 512, 8, 2, 1.0, 0), 1.0, 0.02,
                          note="S=128 H=256 I=512 E=8 top-2 cf=1.0 fp32"),
    "balanced_e16": Workload("balanced_e16", _cfg(4096, 2048, 2048, 16, 2, 1.0, 2), 1.0, 0.02,
                             note="S=4096 H=I=2048 E=16 top-2 cf=1.0 bf16, balanced load"),
    "headline_e64_zipf": Workload("headline_e64_zipf", _cfg(8192, 2048, 2048, 64, 2, 1.0, 2), 1.0, 0.02,
                                  zipf_s=1.1, hot_ratio=4.0,
                                  note="S=8192 H=I=2048 E=64 top-2 cf=1.0 bf16, Zipf(1.1) logit bias, hottest ~4x mean"),
    "mixtral_e8": Workload("mixtral_e8", _cfg(8192, 4096, 14336, 8, 2, 1.25, 2), 1.0, 0.01,
                           note="S=8192 H=4096 I=14336 E=8 top-2 cf=1.25 bf16"),
    "fine_e256_top8": Workload("fine_e256_top8", _cfg(4096, 7168, 2048, 256, 8, 1.0, 2), 1.0, 0.01,
                               note="S=4096 H=7168 I=2048 E=256 top-8 cf=1.0 bf16"),
    # the expert projections of mixtral_e8 (16 384 rows over 8 experts) with every 256-row block full
    "mixtral_full_blocks": Workload("mixtral_full_blocks", _cfg(16384, 4096, 14336, 8, 1, 1.0, 2), 1.0, 0.01,
                                    forced_rows=(2048,) * 8,
                                    note="S=16384 H=4096 I=14336 E=8 top-1 cf=1.0 bf16, 2048 tokens routed to every expert"),
}


def scaled(workload: Workload, **overrides) -> Workload:
    """The same data recipe on different sizes (for parity tests the checker can finish quickly)."""
    cfg = KleosConfig(**{**workload.config.__dict__, **overrides})
    return Workload(workload.name + "_scaled", cfg, workload.x_std, workload.w_std, workload.zipf_s,
                    workload.hot_ratio, workload.forced_rows, workload.note)


def _torch_dtype(derived: DerivedConfig):
    import torch
    if derived.elem_bytes == 4:
        return torch.float32
    return torch.float16 if derived.keys.torch_dtype == 3 else torch.bfloat16


def make_inputs(workload: Workload, seed: int = 0, device: str = "cuda", portable: bool = False):
    """Returns (iP, derived): the packed input buffer as a 1-D torch tensor of Elements on `device`.

    portable=True draws every value from ``portable_normal`` (slow, reproducible anywhere);
    otherwise torch's generator on `device` is used.
    """
    import torch

    d = workload.config.derive()
    S, H, I, E, PX = d.S, d.H, d.I, d.E, d.PX
    dt = _torch_dtype(d)
    buf = torch.zeros(d.in_elems, dtype=dt, device=device)

    if portable:
        def draw(stream, n, std):
            return torch.from_numpy(portable_normal(seed, stream, n, std)).to(device)
    else:
        gen = torch.Generator(device=device)
        gen.manual_seed(seed)

        def draw(stream, n, std):
            return torch.randn(n, generator=gen, device=device, dtype=torch.float32) * std

    # main.cu:44-58: activations, gate weights (E*H only; rows E..PX stay zero), experts, zero bias
    buf[d.off_x:d.off_x + S * H] = draw(0, S * H, workload.x_std).to(dt)
    buf[d.off_gate_w:d.off_gate_w + E * H] = draw(1, E * H, workload.w_std).to(dt)
    for e in range(E):
        a = d.off_w_up + e * I * H
        buf[a:a + I * H] = draw(2 + 2 * e, I * H, workload.w_std).to(dt)
        b = d.off_w_down + e * H * I
        buf[b:b + H * I] = draw(3 + 2 * e, H * I, workload.w_std).to(dt)

    if workload.zipf_s > 0:
        _inject_zipf_bias(buf, d, workload, seed)
    if workload.forced_rows:
        _force_routing(buf, d, workload, seed)
    if d.keys.torch_dtype == 1:
        _round_tf32_(buf)   # main.cu:59-62 converts every input to Element, here tfloat32_t
    return buf, d


def _round_tf32_(buf) -> None:
    """In place: fp32 values to tf32 held in 32 bits (10 mantissa bits, ties to even, lower bits cleared)."""
    import torch
    u = buf.view(torch.int32)
    finite = (u & 0x7F800000) != 0x7F800000
    u.copy_(torch.where(finite, u + 0x0FFF + ((u >> 13) & 1), u) & ~0x1FFF)


def _force_routing(buf, d: DerivedConfig, w: Workload, seed: int) -> None:
    """Routing decided by the data (top-1): the first E hidden features of a token are one-hot in the
    expert it is meant for, and the gate weights read them back (Wg[e, :E] = unit vector e, the other
    gate weights damped), so that expert e receives exactly forced_rows[e] tokens, in a shuffled order."""
    import torch

    S, H, E = d.S, d.H, d.E
    assert d.k == 1 and len(w.forced_rows) == E and sum(w.forced_rows) == S
    x = buf[d.off_x:d.off_x + S * H].view(S, H)
    wg = buf[d.off_gate_w:d.off_gate_w + E * H].view(E, H)
    owner = np.repeat(np.arange(E), w.forced_rows)[portable_permutation(seed, 2000, S)]
    owner = torch.from_numpy(owner.astype(np.int64)).to(buf.device)
    x[:, :E] = 0.0
    x[torch.arange(S, device=buf.device), owner] = 8.0
    wg[:, :E] = torch.eye(E, dtype=buf.dtype, device=buf.device)
    wg[:, E:] *= 0.25


def _inject_zipf_bias(buf, d: DerivedConfig, w: Workload, seed: int) -> float:
    """Per-expert logit bias b_e = c * (-s * ln rank_e) carried by the data: the last hidden feature
    of every token is set to 1 and Wg[e, H-1] = b_e, so the gate (which has no bias term,
    reference gate.cuh:87-88) produces logits shifted by b_e. c is found by bisection so that the
    hottest expert is routed about hot_ratio times the mean load."""
    import torch

    S, H, E, k = d.S, d.H, d.E, d.k
    x = buf[d.off_x:d.off_x + S * H].view(S, H)
    wg = buf[d.off_gate_w:d.off_gate_w + E * H].view(E, H)
    x[:, H - 1] = 1.0
    wg[:, H - 1] = 0.0
    base = x.float() @ wg.float().t()                                   # logits without the bias
    rank = torch.from_numpy(portable_permutation(seed, 1000, E).astype(np.float64) + 1.0).to(buf.device)
    shape = (-w.zipf_s * torch.log(rank)).float()                       # <= 0, best-ranked expert has 0
    target = w.hot_ratio * S * k / E

    def hottest(c: float) -> int:
        bias = (c * shape).to(buf.dtype).float()
        top = torch.topk(base + bias, k, dim=1).indices
        return int(torch.bincount(top.flatten(), minlength=E).max())

    lo, hi = 0.0, 8.0
    for _ in range(24):
        mid = 0.5 * (lo + hi)
        if hottest(mid) < target:
            lo = mid
        else:
            hi = mid
    c = 0.5 * (lo + hi)
    wg[:, H - 1] = (c * shape).to(buf.dtype)
    return c


def alloc_outputs(d: DerivedConfig, device: str = "cuda"):
    import torch
    return torch.empty(d.out_elems, dtype=_torch_dtype(d), device=device)


def split_outputs(oP, d: DerivedConfig):
    """(gateOut[S, PX], moeOut[S, H]) views of the packed output buffer (moe.cuh:97-98)."""
    return (oP[d.off_gate_out:d.off_gate_out + d.S * d.PX].view(d.S, d.PX),
            oP[d.off_moe_out:d.off_moe_out + d.S * d.H].view(d.S, d.H))


def layer_flops(d: DerivedConfig, kept_pairs: int) -> float:
    """Algorithmic FLOPs of one forward: gate 2*S*H*E plus experts 4*T*H*I for T kept pairs."""
    return 2.0 * d.S * d.H * d.E + 4.0 * kept_pairs * d.H * d.I


def expert_flops(d: DerivedConfig, kept_pairs: int) -> float:
    return 4.0 * kept_pairs * d.H * d.I
