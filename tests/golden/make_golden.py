"""Regenerates tests/golden/tiny_fp32_seed0.npz: the S=128 H=256 I=512 E=8 top-2 cf=1.0 fp32 layer
on seed-0 inputs from the portable generator, evaluated by the C oracle and cross-checked against
the independent numpy restatement before anything is written.

The reference holds no vectors for this path and cannot be built or run here (CUDA + NVSHMEM +
network-fetched CUTLASS), so the expected outputs come from the oracle, which tests/test_oracle_pins.py
pins by other means.

    python tests/golden/make_golden.py
"""
import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(HERE))

from aristos_amd import synth  # noqa: E402
from oracle import moe_ref  # noqa: E402
import np_restatement as npr  # noqa: E402
from helpers import unpack_inputs, rel_fro  # noqa: E402


def main():
    w = synth.WORKLOADS["tiny_fp32"]
    iP, d = synth.make_inputs(w, seed=0, device="cpu", portable=True)
    iP = iP.numpy()
    c = moe_ref.cfg_from_keys(w.config)
    out = moe_ref.forward(c, iP)
    x, wg, w_up, w_down, b_up, b_down = unpack_inputs(c, iP)
    chk = npr.forward(x, wg, w_up, w_down, b_up, b_down, c.k, 1.0, 1, 0, bf16=False, logits=out["logits"])
    for name in ("topk_expert", "topk_slot", "expert_count", "slot_token"):
        np.testing.assert_array_equal(out[name], chk[name], err_msg=name)
    assert rel_fro(out["moe_out"], chk["moe_out"]) < 2e-6
    # the fixture must not sit on a routing knife edge: gap between the k-th and (k+1)-th logit
    srt = np.sort(out["logits"], axis=1)[:, ::-1]
    gap = float((srt[:, c.k - 1] - srt[:, c.k]).min())
    assert gap > 1e-4, gap
    assert (out["topk_slot"] < 0).any(), "the fixture should exercise token dropping"
    np.savez_compressed(
        os.path.join(HERE, "tiny_fp32_seed0.npz"),
        input_sha256=np.frombuffer(hashlib.sha256(iP.tobytes()).digest(), dtype=np.uint8),
        logits=out["logits"], topk_expert=out["topk_expert"], topk_slot=out["topk_slot"],
        expert_count=out["expert_count"], combine_den=out["combine_den"],
        gate_out=out["gate_out"][:, :c.E].copy(), moe_out=out["moe_out"], min_logit_gap=np.float32(gap))
    print("wrote tiny_fp32_seed0.npz; min top-k logit gap", gap, "dropped pairs", int((out["topk_slot"] < 0).sum()))


if __name__ == "__main__":
    main()
