"""Pins the C oracle (oracle/moe_ref.c) without the reference running: the reference holds no
vectors for this path, so each function is checked against library routines at higher precision,
brute force, invariants and closed forms chosen so that a dropped term, a wrong index or a
transposed operand fails at least one of them."""
import numpy as np
import pytest
import torch

import np_restatement as npr
from helpers import pack_inputs, random_layer, rel_fro


# ------------------------------------------------------------------ derived sizes (types.cuh:471-507)
@pytest.mark.parametrize("S,H,I,E,k,cf,dt,PX,EC,pEC", [
    (128, 256, 512, 8, 2, 1.0, 0, 64, 32, 128),
    (4096, 2048, 2048, 16, 2, 1.0, 2, 64, 512, 512),
    (8192, 2048, 2048, 64, 2, 1.0, 2, 64, 256, 256),
    (8192, 4096, 14336, 8, 2, 1.25, 2, 64, 2560, 2560),
    (4096, 7168, 2048, 256, 8, 1.0, 2, 256, 128, 128),
    (384, 64, 64, 5, 3, 2.0, 2, 64, 462, 512),     # ceil(384/5)=77 -> 77*2*3
])
def test_derived_sizes_closed_form(oracle, S, H, I, E, k, cf, dt, PX, EC, pEC):
    c = oracle.make_cfg(S, H, I, E, k, cf, dtype=dt)
    assert (c.PX, c.EC, c.pEC) == (PX, EC, pEC)
    assert c.cap_rows == min(pEC, S)
    assert npr.derive(S, E, k, cf, 1)[:3] == (PX, EC, pEC)


def test_no_drop_capacity_is_S_times_cf_times_k(oracle):
    c = oracle.make_cfg(256, 64, 64, 4, 2, 1.0, drop_tokens=0)
    assert c.EC == 256 * 2 and c.cap_rows == 256


# ------------------------------------------------------------------ Element rounding
def test_bf16_round_matches_torch(oracle):
    rng = np.random.default_rng(1)
    v = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.integers(-20, 20, 20000),
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, 1e-40], np.float32)])
    want = torch.from_numpy(v).to(torch.bfloat16).float().numpy()
    got_np = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(v))
    got_c = np.array([oracle.lib().moe_ref_round_bf16(float(a)) for a in v[:2000]], np.float32)
    np.testing.assert_array_equal(got_np, want)
    np.testing.assert_array_equal(got_c, want[:2000])
    np.testing.assert_array_equal(npr.round_bf16(v), want)


# ------------------------------------------------------------------ gate GEMM
@pytest.mark.parametrize("dt", [0, 2])
def test_gate_logits_vs_fp64_matmul(oracle, dt):
    c = oracle.make_cfg(256, 320, 64, 24, 2, dtype=dt)
    x, wg, *_ = random_layer(c, seed=3)
    out = oracle.forward(c, pack_inputs(c, x, wg, np.zeros((c.E, c.I, c.H)), np.zeros((c.E, c.H, c.I))))
    want = torch.from_numpy(x).double() @ torch.from_numpy(wg).double().T
    err = np.abs(out["logits"] - want.numpy()).max()
    assert err < 2e-5, err
    # a transposed Wg or a stride bug would be O(1) off
    assert rel_fro(out["logits"], want.numpy()) < 1e-6


# ------------------------------------------------------------------ softmax
def test_softmax_vs_fp64_and_invariants(oracle):
    rng = np.random.default_rng(4)
    S, E = 128, 24
    c = oracle.make_cfg(S, 64, 64, E, 2)
    logits = (rng.standard_normal((S, E)) * 3).astype(np.float32)
    r = oracle.route(c, logits)
    want = torch.softmax(torch.from_numpy(logits).double(), dim=1).numpy()
    assert np.abs(r["probs"] - want).max() < 3e-7
    np.testing.assert_allclose(r["probs"].sum(axis=1), 1.0, atol=2e-6)
    shifted = oracle.route(c, logits + np.float32(7.0))
    assert np.abs(shifted["probs"] - r["probs"]).max() < 2e-6     # shift invariance
    huge = oracle.route(c, logits + np.float32(1e4))              # no overflow: max is subtracted
    assert np.isfinite(huge["probs"]).all()


def test_softmax_ignores_padded_experts(oracle):
    """E = 8 real experts inside PX = 64 columns: the 56 zero-weight columns must not enter the
    denominator (gate.cuh:550)."""
    c = oracle.make_cfg(128, 64, 64, 8, 2, dtype=0)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=5, w_std=0.5)
    out = oracle.forward(c, pack_inputs(c, x, wg, w_up, w_down))
    want = torch.softmax(torch.from_numpy(x).double() @ torch.from_numpy(wg).double().T, dim=1).numpy()
    assert np.abs(out["gate_out"][:, :8] - want).max() < 1e-6
    assert (out["gate_out"][:, 8:] == 0).all()
    np.testing.assert_allclose(out["gate_out"].sum(axis=1), 1.0, atol=1e-5)


# ------------------------------------------------------------------ top-k
def test_topk_vs_stable_sort_bruteforce(oracle):
    rng = np.random.default_rng(6)
    S, E, k = 256, 40, 5
    c = oracle.make_cfg(S, 64, 64, E, k)
    # coarse values -> many exact ties
    logits = rng.integers(-3, 4, size=(S, E)).astype(np.float32)
    r = oracle.route(c, logits)
    np.testing.assert_array_equal(r["topk_expert"], npr.topk_lowest_index_first(logits, k))
    # selected probabilities and their sum
    np.testing.assert_array_equal(r["topk_prob"], np.take_along_axis(r["probs"], r["topk_expert"], axis=1))
    den = np.zeros(S, np.float32)
    for j in range(k):
        den = den + r["topk_prob"][:, j]
    np.testing.assert_array_equal(r["combine_den"], den)


def test_topk_crafted_ties_and_k_equals_E(oracle):
    S, E = 128, 6
    c = oracle.make_cfg(S, 64, 64, E, 3)
    logits = np.zeros((S, E), np.float32)                     # all equal -> lowest indices 0,1,2
    r = oracle.route(c, logits)
    assert (r["topk_expert"] == np.array([0, 1, 2])).all()
    logits[:, 4] = 1.0; logits[:, 2] = 1.0                    # two equal maxima -> 2 before 4, then 0
    r = oracle.route(c, logits)
    assert (r["topk_expert"] == np.array([2, 4, 0])).all()
    cE = oracle.make_cfg(S, 64, 64, E, E)
    r = oracle.route(cE, np.random.default_rng(0).standard_normal((S, E)).astype(np.float32))
    assert (np.sort(r["topk_expert"], axis=1) == np.arange(E)).all()     # k = E selects everything
    np.testing.assert_allclose(r["combine_den"], 1.0, atol=1e-6)


# ------------------------------------------------------------------ slots / drops
@pytest.mark.parametrize("cf,drop", [(1.0, 1), (2.0, 1), (1.0, 0)])
def test_slots_vs_bruteforce_and_invariants(oracle, cf, drop):
    rng = np.random.default_rng(7)
    S, E, k = 384, 12, 3
    c = oracle.make_cfg(S, 64, 64, E, k, cf, drop_tokens=drop)
    logits = rng.standard_normal((S, E)).astype(np.float32)
    logits[:, 3] += 2.0                                        # a hot expert that overflows at cf = 1
    r = oracle.route(c, logits)
    slot, count, slot_token = npr.slots_bruteforce(r["topk_expert"], E, c.EC, c.cap_rows)
    np.testing.assert_array_equal(r["topk_slot"], slot)
    np.testing.assert_array_equal(r["expert_count"], count)
    np.testing.assert_array_equal(r["slot_token"], slot_token)
    assert int(count.sum()) == S * k
    for e in range(E):
        kept = min(int(count[e]), c.EC, c.cap_rows)
        toks = r["slot_token"][e, :kept]
        assert (np.diff(toks) > 0).all()                       # token order inside an expert
        assert (r["slot_token"][e, kept:] == -1).all()
        sel = np.argwhere(r["topk_expert"] == e)
        ranks = np.arange(len(sel))
        got = r["topk_slot"][sel[:, 0], sel[:, 1]]
        np.testing.assert_array_equal(got, np.where(ranks < kept, ranks, -1))   # kept iff rank < EC
    if drop == 0 or cf >= 2.0:
        assert (r["topk_slot"] >= 0).all() or cf == 2.0
    if drop == 0:
        assert (r["topk_slot"] >= 0).all()                     # nothing is ever dropped
    if cf == 1.0 and drop == 1:
        assert (r["topk_slot"][r["topk_expert"] == 3] < 0).any()   # the hot expert does drop


def test_single_expert_is_identity_permutation(oracle):
    c = oracle.make_cfg(128, 64, 64, 1, 1)
    r = oracle.route(c, np.zeros((128, 1), np.float32))
    np.testing.assert_array_equal(r["topk_slot"][:, 0], np.arange(128))
    np.testing.assert_array_equal(r["slot_token"][0], np.arange(128))


# ------------------------------------------------------------------ whole layer vs the numpy restatement
@pytest.mark.parametrize("dt,act,k,E,cf,bias", [
    (0, 0, 2, 8, 1.0, 0.0), (2, 0, 2, 8, 1.0, 0.0), (2, 1, 2, 8, 1.0, 0.1), (0, 1, 3, 12, 1.0, 0.1),
    (2, 0, 1, 4, 1.0, 0.1), (2, 0, 4, 4, 1.0, 0.0), (0, 0, 1, 1, 1.0, 0.2),
])
def test_layer_vs_numpy_restatement(oracle, dt, act, k, E, cf, bias):
    c = oracle.make_cfg(128, 128, 192, E, k, cf, hidden_act=act, dtype=dt)
    x, wg, w_up, w_down, b_up, b_down = random_layer(c, seed=11, w_std=0.08, bias_std=bias)
    got = oracle.forward(c, pack_inputs(c, x, wg, w_up, w_down, b_up, b_down))
    # feed the oracle's fp32 logits so that both route identically, then demand identical routing
    want = npr.forward(x, wg, w_up, w_down, b_up, b_down, k, cf, 1, act, bf16=(dt == 2), logits=got["logits"])
    for name in ("topk_expert", "topk_slot", "expert_count", "slot_token"):
        np.testing.assert_array_equal(got[name], want[name], err_msg=name)
    assert np.abs(got["probs"] - want["probs"]).max() < 3e-7
    assert np.abs(got["logits"] - (x.astype(np.float64) @ wg.astype(np.float64).T)).max() < 2e-5
    # fp64 GEMMs in the restatement vs fp32 accumulation here: bf16 results may differ by an ulp
    # where a sum lands next to a rounding boundary
    tol = 4e-3 if dt == 2 else 2e-6
    assert rel_fro(got["moe_out"], want["moe_out"]) < tol
    assert rel_fro(got["gate_out"], want["gate_out"]) < (2e-3 if dt == 2 else 1e-6)


# ------------------------------------------------------------------ combine closed forms
def _identity_layer(c, x, wg):
    E, H = c.E, c.H
    eye = np.broadcast_to(np.eye(H, dtype=np.float32), (E, H, H)).copy()
    return pack_inputs(c, x, wg, eye, eye)


@pytest.mark.parametrize("dt", [0, 2])
def test_identity_experts_return_input(oracle, dt):
    """H = I, Wup = Wdown = identity, x >= 0, zero bias, no drops: every expert returns x and the
    combine weights sum to one, so out = x (the reference author's 'eye weights' check,
    csrc/main.cu:16). Exact in fp32 up to the weight normalisation; bf16 within rounding."""
    c = oracle.make_cfg(128, 64, 64, 8, 2, 8.0, dtype=dt)     # cf = E: nothing dropped
    rng = np.random.default_rng(12)
    x = np.abs(rng.standard_normal((128, 64))).astype(np.float32)
    wg = rng.standard_normal((8, 64)).astype(np.float32) * 0.3
    if dt == 2:
        x, wg = npr.round_bf16(x), npr.round_bf16(wg)
    out = oracle.forward(c, _identity_layer(c, x, wg))
    assert (out["topk_slot"] >= 0).all()
    assert rel_fro(out["moe_out"], x) < (1e-2 if dt == 2 else 3e-7)


def test_identical_experts_give_kept_weight_share(oracle):
    """All experts identical: out[t] = FFN(x_t) * (sum of kept p) / (sum of selected p)."""
    c = oracle.make_cfg(128, 64, 128, 4, 2, 1.0, dtype=0)
    rng = np.random.default_rng(13)
    x = rng.standard_normal((128, 64)).astype(np.float32)
    wg = rng.standard_normal((4, 64)).astype(np.float32)
    wg[0] *= 3                                                  # expert 0 overflows -> some drops
    wu = rng.standard_normal((128, 64)).astype(np.float32) * 0.1
    wd = rng.standard_normal((64, 128)).astype(np.float32) * 0.1
    out = oracle.forward(c, pack_inputs(c, x, wg, np.broadcast_to(wu, (4, 128, 64)), np.broadcast_to(wd, (4, 64, 128))))
    ffn = np.maximum(x.astype(np.float64) @ wu.T.astype(np.float64), 0) @ wd.T.astype(np.float64)
    kept = (out["topk_slot"] >= 0)
    assert (~kept).any()
    share = (out["topk_prob"] * kept).sum(axis=1) / out["combine_den"]
    assert rel_fro(out["moe_out"], ffn * share[:, None]) < 2e-6


def test_k_equals_E_is_dense_mixture(oracle):
    """k = E and capacity for everything: out = sum_e p_e FFN_e(x)."""
    c = oracle.make_cfg(128, 64, 64, 4, 4, 4.0, dtype=0)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=14, w_std=0.2)
    out = oracle.forward(c, pack_inputs(c, x, wg, w_up, w_down))
    p = torch.softmax(torch.from_numpy(x).double() @ torch.from_numpy(wg).double().T, dim=1).numpy()
    want = np.zeros((128, 64))
    for e in range(4):
        want += p[:, e:e + 1] * (np.maximum(x.astype(np.float64) @ w_up[e].T, 0) @ w_down[e].T.astype(np.float64))
    assert rel_fro(out["moe_out"], want) < 2e-6


def test_k1_is_unscaled_argmax_expert_and_dropped_rows_are_zero(oracle):
    c = oracle.make_cfg(128, 64, 64, 4, 1, 1.0, dtype=0)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=15, w_std=0.3)
    out = oracle.forward(c, pack_inputs(c, x, wg, w_up, w_down))
    arg = np.argmax(x.astype(np.float64) @ wg.T.astype(np.float64), axis=1)
    np.testing.assert_array_equal(out["topk_expert"][:, 0], arg)
    dropped = out["topk_slot"][:, 0] < 0
    assert dropped.any() and (~dropped).any()
    for t in range(128):
        e = arg[t]
        want = np.zeros(64) if dropped[t] else np.maximum(x[t].astype(np.float64) @ w_up[e].T, 0) @ w_down[e].T
        assert np.abs(out["moe_out"][t] - want).max() < 1e-5     # no probability scaling when k = 1


def test_all_experts_dropped_gives_zero_row(oracle):
    """Every token prefers experts 0 and 1; capacity 64 each -> tokens 64.. lose both and must be zero."""
    c = oracle.make_cfg(128, 64, 64, 4, 2, 1.0, dtype=0)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=16, w_std=0.3)
    x[:, 0] = 50.0
    wg[:] = 0; wg[0, 0] = 1.0; wg[1, 0] = 0.5
    out = oracle.forward(c, pack_inputs(c, x, wg, w_up, w_down))
    assert c.EC == 64
    assert (out["topk_slot"][:64] >= 0).all() and (out["topk_slot"][64:] < 0).all()
    assert (out["moe_out"][64:] == 0).all() and np.abs(out["moe_out"][:64]).sum() > 0


def test_single_expert_is_plain_ffn(oracle):
    """E = 1 (the reference switches to a dense FFN kernel, moe.cuh:174-177)."""
    c = oracle.make_cfg(128, 64, 128, 1, 1, 1.0, dtype=0)
    x, wg, w_up, w_down, b_up, b_down = random_layer(c, seed=17, w_std=0.2, bias_std=0.1)
    out = oracle.forward(c, pack_inputs(c, x, wg, w_up, w_down, b_up, b_down))
    want = (np.maximum(x.astype(np.float64) @ w_up[0].T + b_up[0], 0)) @ w_down[0].T.astype(np.float64) + b_down[0]
    assert rel_fro(out["moe_out"], want) < 2e-6


def test_token_mask_matches_full_run(oracle):
    c = oracle.make_cfg(256, 64, 128, 8, 2, 1.0, dtype=2)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=18, w_std=0.1)
    iP = pack_inputs(c, x, wg, w_up, w_down)
    full = oracle.forward(c, iP)
    mask = np.zeros(256, np.uint8); mask[::7] = 1
    part = oracle.forward(c, iP, token_mask=mask)
    np.testing.assert_array_equal(part["moe_out"][mask == 1], full["moe_out"][mask == 1])
    assert (part["moe_out"][mask == 0] == 0).all()
    np.testing.assert_array_equal(part["topk_slot"], full["topk_slot"])


def test_given_logits_drive_the_routing(oracle):
    c = oracle.make_cfg(128, 64, 64, 8, 2, 1.0, dtype=0)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=19, w_std=0.1)
    iP = pack_inputs(c, x, wg, w_up, w_down)
    base = oracle.forward(c, iP)
    flipped = oracle.forward(c, iP, logits=-base["logits"])
    np.testing.assert_array_equal(flipped["topk_expert"], npr.topk_lowest_index_first(-base["logits"], 2))
    same = oracle.forward(c, iP, logits=base["logits"])
    np.testing.assert_array_equal(same["oP"], base["oP"])


# ------------------------------------------------------------------ training-mode gate loss
def test_gate_loss_uniform_logits_closed_form(oracle):
    """Equal logits: every probability is 1/E, so loss = sum_e (1/E)(c_e/S)/E = k/E^2 whatever the
    routing does (the counts sum to S*k)."""
    for S, E, k in ((256, 8, 2), (128, 64, 8), (384, 24, 3)):
        c = oracle.make_cfg(S=S, H=64, I=64, E=E, k=k, dtype=0)
        r = oracle.route(c, np.zeros((S, E), np.float32))
        g = oracle.gate_loss(c, r["probs"], r["expert_count"])
        assert abs(g["loss"] - k / E**2) < 1e-7
        np.testing.assert_allclose(g["mean_prob"], 1.0 / E, rtol=1e-6)
        # ties go to the lowest indices: the first k experts take every token
        np.testing.assert_allclose(g["mean_count"][:k], 1.0, rtol=0, atol=0)
        assert (g["mean_count"][k:] == 0).all()


def test_gate_loss_vs_numpy_and_invariants(oracle):
    rng = np.random.default_rng(17)
    S, E, k = 512, 48, 4
    c = oracle.make_cfg(S=S, H=64, I=64, E=E, k=k, dtype=0)
    logits = (rng.standard_normal((S, E)) * 2.0).astype(np.float32)
    r = oracle.route(c, logits)
    g = oracle.gate_loss(c, r["probs"], r["expert_count"])
    # independent: float64 softmax, counts from a brute-force top-k
    l64 = logits.astype(np.float64)
    p = np.exp(l64 - l64.max(1, keepdims=True)); p /= p.sum(1, keepdims=True)
    te = npr.topk_lowest_index_first(logits, k)
    counts = np.bincount(te.ravel(), minlength=E)
    expect = float((p.mean(0) * counts / S).sum() / E)
    assert abs(g["loss"] - expect) < 1e-6 * max(1.0, expect)
    assert abs(g["mean_prob"].sum() - 1.0) < 1e-5
    assert abs(g["mean_count"].sum() - k) < 1e-5
    # a transposed or mis-scaled term would break this: doubling one expert's count moves the loss
    # by exactly mean_prob[e] * count[e] / (S * E)
    cnt2 = r["expert_count"].copy(); cnt2[5] *= 2
    g2 = oracle.gate_loss(c, r["probs"], cnt2)
    assert abs((g2["loss"] - g["loss"]) - g["mean_prob"][5] * r["expert_count"][5] / (S * E)) < 1e-7


# ------------------------------------------------------------------ fp16 Element
def test_f16_round_matches_numpy(oracle):
    """The oracle's integer-arithmetic binary16 conversion against numpy's float16 (an independent
    implementation): random values over the whole range, exact ties, subnormals, overflow."""
    rng = np.random.default_rng(5)
    vals = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 4000).astype(np.float32),
        np.array([0.0, -0.0, 1.0, 65504.0, 65519.9, 65520.0, 65536.0, 1e6, -1e6, 2.0**-24, 2.0**-25, 1.5 * 2.0**-25,
                  2.0**-26, 6.1e-5, 6.097555e-05, 1.0 + 2.0**-11, 1.0 + 3 * 2.0**-11, 1.0 + 2.0**-11 + 2.0**-20],
                 dtype=np.float32),
    ])
    lib = oracle.lib()
    got = np.array([lib.moe_ref_f32_to_f16_bits(float(v)) for v in vals], dtype=np.uint16)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    np.testing.assert_array_equal(got, want)
    back = np.array([lib.moe_ref_f16_bits_to_f32(int(b)) for b in range(0, 0x7c00, 7)], dtype=np.float32)
    np.testing.assert_array_equal(back, np.arange(0, 0x7c00, 7, dtype=np.uint16).view(np.float16).astype(np.float32))


def test_layer_fp16_vs_numpy_restatement(oracle):
    """Whole layer with fp16 Elements against the independent restatement (which rounds with
    numpy's float16)."""
    c = oracle.make_cfg(S=128, H=64, I=128, E=8, k=2, dtype=3)
    x, wg, w_up, w_down, b_up, b_down = random_layer(c, seed=3, w_std=0.1, bias_std=0.05)
    iP = pack_inputs(c, x, wg, w_up, w_down, b_up, b_down)
    got = oracle.forward(c, iP)
    ref = npr.forward(x, wg, w_up, w_down, b_up, b_down, k=2, elem="f16")
    np.testing.assert_array_equal(got["topk_expert"], ref["topk_expert"])
    np.testing.assert_array_equal(got["topk_slot"], ref["topk_slot"])
    assert rel_fro(got["moe_out"], ref["moe_out"]) < 2e-3


def test_tf32_round_matches_an_independent_rounding(oracle):
    """tf32 keeps 10 mantissa bits. The oracle rounds on the bit pattern (add, mask); pinned against a
    rounding that never looks at bits (frexp, rint on the scaled mantissa, ldexp), on random values,
    exact ties (which go to the even neighbour), a carry into the exponent, and the special values."""
    lib = oracle.lib()
    rng = np.random.default_rng(11)
    vals = np.concatenate([rng.standard_normal(4000).astype(np.float32) * 3.0,
                           rng.standard_normal(2000).astype(np.float32) * 1e-20,
                           np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 1.0 + 2.0 ** -11 + 2.0 ** -20,
                                     2.0 - 2.0 ** -12, -(2.0 - 2.0 ** -12), 0.0, -0.0, 65504.0, 3.0e38], np.float32)])
    got = np.array([lib.moe_ref_round_tf32(float(v)) for v in vals], np.float32)
    np.testing.assert_array_equal(got, npr.round_tf32(vals))
    np.testing.assert_array_equal(got, oracle.round_tf32(vals))        # the wrapper's numpy form of the same bits
    assert (got.view(np.uint32) & 0x1FFF == 0).all()
    assert lib.moe_ref_round_tf32(1.0 + 2.0 ** -11) == 1.0                       # tie: down to the even mantissa
    assert lib.moe_ref_round_tf32(1.0 + 3 * 2.0 ** -11) == 1.0 + 2.0 ** -9       # tie: up to the even mantissa
    assert lib.moe_ref_round_tf32(2.0 - 2.0 ** -12) == 2.0                       # carries into the exponent
    assert np.isinf(lib.moe_ref_round_tf32(float("inf"))) and np.isnan(lib.moe_ref_round_tf32(float("nan")))
    # what a tensor core reads of an operand: the lower 13 bits dropped, nothing rounded
    assert lib.moe_ref_tf32_operand(1.0 + 2.0 ** -10 + 2.0 ** -11 + 2.0 ** -12) == 1.0 + 2.0 ** -10


def test_layer_tf32_vs_numpy_restatement(oracle):
    """Whole layer with tf32 Elements against the independent restatement; then the same layer with the
    lower mantissa bits of x and the weights filled in: a tf32 matrix product does not see them, the
    bias add does (it reads the stored 32 bits)."""
    c = oracle.make_cfg(S=128, H=64, I=128, E=8, k=2, dtype=1)
    x, wg, w_up, w_down, b_up, b_down = random_layer(c, seed=4, w_std=0.1, bias_std=0.05)
    iP = pack_inputs(c, x, wg, w_up, w_down, b_up, b_down)
    got = oracle.forward(c, iP)
    ref = npr.forward(x, wg, w_up, w_down, b_up, b_down, k=2, elem="tf32")
    np.testing.assert_array_equal(got["topk_expert"], ref["topk_expert"])
    np.testing.assert_array_equal(got["topk_slot"], ref["topk_slot"])
    assert rel_fro(got["moe_out"], ref["moe_out"]) < 2e-3
    assert (got["moe_out"].view(np.uint32) & 0x1FFF == 0).all() and (got["gate_out"].view(np.uint32) & 0x1FFF == 0).all()
    noisy = iP.copy()
    n_mm = c.S * c.H + c.PX * c.H + 2 * c.E * c.I * c.H          # everything in front of the bias vectors
    noisy[:n_mm] = (noisy[:n_mm].view(np.uint32) | 0x0ABC).view(np.float32)
    again = oracle.forward(c, noisy)
    np.testing.assert_array_equal(again["moe_out"], got["moe_out"])
    np.testing.assert_array_equal(again["logits"], got["logits"])
