"""Parity of the HIP path against the CPU oracle, through the C ABI (ctypes), on a real MI355X.

Protocol (the reference's routing is decided by fp32 logits whose last bits depend on the GEMM's
summation order, so it is checked "given the same fp32 logits"):
  1. GPU logits vs oracle logits: within tolerance;
  2. oracle routing applied to the GPU's own fp32 logits == GPU routing, bit for bit
     (top-k experts in selection order, slots, drops, per-expert counts, slot->token table);
  3. oracle outputs computed from the GPU's logits vs GPU outputs: relative Frobenius error
     <= 1e-2 for bf16, <= 1e-5 for fp32 (the tolerances the task states).
"""
import os

import numpy as np
import pytest
import torch

import aristos_amd as ka
from aristos_amd import synth
from helpers import pack_inputs, random_layer, rel_fro
from oracle import moe_ref

pytestmark = pytest.mark.gpu

TOL_OUT = {0: 1e-5, 1: 2e-3, 2: 1e-2, 3: 2e-3}      # relative Frobenius, moeOut (tf32 keeps 10 mantissa bits, like fp16)
TOL_LOGIT = {0: 2e-5, 1: 2e-5, 2: 2e-5, 3: 2e-5}    # absolute, fp32 accumulation of exact products, different order
TOL_PROB = {0: 2e-6, 1: 5e-4, 2: 4e-3, 3: 5e-4}     # gateOut: fp32 exp/div ulps, or one bf16 / fp16 rounding


def tol_out(c):
    """moeOut. The reference adds the k scaled expert rows of a token into the output one by one in
    Element (atomicAdd, processor.cuh:157,165), and so does the oracle: k roundings of the running sum,
    a random walk of about u * sqrt(k / 3) relative (u = 2^-9 for bf16: 0.96 % at k = 72), while the GPU
    sums in fp32 and rounds once. Up to k = 16 that stays inside the stated tolerance; above, the bound
    grows with sqrt(k) like the walk it allows for (k = 72 in bf16 measures 1.2 %)."""
    return TOL_OUT[c.dtype] * max(1.0, (c.k / 16.0) ** 0.5)


def tol_prob(c):
    """gateOut. In fp32 the softmax denominator is a sum of E terms that the GPU adds in a tree over lanes
    and the oracle in index order (gate.cuh:574-580): next to a probability close to 1 the two orders
    differ by about 2^-24 * sqrt(E) (500 experts with one dominant expert measure 2.4e-6). The bound
    grows with sqrt(E) above 128 experts; the 16-bit Elements are bounded by their own rounding."""
    if c.dtype == 0:
        return TOL_PROB[0] * max(1.0, (c.E / 128.0) ** 0.5)
    return TOL_PROB[c.dtype]


def _to_device(c, iP_np):
    if c.dtype in (2, 3):
        return torch.from_numpy(iP_np.view(np.int16)).cuda().view(torch.bfloat16 if c.dtype == 2 else torch.float16)
    return torch.from_numpy(iP_np).cuda()


def _out_to_np(c, oP):
    if c.dtype in (2, 3):
        return oP.view(torch.int16).cpu().numpy().view(np.uint16)
    return oP.cpu().numpy()


def _apply(mode):
    """mode: a MODE_* value or a (MODE_*, SCHEDULE_*) pair."""
    if isinstance(mode, tuple):
        ka.moe.set_mode(mode[0])
        ka.moe.set_schedule(mode[1])
    else:
        ka.moe.set_mode(mode)


def run_gpu(keys: ka.KleosConfig, iP_dev, mode, launches=1):
    d = ka.initialize(keys)
    try:
        _apply(mode)
        oP = synth.alloc_outputs(d)
        oP.fill_(float("nan"))           # every output element must be written by the layer
        torch.cuda.synchronize()
        for _ in range(launches):
            ka.moe.forward_host(iP_dev, oP)
        ka.moe.stream_synchronize()
        views = ka.moe.debug_views(d)
        return d, oP, views
    finally:
        ka.finalize()


def check_against_oracle(c, keys, iP_np, mode, launches=1, token_mask=None, logits_ref=None):
    iP_dev = _to_device(c, iP_np)
    d, oP, v = run_gpu(keys, iP_dev, mode, launches)
    assert (d.S, d.PX, d.EC, d.cap_rows) == (c.S, c.PX, c.EC, c.cap_rows)
    ref = moe_ref.forward(c, iP_np, logits=v["logits"], token_mask=token_mask)
    # 1. logits
    if logits_ref is None:
        logits_ref = moe_ref.forward(c, iP_np, token_mask=np.zeros(c.S, np.uint8))["logits"]
    assert np.abs(v["logits"] - logits_ref).max() < TOL_LOGIT[c.dtype] * max(1.0, np.abs(logits_ref).max())
    # 2. routing, bit-exact given the same logits
    np.testing.assert_array_equal(v["topk_expert"], ref["topk_expert"])
    np.testing.assert_array_equal(v["topk_slot"], ref["topk_slot"])
    np.testing.assert_array_equal(v["expert_count"], ref["expert_count"])
    for e in range(c.E):
        kept = min(int(ref["expert_count"][e]), c.EC, c.cap_rows)
        np.testing.assert_array_equal(v["slot_token"][e, :kept], ref["slot_token"][e, :kept])
    # probabilities: the fast exponential of the GPU against expf of the oracle, a few ulp of values up to 1
    assert np.abs(v["topk_prob"] - ref["topk_prob"]).max() < 4e-6
    assert np.abs(v["combine_den"] - ref["combine_den"]).max() < 8e-6
    # 3. outputs
    out = moe_ref.elems_to_f32(_out_to_np(c, oP), c)
    assert np.isfinite(out).all(), "the layer left output elements unwritten"
    gate_out = out[:c.S * c.PX].reshape(c.S, c.PX)
    moe_out = out[c.S * c.PX:].reshape(c.S, c.H)
    assert np.abs(gate_out - ref["gate_out"]).max() < tol_prob(c)
    assert (gate_out[:, c.E:] == 0).all()
    if token_mask is not None:
        sel = token_mask.astype(bool)
        err = rel_fro(moe_out[sel], ref["moe_out"][sel])
    else:
        err = rel_fro(moe_out, ref["moe_out"])
    assert err < tol_out(c), f"relative Frobenius error {err}"
    # tokens dropped by every expert are zero rows
    all_dropped = (v["topk_slot"] < 0).all(axis=1)
    assert (moe_out[all_dropped] == 0).all()
    return d, v, moe_out, err


# (mode, schedule of the persistent launch)
MODES = [(ka.MODE_PHASED, ka.SCHEDULE_AUTO), (ka.MODE_FUSED, ka.SCHEDULE_DYNAMIC), (ka.MODE_FUSED, ka.SCHEDULE_STATIC)]
MODE_IDS = ["phased", "fused", "fused-static"]


def _keys(S, H, I, E, k, cf=1.0, drop=1, act=0, dt=2):
    return ka.KleosConfig(capacity_factor=cf, drop_tokens=drop, expert_top_k=k, hidden_act=act, hidden_size=H,
                          intermediate_size=I, num_experts=E, sequence_len=S, mini_batch=1, torch_dtype=dt)


# ------------------------------------------------------------------ the reference's CPU-sized case
@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
def test_tiny_fp32_config(mode):
    """S=128 H=256 I=512 E=8 top-2 cf=1.0 fp32, seed 0."""
    w = synth.WORKLOADS["tiny_fp32"]
    iP, d = synth.make_inputs(w, seed=0, device="cpu", portable=True)
    c = moe_ref.cfg_from_keys(w.config)
    d, v, moe_out, _ = check_against_oracle(c, w.config, iP.numpy(), mode)
    # and against the committed fixture of this configuration
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_fp32_seed0.npz"))
    assert np.abs(v["logits"] - g["logits"]).max() < 2e-5 < float(g["min_logit_gap"]) / 4
    np.testing.assert_array_equal(v["topk_expert"], g["topk_expert"])
    np.testing.assert_array_equal(v["topk_slot"], g["topk_slot"])
    np.testing.assert_array_equal(v["expert_count"], g["expert_count"])
    assert rel_fro(moe_out, g["moe_out"]) < 1e-5


# ------------------------------------------------------------------ shapes and edge cases
CASES = [
    # S, H, I, E, k, cf, drop, act, dt, bias_std
    (256, 128, 256, 8, 2, 1.0, 1, 0, 2, 0.0),
    (256, 128, 256, 8, 2, 1.0, 1, 1, 2, 0.1),      # gelu + biases
    (256, 192, 320, 12, 3, 1.0, 1, 0, 2, 0.1),     # E not a multiple of 8, H and I not multiples of 128
    (256, 128, 128, 16, 1, 1.0, 1, 0, 2, 0.0),     # k = 1: unscaled copy, dropped rows zero
    (128, 128, 128, 4, 4, 1.0, 1, 0, 2, 0.0),      # k = E: dense mixture
    (128, 128, 256, 1, 1, 1.0, 1, 0, 2, 0.1),      # E = 1: plain FFN
    (256, 128, 128, 8, 2, 1.0, 0, 0, 2, 0.0),      # drop_tokens = 0
    (256, 128, 128, 8, 2, 2.5, 1, 0, 2, 0.0),      # real-valued capacity factor
    (512, 128, 128, 64, 2, 1.0, 1, 0, 2, 0.0),     # E = 64
    (256, 128, 64, 130, 8, 1.0, 1, 0, 2, 0.0),     # E > 128 (gate handles up to 256 experts)
    (256, 128, 64, 256, 8, 1.0, 1, 0, 2, 0.0),     # E = 256, top-8
    (128, 128, 64, 96, 72, 1.0, 1, 0, 3, 0.0),     # fp16, 64 < E <= 256 with k > 64: more picks per token than a wavefront has lanes
    (128, 128, 64, 96, 72, 1.0, 1, 0, 2, 0.0),     # the same in bf16: 72 Element additions per output row in the oracle (tol_out)
    (256, 448, 320, 500, 20, 1.25, 0, 0, 0, 0.1),  # fp32, 500 experts, top-20, no dropping: the softmax denominator's 500 terms (tol_prob)
    (256, 128, 64, 200, 5, 1.5, 1, 0, 3, 0.1),     # fp16, E = 200 (padded to 256 columns, not a multiple of 16)
    (256, 128, 192, 8, 2, 1.0, 1, 1, 0, 0.1),      # fp32 + gelu
    (256, 64, 64, 24, 3, 1.0, 1, 0, 0, 0.0),       # fp32, E = 24
    (256, 128, 192, 8, 2, 1.0, 1, 0, 1, 0.1),      # tf32 (the dtype the reference ships): 32-bit Elements of 10 mantissa bits
    (512, 192, 128, 64, 2, 1.0, 1, 1, 1, 0.1),     # tf32, E = 64, gelu
    (256, 64, 64, 300, 4, 1.0, 1, 0, 1, 0.0),      # tf32, E = 300: the gate in passes
    (1024, 192, 320, 4, 2, 1.0, 1, 0, 2, 0.1),     # 512 rows per expert: 256-row tiles, odd slice counts
    (512, 64, 64, 2, 1, 1.0, 1, 1, 2, 0.1),        # 256-row tiles over a single K slice
    (768, 128, 192, 2, 2, 1.0, 1, 0, 3, 0.0),      # fp16, 256-row tiles, a partial row block
    (256, 128, 256, 8, 2, 1.0, 1, 0, 3, 0.0),      # fp16
    (256, 192, 320, 12, 3, 1.0, 1, 1, 3, 0.1),     # fp16, gelu + biases, ragged sizes
    (512, 256, 256, 64, 2, 1.0, 1, 0, 3, 0.0),     # fp16, E = 64, several K slices
    (2048, 192, 320, 2, 2, 1.0, 1, 1, 2, 0.1),     # 2048 rows per expert: the tile variant of large experts
    (512, 128, 64, 320, 8, 1.0, 1, 0, 2, 0.0),     # E > 256: the gate in passes of 256 experts
    (256, 192, 64, 512, 6, 2.0, 1, 1, 2, 0.1),     # E = 512, cf = 2, gelu + biases
    (256, 64, 64, 384, 4, 1.0, 1, 0, 0, 0.0),      # fp32, E = 384
    (256, 1088, 64, 320, 4, 1.0, 1, 0, 2, 0.0),    # E = 320 over a long hidden dimension: batched and single K steps
    (128, 320, 64, 96, 40, 1.0, 1, 0, 2, 0.0),     # 40 picks per token (the combine that re-reads its routing) over output rows of two 256-column pieces
    (256, 576, 128, 16, 2, 1.0, 1, 1, 3, 0.1),     # fp16, output rows of two pieces and a quarter
]


@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
@pytest.mark.parametrize("S,H,I,E,k,cf,drop,act,dt,bias", CASES)
def test_shapes_and_edges(mode, S, H, I, E, k, cf, drop, act, dt, bias):
    keys = _keys(S, H, I, E, k, cf, drop, act, dt)
    c = moe_ref.cfg_from_keys(keys)
    x, wg, w_up, w_down, b_up, b_down = random_layer(c, seed=S + E + k, w_std=0.08, bias_std=bias)
    wg[0] *= 2.5                                      # an expert that overflows its capacity
    if c.dtype == 2:
        from np_restatement import round_bf16
        wg = round_bf16(wg)
    iP = pack_inputs(c, x, wg, w_up, w_down, b_up, b_down)
    check_against_oracle(c, keys, iP, mode)


def _drawn_case(index):
    """A configuration drawn from a fixed seed: sizes, expert count (1 to 512, around every boundary of
    the gate variants), top-k, capacity factor, activation, Element type and bias at random."""
    import random
    rng = random.Random(1000 + index)
    S = rng.choice([128, 256, 384, 512, 1024])
    H, I = 64 * rng.randint(1, 8), 64 * rng.randint(1, 8)
    E = rng.choice([1, 2, 3, 5, 8, 12, 16, 24, 33, 64, 65, 70, 96, 128, 129, 130, 192, 200, 255, 256, 257, 300, 384, 500, 512])
    k = rng.randint(1, min(E, rng.choice([2, 4, 8, 16, 32])))
    cf = rng.choice([1.0, 1.0, 1.25, 1.5, 2.5, 4.0])
    return (S, H, I, E, k, cf, rng.choice([0, 1, 1]), rng.choice([0, 1]), rng.choice([2, 2, 3, 0]), rng.choice([0.0, 0.1]))


@pytest.mark.parametrize("index", range(12))
def test_drawn_configurations(index):
    """Twelve configurations nobody picked by hand, each through the phased launches and the persistent
    launch under both schedules."""
    for mode in MODES:
        test_shapes_and_edges(mode, *_drawn_case(index))


@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
def test_exact_ties_go_to_the_lower_index(mode):
    """Duplicate gate rows give bit-identical logits for expert pairs; the lower index must win, and
    an all-equal row must select experts 0..k-1."""
    keys = _keys(256, 128, 128, 16, 3)
    c = moe_ref.cfg_from_keys(keys)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=5, w_std=0.1)
    wg[5] = wg[2]; wg[9] = wg[2]; wg[11] = wg[7]
    x[:16] = 0.0                                      # all logits exactly 0 for these tokens
    iP = pack_inputs(c, x, wg, w_up, w_down)
    d, v, _, _ = check_against_oracle(c, keys, iP, mode)
    assert (v["topk_expert"][:16] == np.array([0, 1, 2])).all()
    lg = v["logits"]
    assert (lg[:, 5] == lg[:, 2]).all() and (lg[:, 11] == lg[:, 7]).all()
    te = v["topk_expert"]
    for t in range(256):
        sel = list(te[t])
        if 5 in sel: assert 2 in sel and sel.index(2) < sel.index(5)
        if 9 in sel: assert 5 in sel
        if 11 in sel: assert 7 in sel and sel.index(7) < sel.index(11)


@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
def test_everything_routed_to_two_experts(mode):
    """Heavy overflow: every token prefers experts 0 and 1, the rest of the batch is dropped whole."""
    keys = _keys(512, 128, 128, 8, 2, dt=0)
    c = moe_ref.cfg_from_keys(keys)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=6, w_std=0.1)
    x[:, 0] = 30.0
    wg[:] = 0; wg[0, 0] = 1.0; wg[1, 0] = 0.5
    d, v, moe_out, _ = check_against_oracle(c, keys, pack_inputs(c, x, wg, w_up, w_down), mode)
    assert c.EC == 128
    assert (v["topk_slot"][:128] >= 0).all() and (v["topk_slot"][128:] < 0).all()
    assert (moe_out[128:] == 0).all()


@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
def test_identity_experts_return_input(mode):
    """The reference author's own check (csrc/main.cu:16): identity expert weights."""
    keys = _keys(256, 128, 128, 8, 2, cf=8.0, dt=0)
    c = moe_ref.cfg_from_keys(keys)
    rng = np.random.default_rng(7)
    x = np.abs(rng.standard_normal((256, 128))).astype(np.float32)
    wg = rng.standard_normal((8, 128)).astype(np.float32) * 0.2
    eye = np.broadcast_to(np.eye(128, dtype=np.float32), (8, 128, 128))
    d, v, moe_out, _ = check_against_oracle(c, keys, pack_inputs(c, x, wg, eye, eye), mode)
    assert rel_fro(moe_out, x) < 1e-6


@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
@pytest.mark.parametrize("k", [1, 2])
def test_tile_heights_mixed_inside_one_layer(mode, k):
    """A layer whose experts may hold 1024 rows and more walks 256-row blocks, and gives an expert's last
    block to a 128-row tile when it holds at most 128 rows: experts of 40, 100, 129, 300, 2100 and 403
    rows (and two without any) in one launch, i.e. blocks of 40 and 100 rows (128-row tile), 129 rows
    (256-row tile), 256 + 44, 8 x 256 + 52 (full tiles followed by a 128-row tile) and 256 + 147. With
    k = 2 every token also goes to the next expert, which gives blocks of 140, 229, 173, 96 and 199
    rows. Token t is sent to its experts by one-hot input features that the gate weights pick up."""
    S, H, I, E = 3072, 128, 256, 8
    keys = _keys(S, H, I, E, k, cf=1.0, drop=0)
    c = moe_ref.cfg_from_keys(keys)
    assert c.cap_rows >= 1024
    x, wg, w_up, w_down, b_up, b_down = random_layer(c, seed=91, w_std=0.08, bias_std=0.1)
    rows = [40, 100, 129, 300, 2100, 403, 0, 0]
    first = np.repeat(np.arange(E), rows)
    rng = np.random.default_rng(5)
    rng.shuffle(first)
    x[:, :E] = 0.0
    x[np.arange(S), first] = 8.0
    x[np.arange(S), (first + 1) % E] = 4.0
    wg[:, :E] = np.eye(E, dtype=np.float32)
    wg[:, E:] *= 0.25                                  # the other features only perturb the logits (by about 0.2)
    iP = pack_inputs(c, x, wg, w_up, w_down, b_up, b_down)
    d, v, moe_out, err = check_against_oracle(c, keys, iP, mode)
    expect = np.array(rows)
    if k == 2:
        expect = expect + np.roll(expect, 1)
    np.testing.assert_array_equal(v["expert_count"], expect)
    assert (v["topk_slot"] >= 0).all()


def test_last_down_tiles_of_a_queue_are_handed_out_in_halves():
    """Dynamic schedule of a layer that holds both tile heights: every XCD queue hands out its last
    down-projection tiles (as many as half of the XCD's workgroups) as two tickets of 128 rows each,
    except where a last block holds at most 128 rows anyway. The persistent launch therefore counts
    more tiles than row blocks x column tiles, by a number the test works out from the rows per expert,
    and its output has the bits of the separate launches per phase, which never halve a tile."""
    S, H, I, E, k = 3072, 512, 256, 8, 2
    keys = _keys(S, H, I, E, k, cf=1.0, drop=0)
    c = moe_ref.cfg_from_keys(keys)
    assert c.cap_rows >= 1024
    x, wg, w_up, w_down, b_up, b_down = random_layer(c, seed=93, w_std=0.08, bias_std=0.1)
    rows = [40, 100, 129, 300, 2100, 403, 0, 0]
    first = np.repeat(np.arange(E), rows)
    np.random.default_rng(6).shuffle(first)
    x[:, :E] = 0.0
    x[np.arange(S), first] = 8.0
    x[np.arange(S), (first + 1) % E] = 4.0
    wg[:, :E] = np.eye(E, dtype=np.float32)
    wg[:, E:] *= 0.25
    iP_np = pack_inputs(c, x, wg, w_up, w_down, b_up, b_down)
    iP = _to_device(c, iP_np)
    _, ref, v = run_gpu(keys, iP, ka.MODE_PHASED)
    ref = _out_to_np(c, ref)
    kept = np.array(rows) + np.roll(rows, 1)
    np.testing.assert_array_equal(v["expert_count"], kept)
    d = ka.initialize(keys)
    try:
        ka.moe.set_mode(ka.MODE_FUSED)
        ka.moe.set_schedule(ka.SCHEDULE_DYNAMIC)
        oP = synth.alloc_outputs(d)
        ka.moe.forward_host(iP, oP)
        ka.moe.stream_synchronize()
        np.testing.assert_array_equal(_out_to_np(c, oP), ref)
        ka.moe.forward_host_bench(iP, oP, skip=1, trials=2)
        np.testing.assert_array_equal(_out_to_np(c, oP), ref)
        st = ka.moe.scheduler_stats()
        members = ka.moe.phase_stamps().shape[0] // 8        # workgroups per XCD
    finally:
        ka.finalize()
    tn_up, tn_down = -(-I // 256), -(-H // 256)
    expect = 0
    for r in kept:                                       # by-index placement: queue q holds expert q alone
        mt = -(-int(r) // 256)
        expect += mt * (tn_up + tn_down)
        tiles = [(n, m) for n in range(tn_down) for m in range(mt)]      # row blocks fastest
        for n, m in tiles[len(tiles) - min(len(tiles), members // 2):]:
            expect += int(r - m * 256 > 128)             # a second ticket unless the block fits one 128-row tile
    assert members >= 2 and int(st["tiles"]) == expect
    assert expect > sum(-(-int(r) // 256) for r in kept) * (tn_up + tn_down)


@pytest.mark.parametrize("dt", [2, 0])
def test_dense_packing_of_a_single_expert(dt):
    """num_experts == 1 on the packing the reference's fffn kernel reads (fffn.cuh:43-49): iP = x | Wup |
    Wdown | bup | bdown with no gate weights, oP = moeOut with no gate output. kleos_moe_forward_dense
    gives the bits kleos_moe_forward gives on the driver's packing of the same operands (which the
    other tests check against the oracle), and refuses a context with more than one expert."""
    S, H, I = 256, 128, 192                            # I != H: the second bias vector follows I entries
    keys = _keys(S, H, I, 1, 1, dt=dt)
    c = moe_ref.cfg_from_keys(keys)
    x, wg, w_up, w_down, b_up, b_down = random_layer(c, seed=57, w_std=0.08, bias_std=0.1)
    iP_np = pack_inputs(c, x, wg, w_up, w_down, b_up, b_down)
    check_against_oracle(c, keys, iP_np, ka.MODE_FUSED)
    # the same operands without the 64 x H gate block: everything behind x moves up
    dense_np = np.concatenate([iP_np[:S * H], iP_np[S * H + c.PX * H:]])
    assert dense_np.size == S * H + 2 * I * H + I + H
    d = ka.initialize(keys)
    try:
        oP = synth.alloc_outputs(d)
        ka.moe.forward_host(_to_device(c, iP_np), oP)
        ka.moe.stream_synchronize()
        want = _out_to_np(c, oP)[S * c.PX:].copy()
        dense_out = torch.full((S * H,), float("nan"), dtype=oP.dtype, device="cuda")
        for mode in (ka.MODE_FUSED, ka.MODE_PHASED):
            ka.moe.set_mode(mode)
            dense_out.fill_(float("nan"))
            torch.cuda.synchronize()
            ka.moe.forward_host_dense(_to_device(c, dense_np), dense_out)
            ka.moe.stream_synchronize()
            np.testing.assert_array_equal(_out_to_np(c, dense_out), want)
    finally:
        ka.finalize()
    d = ka.initialize(_keys(S, H, I, 4, 1, dt=dt))
    try:
        with pytest.raises(ka.KleosError) as ei:
            ka.moe.forward_host_dense(16, 16)
        assert ei.value.code == ka._capi.KLEOS_ESTATE
    finally:
        ka.finalize()


# ------------------------------------------------------------------ back-to-back launches
@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
def test_experts_that_fill_a_tile_to_every_quarter(mode):
    """256-row tiles (the variant for experts of 129 to 1023 rows) whose experts hold 12, 62, 81, 147, 220
    and 256 + 64 rows: the wavefronts of a tile own 64 rows each, and those whose rows do not exist leave
    the arithmetic of the tile out. A constant input feature times a per-expert gate weight skews the
    routing; the two hottest experts overflow their capacity of 512."""
    keys = _keys(1024, 128, 256, 8, 2, cf=2.0)
    c = moe_ref.cfg_from_keys(keys)
    assert c.EC == 512
    x, wg, w_up, w_down, *_ = random_layer(c, seed=77, w_std=0.08)
    x[:, 0] = 4.0
    wg[:, 0] = np.array([1.2, 0.9, 0.6, 0.3, 0.1, -0.1, -0.4, -0.9], np.float32) * 0.3
    iP = pack_inputs(c, x, wg, w_up, w_down)
    d, v, moe_out, err = check_against_oracle(c, keys, iP, mode)
    kept = np.minimum(v["expert_count"].astype(np.int64), c.EC) % 256
    quarters = {int((r - 1) // 64) for r in kept if r}
    assert quarters == {0, 1, 2, 3}, sorted(kept)
    assert (v["topk_slot"] < 0).sum() > 0


def _one_hot_layer(c, rows, seed):
    """A layer whose token t goes to one chosen expert (k = 1): `rows[e]` tokens to expert e, the rest to
    the last expert; one-hot input features that the gate weights pick up decide it."""
    x, wg, w_up, w_down, b_up, b_down = random_layer(c, seed=seed, w_std=0.08, bias_std=0.1)
    E = c.E
    first = np.repeat(np.arange(E), rows)
    assert first.size == c.S
    np.random.default_rng(seed).shuffle(first)
    x[:, :E] = 0.0
    x[np.arange(c.S), first] = 8.0
    wg[:, :E] = np.eye(E, dtype=np.float32)
    wg[:, E:] *= 0.25
    return pack_inputs(c, x, wg, w_up, w_down, b_up, b_down)


@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
@pytest.mark.parametrize("variant", ["256-row tiles", "128-row tiles"])
def test_experts_that_end_inside_and_at_the_edges_of_16_row_blocks(mode, variant):
    """A wavefront computes only the blocks of 16 rows that hold rows of its tile (four versions of the
    main loop, for 1 to 4 blocks of its 64 rows). Experts of 1, 15, 16, 17, 31, 33, 47, 48, 49, 63, 64, 65,
    ... rows put the last row at the start, inside and at the end of every such block, in the 256-row
    tile (capacity 256) and in the 128-row tile (capacity 128)."""
    if variant == "256-row tiles":
        rows = [1, 15, 16, 17, 31, 33, 47, 48, 49, 63, 64, 65, 100, 129, 200, 255]
        S, E = 2048, 32
        rows = rows + [17] * 15
        rows.append(S - sum(rows))                   # the last expert takes the rest (and overflows its capacity)
        keys = _keys(S, 128, 256, E, 1, cf=4.0)      # EC = 256
    else:
        rows = [1, 15, 16, 17, 31, 33, 47, 48, 49, 63, 64, 65, 79, 81, 100, 127]
        S, E = 1024, 32
        rows = rows + [9] * 15
        rows.append(S - sum(rows))
        keys = _keys(S, 128, 256, E, 1, cf=4.0)      # EC = 128
    c = moe_ref.cfg_from_keys(keys)
    assert c.EC == (256 if variant == "256-row tiles" else 128)
    iP = _one_hot_layer(c, rows, seed=97)
    d, v, moe_out, err = check_against_oracle(c, keys, iP, mode)
    np.testing.assert_array_equal(v["expert_count"], np.array(rows))
    assert (v["topk_slot"] < 0).sum() == max(0, rows[-1] - c.EC)      # only the last expert can drop tokens


@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
def test_back_to_back_launches_need_no_host_reset(mode):
    """The reference resets its state inside the kernel (moe.cuh:31-70) so launches can follow each
    other; here the same must hold for counters and the double-buffered histograms. Five launches,
    then the usual parity check on the last one, and bitwise equality with a single launch."""
    keys = _keys(512, 128, 256, 16, 2)
    c = moe_ref.cfg_from_keys(keys)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=8, w_std=0.08)
    iP = pack_inputs(c, x, wg, w_up, w_down)
    _, v5, out5, _ = check_against_oracle(c, keys, iP, mode, launches=5)
    _, v1, out1, _ = check_against_oracle(c, keys, iP, mode, launches=1)
    np.testing.assert_array_equal(out5, out1)
    np.testing.assert_array_equal(v5["topk_slot"], v1["topk_slot"])


@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
def test_new_inputs_in_the_same_context(mode):
    """Routing tables, h1 and y of one launch must not leak into the next: three different batches
    (different routing, different drops) run through one context, each checked against the oracle.
    Every table that crosses workgroups is rewritten by other CUs and XCDs than the ones that read
    it last time, which is what a stale cache line would show up in."""
    keys = _keys(1024, 128, 256, 24, 2)
    c = moe_ref.cfg_from_keys(keys)
    d = ka.initialize(keys)
    try:
        _apply(mode)
        oP = synth.alloc_outputs(d)
        for seed in (21, 22, 23):
            x, wg, w_up, w_down, *_ = random_layer(c, seed=seed, w_std=0.3 if seed == 22 else 0.08)
            iP_np = pack_inputs(c, x, wg, w_up, w_down)
            iP = _to_device(c, iP_np)
            oP.fill_(float("nan"))
            torch.cuda.synchronize()
            ka.moe.forward_host(iP, oP)
            ka.moe.forward_host(iP, oP)
            ka.moe.stream_synchronize()
            v = ka.moe.debug_views(d)
            ref = moe_ref.forward(c, iP_np, logits=v["logits"])
            for name in ("topk_expert", "topk_slot", "expert_count"):
                np.testing.assert_array_equal(v[name], ref[name], err_msg=f"{name}, seed {seed}")
            out = moe_ref.elems_to_f32(_out_to_np(c, oP), c)
            assert np.isfinite(out).all()
            moe_out = out[c.S * c.PX:].reshape(c.S, c.H)
            assert rel_fro(moe_out, ref["moe_out"]) < TOL_OUT[c.dtype], f"seed {seed}"
    finally:
        ka.finalize()


def test_timing_interfaces_of_the_persistent_launch():
    """kleos_phase_times, kleos_scheduler_stats and kleos_phase_stamps after a fused bench run: the
    stamps are monotonic per workgroup, every expert tile is counted once, phases add up to less
    than the event-timed launch."""
    keys = _keys(2048, 512, 512, 16, 2)
    c = moe_ref.cfg_from_keys(keys)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=31, w_std=0.05)
    iP = _to_device(c, pack_inputs(c, x, wg, w_up, w_down))
    d = ka.initialize(keys)
    try:
        ka.moe.set_mode(ka.MODE_FUSED)
        oP = synth.alloc_outputs(d)
        ms = ka.moe.forward_host_bench(iP, oP, skip=2, trials=4)
        ph = ka.moe.phase_times()
        st = ka.moe.scheduler_stats()
        stamps = ka.moe.phase_stamps()
        v = ka.moe.debug_views(d)
    finally:
        ka.finalize()
    assert ms > 0 and all(t >= 0 for t in ph.values())
    assert sum(ph.values()) <= ms * 1.5 + 0.05
    assert stamps.shape[1] == 8 and stamps.shape[0] >= 1
    assert (np.diff(stamps.astype(np.int64), axis=1) >= 0).all()
    kept = np.minimum(v["expert_count"].astype(np.int64), d.kept_capacity)
    row_blocks = -(-kept // 256)
    assert int(st["tiles"]) == int(row_blocks.sum()) * (-(-d.I // 256) + -(-d.H // 256))
    assert st["foreign_tiles"] <= st["tiles"]


def test_matrix_instruction_probe_runs_and_reports_a_rate():
    """kleos_debug_mfma_probe: both instructions, random and zero operands, give a positive duration
    and a rate below the published peak; bad arguments are refused."""
    for tile in (32, 16):
        for zero in (False, True):
            r = ka.moe.debug_mfma_probe(tile, iterations=2000, zero_operands=zero)
            assert r["ms"] > 0 and 100.0 < r["tflops"] < 2600.0, (tile, zero, r)
    with pytest.raises(ka.KleosError):
        ka.moe.debug_mfma_probe(8, 100)
    with pytest.raises(ka.KleosError):
        ka.moe.debug_mfma_probe(16, 0)


def test_cooperative_launch_gives_the_same_bits():
    """kleos_set_cooperative_launch(1): the runtime checks the grid's residency at every launch; the
    kernel and its results are the same."""
    keys = _keys(1024, 256, 256, 16, 2)
    c = moe_ref.cfg_from_keys(keys)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=10, w_std=0.06)
    iP = _to_device(c, pack_inputs(c, x, wg, w_up, w_down))
    _, plain, _ = run_gpu(keys, iP, ka.MODE_FUSED)
    d = ka.initialize(keys)
    try:
        ka.moe.set_cooperative_launch(True)
        oP = synth.alloc_outputs(d)
        for _ in range(3):
            ka.moe.forward_host(iP, oP)
        ka.moe.stream_synchronize()
        np.testing.assert_array_equal(_out_to_np(c, oP), _out_to_np(c, plain))
        ka.moe.set_cooperative_launch(False)
        ka.moe.forward_host(iP, oP)
        ka.moe.stream_synchronize()
        np.testing.assert_array_equal(_out_to_np(c, oP), _out_to_np(c, plain))
    finally:
        ka.finalize()


def test_fused_and_phased_agree_bitwise():
    keys = _keys(1024, 256, 256, 16, 2)
    c = moe_ref.cfg_from_keys(keys)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=9, w_std=0.06)
    iP_np = pack_inputs(c, x, wg, w_up, w_down)
    iP = _to_device(c, iP_np)
    outs = []
    for mode in MODES:
        d, oP, v = run_gpu(keys, iP, mode)
        outs.append((_out_to_np(c, oP), v))
    for other in outs[1:]:
        np.testing.assert_array_equal(outs[0][0], other[0])
        for name in ("logits", "topk_expert", "topk_slot", "expert_count"):
            np.testing.assert_array_equal(outs[0][1][name], other[1][name])


def test_schedule_of_the_persistent_launch():
    """KLEOS_SCHEDULE_AUTO takes the static schedule when striding through the XCD queues costs no
    extra round of tiles and the dynamic one when it would; a context that alternates between the two (the static schedule
    holds a grid barrier of its own, whose counters advance only with it) returns the same bits every
    time, and the same as separate launches per phase."""
    keys = _keys(8192, 128, 512, 8, 2, cf=8.0)
    c = moe_ref.cfg_from_keys(keys)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=51, w_std=0.05)
    balanced = _to_device(c, pack_inputs(c, x, wg, w_up, w_down))
    # every token to experts 0 and 1, nothing dropped: two XCD queues hold 64 tiles each per
    # projection, two rounds for their XCDs' 32 workgroups, one round if the grid shares them
    wg2 = np.zeros_like(wg)
    wg2[0, :] = 1.0
    wg2[1, :] = 0.5
    skewed = _to_device(c, pack_inputs(c, np.abs(x), wg2, w_up, w_down))
    _, ref_b, _ = run_gpu(keys, balanced, ka.MODE_PHASED)
    _, ref_s, _ = run_gpu(keys, skewed, ka.MODE_PHASED)
    ref_b, ref_s = _out_to_np(c, ref_b), _out_to_np(c, ref_s)
    d = ka.initialize(keys)
    try:
        ka.moe.set_mode(ka.MODE_FUSED)
        assert ka._capi.lib().kleos_get_schedule() == ka.SCHEDULE_AUTO
        with pytest.raises(ka.KleosError):
            ka.moe.set_schedule(7)
        oP = synth.alloc_outputs(d)
        plan = [(ka.SCHEDULE_AUTO, balanced, ref_b, ka.SCHEDULE_STATIC),
                (ka.SCHEDULE_AUTO, skewed, ref_s, ka.SCHEDULE_DYNAMIC),
                (ka.SCHEDULE_AUTO, balanced, ref_b, ka.SCHEDULE_STATIC),
                (ka.SCHEDULE_DYNAMIC, balanced, ref_b, ka.SCHEDULE_DYNAMIC),
                (ka.SCHEDULE_STATIC, skewed, ref_s, ka.SCHEDULE_STATIC),
                (ka.SCHEDULE_DYNAMIC, skewed, ref_s, ka.SCHEDULE_DYNAMIC),
                (ka.SCHEDULE_STATIC, balanced, ref_b, ka.SCHEDULE_STATIC),
                (ka.SCHEDULE_STATIC, balanced, ref_b, ka.SCHEDULE_STATIC)]
        for step, (schedule, iP, ref, taken) in enumerate(plan):
            ka.moe.set_schedule(schedule)
            oP.fill_(float("nan"))
            torch.cuda.synchronize()
            ka.moe.forward_host(iP, oP)
            assert ka.moe.schedule_taken() == taken, f"step {step}"
            np.testing.assert_array_equal(_out_to_np(c, oP), ref, err_msg=f"step {step}")
    finally:
        ka.finalize()


# ------------------------------------------------------------------ benchmark-sized configurations
def _full_size(name, mode, n_check, seed=0):
    """Full-size run; the oracle evaluates expert FFNs for a sample of tokens only (its gate and
    routing are always complete)."""
    w = synth.WORKLOADS[name]
    iP, d = synth.make_inputs(w, seed=seed, device="cuda")
    c = moe_ref.cfg_from_keys(w.config)
    iP_np = _out_to_np(c, iP)
    rng = np.random.default_rng(seed)
    mask = np.zeros(c.S, np.uint8)
    mask[rng.choice(c.S, size=n_check, replace=False)] = 1
    return c, w, iP_np, mask


@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
def test_balanced_e16_full_size(mode):
    """S=4096 H=I=2048 E=16 top-2 bf16, balanced load."""
    c, w, iP_np, mask = _full_size("balanced_e16", mode, 256)
    d, v, moe_out, err = check_against_oracle(c, w.config, iP_np, mode, token_mask=mask)
    counts = v["expert_count"].astype(np.int64)
    assert counts.sum() == c.S * c.k and counts.max() < 1.3 * counts.mean()


@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
def test_headline_e64_zipf_full_size(mode):
    """S=8192 H=I=2048 E=64 top-2 bf16 with the Zipf logit bias: the hottest expert is routed about
    four times the mean load, so tokens are dropped and the scheduler sees unequal experts."""
    c, w, iP_np, mask = _full_size("headline_e64_zipf", mode, 384)
    # make sure dropped and kept tokens of the hottest expert are both in the sample
    d, v, moe_out, err = check_against_oracle(c, w.config, iP_np, mode, token_mask=mask)
    counts = v["expert_count"].astype(np.int64)
    mean = c.S * c.k / c.E
    assert 3.5 * mean < counts.max() < 4.6 * mean, counts.max() / mean
    assert (v["topk_slot"] < 0).sum() > 0
    assert (np.minimum(counts, c.EC).sum()) == (v["topk_slot"] >= 0).sum()


@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
def test_mixtral_e8_full_size(mode):
    """S=8192 H=4096 I=14336 E=8 top-2 cf=1.25 bf16: large, compute-bound expert GEMMs with several
    row blocks per expert; the oracle evaluates a sample of the tokens."""
    c, w, iP_np, mask = _full_size("mixtral_e8", mode, 48)
    d, v, moe_out, err = check_against_oracle(c, w.config, iP_np, mode, token_mask=mask)
    assert v["expert_count"].astype(np.int64).sum() == c.S * c.k


@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
def test_fine_e256_top8_full_size(mode):
    """S=4096 H=7168 I=2048 E=256 top-8 bf16: many small experts, dispatch / combine / scheduler
    dominated."""
    c, w, iP_np, mask = _full_size("fine_e256_top8", mode, 48)
    d, v, moe_out, err = check_against_oracle(c, w.config, iP_np, mode, token_mask=mask)
    assert v["expert_count"].astype(np.int64).sum() == c.S * c.k


@pytest.mark.parametrize("mode", MODES, ids=MODE_IDS)
def test_forced_full_row_blocks_at_reduced_width(mode):
    """The recipe of the mixtral_full_blocks workload (top-1, every expert routed exactly the rows of
    its capacity, all row blocks full) on narrower projections: 8 experts x 1 024 rows, so the 256-row
    tiles of the variant for large experts, no ragged block, nothing dropped."""
    full = synth.WORKLOADS["mixtral_full_blocks"]
    w = synth.Workload("full_blocks_small", synth._cfg(8192, 512, 1024, 8, 1, 1.0, 2), full.x_std, 0.03,
                       forced_rows=(1024,) * 8)
    iP, d = synth.make_inputs(w, seed=5, device="cuda")
    c = moe_ref.cfg_from_keys(w.config)
    assert c.EC == 1024
    mask = np.zeros(c.S, np.uint8)
    mask[np.random.default_rng(5).choice(c.S, size=256, replace=False)] = 1
    d, v, moe_out, err = check_against_oracle(c, w.config, _out_to_np(c, iP), mode, token_mask=mask)
    np.testing.assert_array_equal(v["expert_count"], np.full(8, 1024))
    assert (v["topk_slot"] >= 0).all()


@pytest.mark.parametrize("name,schedule", [("headline_e64_zipf", ka.SCHEDULE_STATIC), ("headline_e64_zipf", ka.SCHEDULE_DYNAMIC),
                                           ("balanced_e16", ka.SCHEDULE_AUTO), ("fine_e256_top8", ka.SCHEDULE_AUTO)],
                         ids=["headline-static", "headline-dynamic", "balanced_e16", "fine_e256_top8"])
def test_full_size_batches_alternate_in_one_context(name, schedule):
    """Inside the persistent launch the routing tables, the slot tables, h1 and y pass between
    workgroups on different XCDs, whose L2 caches are not coherent: a reader that got a line as an
    earlier launch left it would compute with the other batch's data. Two full-size batches with
    different routing alternate through one context, every CU busy; each output must equal, bit for
    bit, what the same batch gives launch by launch (phased mode, where kernel boundaries do the
    synchronisation)."""
    w = synth.WORKLOADS[name]
    c = moe_ref.cfg_from_keys(w.config)
    batches = [synth.make_inputs(w, seed=seed, device="cuda")[0] for seed in (0, 1)]
    refs = []
    for iP in batches:
        _, oP, v = run_gpu(w.config, iP, (ka.MODE_PHASED, ka.SCHEDULE_AUTO))
        refs.append((_out_to_np(c, oP), v["topk_slot"].copy(), v["slot_token"].copy()))
        del oP
    assert not np.array_equal(refs[0][1], refs[1][1])
    d = ka.initialize(w.config)
    try:
        _apply((ka.MODE_FUSED, schedule))
        oP = synth.alloc_outputs(d)
        for step, b in enumerate((0, 1, 1, 0, 1, 0)):
            oP.fill_(float("nan"))
            torch.cuda.synchronize()
            ka.moe.forward_host(batches[b], oP)
            ka.moe.stream_synchronize()
            v = ka.moe.debug_views(d)
            np.testing.assert_array_equal(v["topk_slot"], refs[b][1], err_msg=f"step {step}")
            np.testing.assert_array_equal(_out_to_np(c, oP), refs[b][0], err_msg=f"step {step}")
    finally:
        ka.finalize()


# ------------------------------------------------------------------ training mode
@pytest.mark.parametrize("E,k,S", [(16, 2, 1024), (64, 2, 2048), (130, 8, 512), (384, 4, 512)])
def test_training_mode_gate_loss(E, k, S):
    """is_training: 1 adds the load-balancing loss of the gate (gate.cuh:608-635, 700-705, 763-773):
    checked against the oracle evaluated on the GPU's own logits, identical in both modes (every
    sum has a fixed order), and the forward itself is unchanged."""
    keys = _keys(S, 128, 128, E, k)
    keys.is_training = 1
    c = moe_ref.cfg_from_keys(keys)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=41, w_std=0.25)
    iP_np = pack_inputs(c, x, wg, w_up, w_down)
    iP = _to_device(c, iP_np)
    got = {}
    for mode in MODES:
        d = ka.initialize(keys)
        try:
            _apply(mode)
            oP = synth.alloc_outputs(d)
            ka.moe.forward_host(iP, oP)
            ka.moe.forward_host(iP, oP)
            ka.moe.stream_synchronize()
            got[mode] = (ka.moe.gate_loss(d.E), ka.moe.debug_views(d), _out_to_np(c, oP))
        finally:
            ka.finalize()
    g, v, out = got[MODES[1]]
    r = moe_ref.route(c, v["logits"])
    np.testing.assert_array_equal(v["expert_count"], r["expert_count"])
    ref = moe_ref.gate_loss(c, r["probs"], r["expert_count"])
    assert abs(g["loss"] - ref["loss"]) < 2e-5 * ref["loss"] + 1e-9, (g["loss"], ref["loss"])
    np.testing.assert_allclose(g["mean_prob"], ref["mean_prob"], rtol=2e-5, atol=1e-8)
    np.testing.assert_allclose(g["mean_count"], ref["mean_count"], rtol=1e-6, atol=0)
    for other in (MODES[0], MODES[2]):
        gp, vp, outp = got[other]
        assert gp["loss"] == g["loss"]
        np.testing.assert_array_equal(gp["mean_prob"], g["mean_prob"])
        np.testing.assert_array_equal(outp, out)


def test_configurations_this_build_leaves_out_are_refused():
    for keys in (_keys(256, 128, 64, 576, 2), _keys(256, 128, 64, 320, 40)):
        with pytest.raises(ka.KleosError) as ei:
            ka.initialize(keys)
        assert ei.value.code == ka._capi.KLEOS_EUNSUPPORTED
        assert not ka.is_initialized()


def test_gate_loss_needs_training_mode():
    keys = _keys(256, 128, 128, 8, 2)
    d = ka.initialize(keys)
    try:
        with pytest.raises(ka.KleosError):
            ka.moe.gate_loss(d.E)
    finally:
        ka.finalize()


# ------------------------------------------------------------------ the reference's driver, on this library
@pytest.mark.parametrize("dt", [2, 3, 0, 1], ids=["bf16", "fp16", "fp32", "tf32"])
def test_cpp_driver_prints_the_reference_line(tmp_path, dt):
    """csrc/kleos_main is the equivalent of the reference's runOS() (csrc/main.cu:13-73): it reads a
    kleos_config.json, fills the packed buffers on the host, converts them to Element (main.cu:59-62),
    runs forwardHostBench<32,32> through kleos.hpp and prints `epRank: 0 took X ms`. With
    KLEOS_MAIN_CHECK set it also reports how many output Elements are not finite: inputs converted
    to the wrong 16-bit format (N(0, 5) values read as the other format) overflow at once."""
    import re
    import subprocess
    from aristos_amd import build
    if not os.path.exists(build.DRIVER_PATH):
        pytest.skip("the C++ driver is not built")
    cfg = tmp_path / "kleos_config.json"
    cfg.write_text(_keys(512, 128, 128, 16, 2, dt=dt).to_json_text())
    r = subprocess.run([build.DRIVER_PATH, str(cfg)], capture_output=True, text=True, timeout=120,
                       env={**os.environ, "KLEOS_MAIN_CHECK": "1"})
    assert r.returncode == 0, r.stderr
    m = re.search(r"epRank: 0 took ([0-9.]+)\s*ms", r.stdout)
    assert m and float(m.group(1)) > 0, r.stdout
    m = re.search(r"device x: mean (\S+) std (\S+) max relative conversion error (\S+)", r.stdout)
    assert m, r.stdout
    assert abs(float(m.group(1))) < 0.1 and abs(float(m.group(2)) - 5.0) < 0.1
    assert float(m.group(3)) <= {2: 2.0 ** -8, 3: 2.0 ** -10, 0: 0.0, 1: 2.0 ** -11}[dt]


def _bytes_3c_value(dt):
    """The value of an Element whose bytes are all 0x3c."""
    if dt == 0:
        return float(np.frombuffer(b"\x3c" * 4, np.float32)[0])
    bits = np.array([0x3c3c], np.uint16)
    return float(bits.view(np.float16)[0]) if dt == 3 else float(moe_ref.bf16_bits_to_f32(bits)[0])


@pytest.mark.parametrize("dt,act,S,H,I,E", [(2, 0, 2048, 2048, 2048, 16), (2, 1, 1024, 256, 512, 8),
                                            (3, 0, 1024, 128, 256, 8), (0, 1, 512, 128, 192, 4),
                                            (2, 0, 8192, 256, 512, 2)])
def test_throughput_probe_result(dt, act, S, H, I, E):
    """The probe's operands are all one value v (every byte 0x3c), so every element of its result is
    Element(I * Element(act(H v^2 + v)) * v + v), with the rounding points of the expert FFN
    (processor.cuh:475, gemm.cuh:22-31). A wrong grid, a wrong capacity or a skipped tile of the
    probe's E = 1, S = pEC launch leaves elements that differ."""
    import math
    keys = _keys(S, H, I, E, 2, act=act, dt=dt)
    c = moe_ref.cfg_from_keys(keys)
    d = ka.initialize(keys)
    try:
        r = ka.moe.measure_throughput_output(d, trials=3)
    finally:
        ka.finalize()
    assert r["median_ms"] > 0 and r["y"].shape == (d.pEC, H)
    v = _bytes_3c_value(dt)
    pre = H * v * v + v
    h1 = 0.5 * pre * (1.0 + math.erf(pre / math.sqrt(2.0))) if act == 1 else max(pre, 0.0)
    def to_elem(val):
        a = np.array([val], np.float32)
        if dt == 0:
            return float(a[0])
        if dt == 3:
            return float(a.astype(np.float16)[0])
        return float(moe_ref.bf16_bits_to_f32(moe_ref.f32_to_bf16_bits(a))[0])
    expect = to_elem(I * to_elem(h1) * v + v)
    got = moe_ref.elems_to_f32(r["y"].ravel(), c).reshape(d.pEC, H)
    # fp32 accumulation of equal terms in the matrix core's order against one multiplication: far
    # below one rounding step of a 16-bit Element, a few ulp in fp32
    tol = {0: 2e-6, 2: 2.0 ** -8, 3: 2.0 ** -11}[dt] * abs(expect)
    assert np.isfinite(got).all()
    assert np.abs(got - expect).max() <= tol, (expect, got.min(), got.max())


def test_throughput_probe_leaves_the_context_alone():
    """kleos_measure_throughput (the reference's mT, throughput.cuh:104-170) times one expert at
    padded capacity on its own buffers; a forward before and after it gives the same bits."""
    keys = _keys(1024, 256, 512, 8, 2)
    c = moe_ref.cfg_from_keys(keys)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=51, w_std=0.05)
    iP = _to_device(c, pack_inputs(c, x, wg, w_up, w_down))
    d = ka.initialize(keys)
    try:
        oP = synth.alloc_outputs(d)
        ka.moe.forward_host(iP, oP)
        ka.moe.stream_synchronize()
        before = _out_to_np(c, oP).copy()
        r = ka.moe.measure_throughput(8)
        assert r["median_ms"] > 0 and abs(r["throughput"] * r["median_ms"] - 1.0) < 1e-5
        oP.fill_(float("nan"))
        ka.moe.forward_host(iP, oP)
        ka.moe.stream_synchronize()
        np.testing.assert_array_equal(_out_to_np(c, oP), before)
    finally:
        ka.finalize()


# ------------------------------------------------------------------ failure handling
@pytest.mark.parametrize("schedule", [ka.SCHEDULE_DYNAMIC, ka.SCHEDULE_STATIC], ids=["dynamic", "static"])
def test_context_recovers_after_an_expired_wait(schedule):
    """A persistent launch whose grid barriers can never be satisfied (the host counts a launch that
    never ran, so the monotonic arrival counters lag their targets) runs into the wait limit at every
    barrier, drains, and is reported by the next synchronising call. The library then resets its
    scheduler state: later forwards on the same context are bit-identical to a fresh context's.
    The limit is lowered to 0.2 ms first; every kernel exits normally."""
    keys = _keys(1024, 256, 256, 16, 2)
    c = moe_ref.cfg_from_keys(keys)
    x, wg, w_up, w_down, *_ = random_layer(c, seed=61, w_std=0.06)
    iP = _to_device(c, pack_inputs(c, x, wg, w_up, w_down))
    _, fresh, vf = run_gpu(keys, iP, (ka.MODE_FUSED, schedule))
    fresh = _out_to_np(c, fresh)
    d = ka.initialize(keys)
    try:
        _apply((ka.MODE_FUSED, schedule))
        oP = synth.alloc_outputs(d)
        ka.moe.forward_host(iP, oP)
        ka.moe.forward_host(iP, oP)
        ka.moe.stream_synchronize()
        np.testing.assert_array_equal(_out_to_np(c, oP), fresh)
        ka.moe.debug_set_wait_ticks(20000)          # 0.2 ms
        ka.moe.debug_skip_launch_number()
        ka.moe.forward_host(iP, oP)
        with pytest.raises(ka.KleosError) as ei:
            ka.moe.stream_synchronize()
        assert ei.value.code == ka._capi.KLEOS_EHIP and "expired" in ei.value.message
        ka.moe.debug_set_wait_ticks(0)
        for _ in range(3):
            oP.fill_(float("nan"))
            torch.cuda.synchronize()
            ka.moe.forward_host(iP, oP)
            ka.moe.stream_synchronize()
            np.testing.assert_array_equal(_out_to_np(c, oP), fresh)
        v = ka.moe.debug_views(d)
        np.testing.assert_array_equal(v["topk_slot"], vf["topk_slot"])
    finally:
        ka.finalize()
