"""Run-time configuration: same keys, enumerations and checks as the reference's compile-time
configuration (csrc/kleos_config.schema.json, csrc/include/kleos/types.cuh:471-507,
csrc/include/kleos/bootstrap.cuh:542-545)."""
import json
import os

import pytest

import aristos_amd as ka
from aristos_amd import _capi, synth

CONFIG_DIR = os.path.join(os.path.dirname(ka.__file__), "configs")

# the reference's shipped csrc/kleos_config.json, restated key by key
SHIPPED = {"capacity_factor": 1, "drop_tokens": 1, "expert_top_k": 2, "global_batch": 256, "is_training": 0,
           "hidden_act": 0, "hidden_size": 2048, "intermediate_size": 2048, "mini_batch": 1, "moe_frequency": 1,
           "num_experts": 64, "num_layers": 1, "sequence_len": 8192, "torch_dtype": 1, "vocab_size": 32000}


def test_parse_shipped_config_keys():
    cfg = ka.KleosConfig.from_json_text(json.dumps(SHIPPED))
    assert cfg.num_experts == 64 and cfg.expert_top_k == 2 and cfg.sequence_len == 8192
    assert cfg.torch_dtype == 1 and cfg.capacity_factor == 1.0
    # the shipped dtype is tf32: Elements of 32 bits, the derived constants of the headline layer
    d = cfg.derive()
    assert (d.S, d.H, d.I, d.E, d.k, d.EC, d.PX, d.elem_bytes) == (8192, 2048, 2048, 64, 2, 256, 64, 4)
    assert d.in_elems == 8192 * 2048 + 64 * 2048 + 2 * 64 * 2048 * 2048 + 64 * 4096


@pytest.mark.parametrize("name,S,PX,EC,pEC,in_elems", [
    ("tiny_fp32", 128, 64, 32, 128, 128 * 256 + 64 * 256 + 2 * 8 * 512 * 256 + 8 * (512 + 256)),
    ("balanced_e16", 4096, 64, 512, 512, 4096 * 2048 + 64 * 2048 + 2 * 16 * 2048 * 2048 + 16 * 4096),
    ("headline_e64_zipf", 8192, 64, 256, 256, 8192 * 2048 + 64 * 2048 + 2 * 64 * 2048 * 2048 + 64 * 4096),
    ("mixtral_e8", 8192, 64, 2560, 2560, 8192 * 4096 + 64 * 4096 + 2 * 8 * 14336 * 4096 + 8 * (14336 + 4096)),
    ("fine_e256_top8", 4096, 256, 128, 128, 4096 * 7168 + 256 * 7168 + 2 * 256 * 2048 * 7168 + 256 * (2048 + 7168)),
    ("mixtral_full_blocks", 16384, 64, 2048, 2048, 16384 * 4096 + 64 * 4096 + 2 * 8 * 14336 * 4096 + 8 * (14336 + 4096)),
])
def test_workload_configs_derive_the_reference_constants(name, S, PX, EC, pEC, in_elems):
    cfg = ka.KleosConfig.from_json_file(os.path.join(CONFIG_DIR, name + ".json"))
    assert cfg == synth.WORKLOADS[name].config
    d = cfg.derive()
    assert (d.S, d.PX, d.EC, d.pEC) == (S, PX, EC, pEC)
    assert d.in_elems == in_elems                       # main.cu:23-28
    assert d.out_elems == S * PX + S * d.H              # main.cu:29-30
    assert d.off_gate_w == S * d.H and d.off_w_up == d.off_gate_w + PX * d.H
    assert d.off_w_down == d.off_w_up + d.E * d.I * d.H and d.off_b_up == d.off_w_down + d.E * d.I * d.H
    assert d.off_b_down == d.off_b_up + d.E * d.I and d.off_moe_out == S * PX
    assert d.elem_bytes == (4 if cfg.torch_dtype == 0 else 2)


def test_integer_capacity_factor_matches_reference_formula():
    for cf in (1, 2, 3):
        for S, E, k in ((8192, 64, 2), (384, 5, 3), (128, 8, 1)):
            d = ka.KleosConfig(capacity_factor=cf, sequence_len=S, num_experts=E, expert_top_k=k).derive()
            assert d.EC == -(-S // E) * cf * k            # types.cuh:498-499


@pytest.mark.parametrize("override,code,needle", [
    ({"sequence_len": 100}, _capi.KLEOS_EINVAL, "multiple of 128"),
    ({"hidden_size": 100}, _capi.KLEOS_EINVAL, "hidden_size"),
    ({"intermediate_size": 96}, _capi.KLEOS_EINVAL, "intermediate_size"),
    ({"expert_top_k": 65}, _capi.KLEOS_EINVAL, "expert_top_k"),
    ({"num_experts": 70000, "expert_top_k": 2}, _capi.KLEOS_EINVAL, "65535"),
    ({"capacity_factor": 0.5}, _capi.KLEOS_EINVAL, "capacity_factor"),
    ({"hidden_act": 2}, _capi.KLEOS_EINVAL, "hidden_act"),
    ({"drop_tokens": 2}, _capi.KLEOS_EINVAL, "drop_tokens"),
])
def test_invalid_configs_are_rejected_with_a_message(override, code, needle):
    with pytest.raises(ka.KleosError) as ei:
        ka.KleosConfig(**override).derive()
    assert ei.value.code == code and needle in ei.value.message


@pytest.mark.parametrize("text,needle", [
    ("", "expected '{'"),
    ('{"capacity_factor": 1', "expected ','"),
    ('{"capacity_factor": "one"}', "numeric"),
    (json.dumps({k: v for k, v in SHIPPED.items() if k != "num_experts"}), "num_experts"),
    (json.dumps(SHIPPED) + "x", "trailing"),
    ('{"capacity_factor": 1, "capacity_factor": 2}', "twice"),
    (json.dumps({**SHIPPED, "num_experts": -4}), "non-negative integer"),
    (json.dumps({**SHIPPED, "num_experts": 2.5}), "non-negative integer"),
])
def test_malformed_json_is_rejected(text, needle):
    with pytest.raises(ka.KleosError) as ei:
        ka.KleosConfig.from_json_text(text)
    assert ei.value.code == _capi.KLEOS_EPARSE and needle in ei.value.message


def test_global_batch_is_optional_and_unknown_keys_are_ignored():
    d = {k: v for k, v in SHIPPED.items() if k != "global_batch"}
    d["some_future_key"] = 7
    cfg = ka.KleosConfig.from_json_text(json.dumps(d))
    assert cfg.global_batch == 0 and cfg.num_experts == 64


def test_missing_file_reports_io_error(tmp_path):
    with pytest.raises(ka.KleosError) as ei:
        ka.KleosConfig.from_json_file(str(tmp_path / "nope.json"))
    assert ei.value.code == _capi.KLEOS_EIO


def test_json_round_trip(tmp_path):
    cfg = synth.WORKLOADS["mixtral_e8"].config
    p = tmp_path / "c.json"
    p.write_text(cfg.to_json_text())
    assert ka.KleosConfig.from_json_file(str(p)) == cfg


def test_single_expert_keeps_the_packed_moe_layout():
    """E == 1 runs the dense FFN on the layout the reference's driver packs for every expert count
    (csrc/main.cu:23-30: a 64-row gate-weight block after x, a 64-column gateOut block before the
    result), not on the A | B1 | B2 | D1 | D2 -> C layout of the reference's fffn kernel
    (csrc/include/kleos/moe/fffn.cuh:43-49). The offsets a caller needs are pinned here."""
    S, H, I = 256, 128, 192
    d = ka.KleosConfig(sequence_len=S, hidden_size=H, intermediate_size=I, num_experts=1, expert_top_k=1).derive()
    assert (d.E, d.PX, d.k) == (1, 64, 1)
    assert d.off_x == 0 and d.off_gate_w == S * H
    assert d.off_w_up == S * H + 64 * H              # fffn would put B1 at S * H
    assert d.off_w_down == d.off_w_up + I * H
    assert d.off_b_up == d.off_w_down + H * I and d.off_b_down == d.off_b_up + I
    assert d.in_elems == S * H + 64 * H + 2 * I * H + I + H
    assert d.off_gate_out == 0 and d.off_moe_out == S * 64   # fffn would put C at 0
    assert d.out_elems == S * 64 + S * H
