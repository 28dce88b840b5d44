"""HTR-W1 checkpoint reader (docs/FORMAT.md:25-36 of the reference): round trip through safetensors, config table, fused rules."""
import json
import os

import pytest
import torch

from htr_amd import checkpoint, wire


def _mk(tmp_path, overlay=False):
    q = wire.synth_linear(256, 128, 4, 1)
    k = list(wire.synth_linear(128, 128, 4, 2)); k[2] = q[2]
    v = list(wire.synth_linear(128, 128, 4, 3)); v[2] = q[2]
    o = wire.synth_linear(128, 256, 3, 4)
    lin = {"model.layers.0.self_attn.q_proj": q, "model.layers.0.self_attn.k_proj": tuple(k),
           "model.layers.0.self_attn.v_proj": tuple(v), "model.layers.0.self_attn.o_proj": o}
    checkpoint.save_linears(str(tmp_path / "model-00001-of-00001.safetensors"), lin)
    table = {"wire": "HTR-W1", "generator": "rdna24", "L": 16, "tile": 16, "rht_block": 128,
             "modules": {p: {"K": wire.bits_of(t[0])} for p, t in lin.items()}}
    qc = {"quant_method": "quark", "htr_overlay": table} if overlay else dict(quant_method="htr", **table)
    json.dump({"quantization_config": qc}, open(tmp_path / "config.json", "w"))
    return lin


@pytest.mark.parametrize("overlay", [False, True])
def test_round_trip_and_fused(tmp_path, overlay):
    lin = _mk(tmp_path, overlay)
    ck = checkpoint.Checkpoint(str(tmp_path))
    assert ck.prefixes() == sorted(lin)
    assert ck.modules["model.layers.0.self_attn.o_proj"] == 3
    for p, want in lin.items():
        got = ck.linear(p)
        assert all(torch.equal(a, b) for a, b in zip(got, want))
    base = "model.layers.0.self_attn."
    qw, sc, su, sv = ck.fused([base + "q_proj", base + "k_proj", base + "v_proj"])
    assert wire.check_shapes(qw, sc, su, sv) == (512, 128, 4)
    assert torch.equal(qw[16:24], lin[base + "k_proj"][0]) and torch.equal(sv[32:48], lin[base + "k_proj"][3])
    with pytest.raises(ValueError):
        ck.fused([base + "q_proj", base + "o_proj"])                    # different K (and input width)
    with pytest.raises(KeyError):
        ck.linear("model.layers.1.mlp.down_proj")


def test_fused_parts_must_share_su(tmp_path):
    a = wire.synth_linear(128, 128, 4, 1)
    b = wire.synth_linear(128, 128, 4, 2)
    checkpoint.save_linears(str(tmp_path / "m.safetensors"), {"a": a, "b": b})
    ck = checkpoint.Checkpoint(str(tmp_path / "m.safetensors"))
    assert ck.modules is None and ck.prefixes() == ["a", "b"]
    with pytest.raises(ValueError):
        ck.fused(["a", "b"])


def test_config_validation(tmp_path):
    ok = {"quantization_config": {"quant_method": "htr", "wire": "HTR-W1", "modules": {"x": {"K": 5}}}}
    assert checkpoint.read_quantization_config(ok) == {"x": 5}
    for bad in ({"quantization_config": {"quant_method": "htr", "wire": "HTR-W2", "modules": {}}},
                {"quantization_config": {"quant_method": "htr", "generator": "other", "modules": {}}},
                {"quantization_config": {"quant_method": "htr", "modules": {"x": {"K": 9}}}},
                {"quantization_config": {"quant_method": "awq"}}, {}):
        with pytest.raises(ValueError):
            checkpoint.read_quantization_config(bad)
    lin = _mk(tmp_path)
    cfg = json.load(open(tmp_path / "config.json"))
    cfg["quantization_config"]["modules"]["model.layers.0.self_attn.o_proj"]["K"] = 4       # tensors say 3
    json.dump(cfg, open(tmp_path / "config.json", "w"))
    with pytest.raises(ValueError):
        checkpoint.Checkpoint(str(tmp_path)).linear("model.layers.0.self_attn.o_proj")


def test_save_checkpoint_writes_what_the_reader_and_the_plugin_expect(tmp_path):
    from htr_amd import vllm_plugin as vp
    lin = {"model.layers.0.mlp.gate_proj": wire.synth_linear(256, 128, 3, 1), "lm_head": wire.synth_linear(128, 128, 5, 2)}
    cfg = checkpoint.save_checkpoint(str(tmp_path / "ck"), lin, {"architectures": ["X"]})
    qc = cfg["quantization_config"]
    assert qc["quant_method"] == "htr" and qc["wire"] == "HTR-W1" and qc["generator"] == "rdna24"
    assert (qc["L"], qc["tile"], qc["rht_block"]) == (16, 16, 128) and cfg["architectures"] == ["X"]
    ck = checkpoint.Checkpoint(str(tmp_path / "ck"))
    assert ck.modules == {"model.layers.0.mlp.gate_proj": 3, "lm_head": 5}
    for p, want in lin.items():
        assert all(torch.equal(a, b) for a, b in zip(ck.linear(p), want))
    hc = vp.HTRConfig.from_config(qc)
    assert hc.modules == {"layers.0.mlp.gate_proj": 3, "lm_head": 5}
