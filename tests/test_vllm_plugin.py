"""Host logic of the vLLM plugin mirror (htr/vllm_plugin.py:21-150 of the reference), with stand-ins for vLLM's classes."""
import json
import os

import pytest
import torch

from htr_amd import vllm_plugin as vp


class _Linear(vp.LinearBase):
    pass


def test_canon_and_config():
    assert vp.canon("model.layers.3.mlp.down_proj.weight") == "layers.3.mlp.down_proj"
    assert vp.canon("lm_head.weight") == "lm_head"
    assert vp.canon("a.layers.1.b.layers.2.c") == "layers.2.c"
    cfg = vp.HTRConfig.from_config({"quant_method": "htr", "wire": "HTR-W1",
                                    "modules": {"model.layers.0.self_attn.q_proj": {"K": 4}, "lm_head": {"K": 3}}})
    assert cfg.get_name() == "htr" and cfg.get_min_capability() == 0 and cfg.get_config_filenames() == []
    assert cfg.get_supported_act_dtypes() == [torch.bfloat16, torch.float16]
    assert cfg.modules == {"layers.0.self_attn.q_proj": 4, "lm_head": 3}
    with pytest.raises(AssertionError):
        vp.HTRConfig({}, wire="HTR-W2")


def test_quant_method_selection():
    mods = {f"model.layers.0.self_attn.{p}_proj": {"K": 4} for p in "qkv"}
    mods.update({"model.layers.0.mlp.gate_proj": {"K": 3}, "model.layers.0.mlp.up_proj": {"K": 4}, "lm_head": {"K": 4}})
    cfg = vp.HTRConfig(mods)
    cfg.packed_modules_mapping = {"qkv_proj": ["q_proj", "k_proj", "v_proj"], "gate_up_proj": ["gate_proj", "up_proj"]}
    lin = _Linear()
    m = cfg.get_quant_method(lin, "model.layers.0.self_attn.qkv_proj")
    assert isinstance(m, vp.HTRLinearMethod) and m.K == 4
    with pytest.raises(ValueError):                                    # gate K3 / up K4
        cfg.get_quant_method(lin, "model.layers.0.mlp.gate_up_proj")
    assert isinstance(cfg.get_quant_method(lin, "model.layers.0.self_attn.o_proj"), vp.UnquantizedLinearMethod)
    assert isinstance(cfg.get_quant_method(lin, "visual.layers.0.self_attn.qkv_proj"), vp.UnquantizedLinearMethod)
    assert cfg.get_quant_method(torch.nn.Linear(2, 2), "model.layers.0.self_attn.qkv_proj") is None
    head = vp.ParallelLMHead()
    assert cfg.get_quant_method(head, "lm_head").K == 4
    assert cfg.get_quant_method(head, "model.embed_tokens") is None
    assert vp.HTRConfig({}).get_quant_method(head, "lm_head") is None


def test_shard_range():
    sizes = [4096, 1024, 1024]
    assert vp._shard_range(sizes, None, 16) == (0, 384)
    assert vp._shard_range(sizes, "q", 16) == (0, 256)
    assert vp._shard_range(sizes, "k", 1) == (4096, 1024)
    assert vp._shard_range(sizes, "v", 8) == (640, 128)
    assert vp._shard_range(sizes, (1, 2), 16) == (256, 128)
    assert vp._shard_range(sizes, 2, 16) == (320, 64)
    with pytest.raises(AssertionError):
        vp._shard_range(sizes, (0, 2), 16)
    with pytest.raises(AssertionError):
        vp._shard_range([100, 28], 1, 16)


def test_create_weights_and_loaders():
    from htr_amd import wire
    layer = _Linear()
    meth = vp.HTRLinearMethod(4)
    sizes = [256, 128, 128]
    meth.create_weights(layer, 256, sizes, 256, 512, torch.bfloat16)
    assert tuple(layer.htr_qweight.shape) == (32, 16, 32) and layer.htr_qweight.dtype == torch.int32
    assert tuple(layer.htr_scales.shape) == (512,) and layer.htr_scales.dtype == torch.float16
    assert tuple(layer.htr_su.shape) == (32,) and tuple(layer.htr_sv.shape) == (64,) and layer.htr_K == 4
    parts = {"q": wire.synth_linear(256, 256, 4, 1), "k": wire.synth_linear(128, 256, 4, 2), "v": wire.synth_linear(128, 256, 4, 3)}
    su = parts["q"][2]
    for sid, (qw, sc, _, sv) in parts.items():
        layer.htr_qweight.weight_loader(layer.htr_qweight, qw, sid)
        layer.htr_scales.weight_loader(layer.htr_scales, sc, sid)
        layer.htr_sv.weight_loader(layer.htr_sv, sv, sid)
        layer.htr_su.weight_loader(layer.htr_su, su, sid)
    assert torch.equal(layer.htr_qweight.data, torch.cat([parts[s][0] for s in "qkv"]))
    assert torch.equal(layer.htr_scales.data, torch.cat([parts[s][1] for s in "qkv"]))
    assert torch.equal(layer.htr_sv.data, torch.cat([parts[s][3] for s in "qkv"]))
    assert torch.equal(layer.htr_su.data, su)
    with pytest.raises(ValueError):                                    # a shard with another sign vector
        layer.htr_su.weight_loader(layer.htr_su, parts["k"][2], "k")
    with pytest.raises(AssertionError):                                # wrong shard shape
        layer.htr_scales.weight_loader(layer.htr_scales, parts["q"][1], "k")
    # shard id carried on the tensor, and a whole-module load
    t = parts["k"][1].clone()
    t.shard_id = "k"
    layer.htr_scales.weight_loader(layer.htr_scales, t)
    layer.htr_scales.weight_loader(layer.htr_scales, torch.ones(512, dtype=torch.float16))
    assert bool(torch.all(layer.htr_scales.data == 1))
    with pytest.raises(AssertionError):                                # tensor parallel shards are refused
        vp.HTRLinearMethod(4).create_weights(_Linear(), 128, [256], 256, 256, torch.bfloat16)
    with pytest.raises(AssertionError):
        vp.HTRLinearMethod(4).create_weights(_Linear(), 192, [256], 192, 256, torch.bfloat16)


def test_apply_routes_to_ops_linear_and_counts(monkeypatch, tmp_path):
    from htr_amd import ops
    layer = _Linear()
    vp.HTRLinearMethod(4).create_weights(layer, 128, [128], 128, 128, torch.bfloat16)
    seen = {}

    def fake_linear(x, qw, sc, su, sv, bias=None):
        seen["args"] = (x, qw, sc, su, sv, bias)
        return torch.zeros(*x.shape[:-1], 128, dtype=x.dtype)
    monkeypatch.setattr(ops, "linear", fake_linear)
    monkeypatch.setattr(vp, "_COUNT_FILE", str(tmp_path / "census"))
    vp._CENSUS.counts.clear()
    vp._CENSUS.calls = 0
    x = torch.zeros(3, 128, dtype=torch.bfloat16)
    b = torch.zeros(128, dtype=torch.bfloat16)
    for _ in range(512):
        y = vp.HTRLinearMethod(4).apply(layer, x, b)
    assert tuple(y.shape) == (3, 128)
    assert seen["args"][1] is layer.htr_qweight and seen["args"][5] is b
    dumped = json.load(open(f"{tmp_path / 'census'}.{os.getpid()}.json"))
    assert dumped["counts"] == {"M2-8": 512, "K4": 512}


def test_register_needs_vllm():
    if vp.HAVE_VLLM:
        assert vp.register() is vp.HTRConfig
    else:
        with pytest.raises(ImportError):
            vp.register()
