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


# ---- routed-expert chunks (htr/moe_encode.py:26-29, 216-225 of the reference)
GOLDEN_MOE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "moe_L3")


def test_packed_chunk_fixture_reads_and_verifies():
    pe = checkpoint.PackedExperts(GOLDEN_MOE)
    assert pe.plan["format"] == "HTR-W1-P2-PACKED-1" and pe.layers() == [3]
    assert [os.path.basename(p) for p in pe.chunks(3)] == ["c000.pt", "c002.pt"]
    z = checkpoint.read_packed_chunk(pe.chunks(3)[1], verify=True)
    assert z["L"] == 3 and z["K"] == 3 and sorted(z["experts"]) == [2, 3] and z["experts"][3]["n"] == 15
    gate_up, down, K = pe.layer(3, verify=True)
    assert K == 3 and len(gate_up) == len(down) == 4
    for e in range(4):
        assert wire.check_shapes(*gate_up[e]) == (256, 256, 3) and wire.check_shapes(*down[e]) == (256, 128, 3)
        want = wire.synth_linear(128, 256, 3, 7000 + 10 * e)                 # the seeds tests/golden/make_moe_chunk.py uses
        assert torch.equal(gate_up[e][0][:8], want[0]) and torch.equal(gate_up[e][1][:128], want[1])
        assert torch.equal(gate_up[e][2], want[2]) and torch.equal(gate_up[e][3][:16], want[3])
        assert torch.equal(down[e][0], wire.synth_linear(256, 128, 3, 7002 + 10 * e)[0])


def test_packed_chunk_round_trip_and_refusals(tmp_path):
    def expert(e, K=2, same_su=True):
        g = wire.synth_linear(128, 128, K, 10 + e)
        u = wire.synth_linear(128, 128, K, 20 + e)
        if same_su:
            u = (u[0], u[1], g[2], u[3])
        return {"e": e, "n": e, "packed": {"gate": g, "up": u, "down": wire.synth_linear(128, 128, K, 30 + e)}}

    root = tmp_path / "run"
    checkpoint.write_packed_chunk(str(root / "L0" / "c000.pt"), 0, 2, [expert(0), expert(1)])
    gate_up, down, K = checkpoint.PackedExperts(str(root)).layer(0, verify=True)
    assert K == 2 and len(gate_up) == 2 and gate_up[1][0].shape == (16, 8, 16)
    # a flipped payload bit fails the hash check and only the hash check
    z = torch.load(str(root / "L0" / "c000.pt"), weights_only=True)
    z["experts"][0]["packed"]["down"]["qweight"][0, 0, 0] ^= 1
    torch.save(z, str(root / "L0" / "c000.pt"))
    checkpoint.read_packed_chunk(str(root / "L0" / "c000.pt"))
    with pytest.raises(ValueError, match="reconstruction hash"):
        checkpoint.read_packed_chunk(str(root / "L0" / "c000.pt"), verify=True)
    with pytest.raises(ValueError, match="reconstruction hash"):
        checkpoint.read_packed_chunk(str(root / "L0" / "c000.pt"), verify="first")     # the flipped bit is in the first expert
    z2 = torch.load(str(root / "L0" / "c000.pt"), weights_only=True)
    z2["experts"][0]["packed"]["down"]["qweight"][0, 0, 0] ^= 1                        # first expert whole again,
    z2["experts"][1]["packed"]["up"]["qweight"][0, 0, 0] ^= 1                          # the second one damaged
    torch.save(z2, str(tmp_path / "second.pt"))
    checkpoint.read_packed_chunk(str(tmp_path / "second.pt"), verify="first")          # the cheap check looks at the first only
    with pytest.raises(ValueError, match="reconstruction hash"):
        checkpoint.read_packed_chunk(str(tmp_path / "second.pt"), verify=True)
    # another format string, a hole in the expert ids, gate/up with different su, mixed K in one layer, wrong layer
    z["format"] = "HTR-W1-P1"
    torch.save(z, str(tmp_path / "bad.pt"))
    with pytest.raises(ValueError, match="not a HTR-W1-P2-PACKED-1"):
        checkpoint.read_packed_chunk(str(tmp_path / "bad.pt"))
    checkpoint.write_packed_chunk(str(root / "L1" / "c002.pt"), 1, 2, [expert(2), expert(3)])
    with pytest.raises(ValueError, match="chunks missing"):
        checkpoint.PackedExperts(str(root)).layer(1)
    checkpoint.write_packed_chunk(str(root / "L2" / "c000.pt"), 2, 2, [expert(0, same_su=False)])
    with pytest.raises(ValueError, match="share the input sign"):
        checkpoint.PackedExperts(str(root)).layer(2)
    checkpoint.write_packed_chunk(str(root / "L4" / "c000.pt"), 4, 2, [expert(0)])
    checkpoint.write_packed_chunk(str(root / "L4" / "c001.pt"), 4, 3, [expert(1, K=3)])
    with pytest.raises(ValueError, match="earlier chunks"):
        checkpoint.PackedExperts(str(root)).layer(4)
    checkpoint.write_packed_chunk(str(root / "L5" / "c000.pt"), 6, 2, [expert(0)])
    with pytest.raises(ValueError, match="under L5"):
        checkpoint.PackedExperts(str(root)).layer(5)
    with pytest.raises(ValueError, match="not K = 3"):
        checkpoint.write_packed_chunk(str(tmp_path / "k.pt"), 0, 3, [expert(0)])


def test_packed_chunk_loader_executes_nothing(tmp_path):
    """A chunk-shaped pickle that carries a callable is refused by the weights-only loader instead of being run."""
    import pickle

    class Boom:
        def __reduce__(self):
            return (os.system, ("true",))

    with open(tmp_path / "evil.pt", "wb") as f:
        pickle.dump({"format": "HTR-W1-P2-PACKED-1", "L": 0, "K": 2, "experts": [Boom()]}, f)
    with pytest.raises(Exception) as ei:
        checkpoint.read_packed_chunk(str(tmp_path / "evil.pt"))
    assert "Unsupported" in str(ei.value) or "weights_only" in str(ei.value) or "pickle" in str(ei.value).lower()
