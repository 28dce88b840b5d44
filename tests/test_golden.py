"""Committed known-answer vectors (tests/golden/w1_small.npz, made by tests/golden/make_golden.py from the format
text alone) against the CPU oracle (always) and the gfx950 library (on a GPU)."""
import os

import numpy as np
import pytest
import torch

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "w1_small.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD, allow_pickle=False)


def _case(gold, k):
    qw = gold[f"k{k}_qweight"]
    sc = gold[f"k{k}_scales_f16bits"].view(np.float16)
    x = torch.from_numpy(gold[f"k{k}_x_bf16bits"].view(np.int16)).view(torch.bfloat16)
    return qw, sc, gold[f"k{k}_su"], gold[f"k{k}_sv"], x


@pytest.mark.parametrize("k", [2, 3, 4, 5])
def test_oracle_matches_golden(oracle, gold, k):
    qw, sc, su, sv, x = _case(gold, k)
    assert float(gold["rms"][0]) == oracle.c_rms()
    assert np.array_equal(oracle.c_decode_raw(qw), gold[f"k{k}_v"])
    assert np.array_equal(oracle.np_gen_values(oracle.np_unpack_states(qw.reshape(-1, 8 * k), k)).astype(np.int16), gold[f"k{k}_v"])
    y = oracle.c_linear(x.float().numpy(), qw, sc, su, sv)
    assert np.allclose(y, gold[f"k{k}_y"], rtol=0, atol=1e-11 * np.abs(gold[f"k{k}_y"]).max())
    if k == 4:
        assert np.array_equal(oracle.c_dequant_q(qw, sc).view(np.uint32), gold["k4_Q"].view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("k", [2, 3, 4, 5])
def test_gpu_matches_golden(gold, k):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from htr_amd import ops
    print(f"golden K={k}", flush=True)
    dev = torch.device("cuda:0")
    qw, sc, su, sv, x = _case(gold, k)
    d = [torch.from_numpy(np.ascontiguousarray(a)).to(dev) for a in (qw, sc, su, sv)]
    assert np.array_equal(ops.decode_raw(d[0]).cpu().numpy(), gold[f"k{k}_v"])
    if k == 4:
        assert np.array_equal(ops.dequant_q(d[0], d[1]).cpu().numpy().view(np.uint32), gold["k4_Q"].view(np.uint32))
    y = ops.linear_f32out(x.to(dev), *d).cpu().numpy()
    ref = gold[f"k{k}_y"]
    assert np.abs(y - ref).max() <= 1e-3 * np.abs(ref).max()
