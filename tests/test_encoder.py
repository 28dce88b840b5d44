"""The matrix encoder (htr_amd/encode.py; htr/encode.py:45-110 of the reference) and its GPU trellis search.

CPU: the encoder's host logic around the CPU oracle's Viterbi must reproduce, bit for bit, what the reference's
encode_group produced for the same inputs (tests/golden/encode_small.npz, written by tests/golden/make_encoder_golden.py).
GPU: the library's search against the oracle's on identical inputs (states bit-exact), and the whole encoder on the
device against the bars of the reference's own round-trip test (tests/test_release.py:53-73)."""
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def enc_gold():
    return np.load(os.path.join(HERE, "golden", "encode_small.npz"), allow_pickle=False)


@pytest.fixture(scope="module")
def vit_gold():
    return np.load(os.path.join(HERE, "golden", "viterbi.npz"), allow_pickle=False)


@pytest.fixture()
def oracle_search(oracle):
    from htr_amd import encode
    old = encode.VITERBI
    encode.VITERBI = lambda x, w, cb, K: torch.from_numpy(oracle.c_viterbi(x.numpy(), w.numpy(), K).astype(np.int64))
    yield encode
    encode.VITERBI = old


def _same(result, gold, tag):
    assert np.array_equal(result["qweight"].numpy(), gold[f"{tag}_qweight"])
    assert np.array_equal(result["scales"].numpy().view(np.uint16), gold[f"{tag}_scales_f16bits"])
    assert np.array_equal(result["su"].numpy(), gold[f"{tag}_su"]) and np.array_equal(result["sv"].numpy(), gold[f"{tag}_sv"])
    assert np.array_equal(result["What"].numpy(), gold[f"{tag}_What"])


def test_encoder_reproduces_reference_on_its_round_trip_matrix(oracle_search, enc_gold):
    from htr_amd import wire
    w = torch.from_numpy(enc_gold["a_W"])
    r = oracle_search.encode_group([{"W": w, "H": torch.eye(128)}], 4, max_batch=8)[0]
    _same(r, enc_gold, "a")
    # the bars of the reference's own test (tests/test_release.py:69-73)
    actual = wire.dequant(r["qweight"], r["scales"], r["su"], r["sv"])
    assert torch.equal(actual, r["What"]) and tuple(r["qweight"].shape) == (8, 8, 32)
    assert bool(torch.isfinite(actual).all())
    assert float((actual - w).square().sum() / w.square().sum()) < 0.02


def test_encoder_reproduces_reference_with_hessian_and_shared_signs(oracle_search, enc_gold):
    H = torch.from_numpy(enc_gold["b_H"])
    jobs = [{"W": torch.from_numpy(enc_gold["b0_W"]), "H": H}, {"W": torch.from_numpy(enc_gold["b1_W"]), "H": H}]
    rs = oracle_search.encode_group(jobs, 3, seed=4321, max_batch=64)
    _same(rs[0], enc_gold, "b0")
    _same(rs[1], enc_gold, "b1")
    assert np.array_equal(rs[0]["su"].numpy(), rs[1]["su"].numpy())          # one input sign vector for the group


@pytest.mark.parametrize("K", [2, 3, 4, 5])
def test_cpu_search_matches_reference_vectors(vit_gold, K):
    """CPU tensors take the torch search (the GPU kernel's formulation): bit-identical to the reference's vectors,
    the all-ties row included."""
    from htr_amd import encode
    x, w = torch.from_numpy(vit_gold[f"k{K}_x"]), torch.from_numpy(vit_gold[f"k{K}_w"])
    st = encode.viterbi(x, w, None, K)
    assert st.dtype == torch.int64 and np.array_equal(st.numpy().astype(np.uint16), vit_gold[f"k{K}_states"])


@pytest.mark.parametrize("K,B,T,tailbite", [(6, 2, 256, True), (8, 2, 64, True), (4, 3, 100, False), (4, 2, 1, True), (3, 2, 17, False)])
def test_cpu_search_matches_oracle(oracle, K, B, T, tailbite):
    from htr_amd import encode
    g = torch.Generator().manual_seed(100 * K + T)
    x = torch.randn(B, T, generator=g) * 1.2
    w = torch.rand(B, T, generator=g) + 0.25
    x[0, : T // 2] = 0.0
    st = encode.viterbi_cpu(x, w, K, tailbite).numpy()
    assert np.array_equal(st.astype(np.uint32), oracle.c_viterbi(x.numpy(), w.numpy(), K, tailbite=tailbite))


def test_encoder_on_cpu_tensors_without_a_hook(enc_gold):
    """encode_group on CPU tensors with VITERBI unset (the reference falls back to its portable search there,
    htr/encode.py:10-12, 48): the torch search reproduces the reference's round-trip matrix bit for bit."""
    from htr_amd import encode
    assert encode.VITERBI is None
    r = encode.encode_group([{"W": torch.from_numpy(enc_gold["a_W"]), "H": torch.eye(128)}], 4, max_batch=8)[0]
    _same(r, enc_gold, "a")


def test_matrices_of_one_hessian_share_a_factorisation(oracle_search, enc_gold, monkeypatch):
    """Two matrices that come with the same Hessian object under a shared input sign vector are factored once and fed
    back with one product; the result is the one of separate factorisations (the reference's fixture)."""
    calls = []
    real = oracle_search._feedback_factor
    monkeypatch.setattr(oracle_search, "_feedback_factor", lambda Hd: (calls.append(1), real(Hd))[1])
    H = torch.from_numpy(enc_gold["b_H"])
    jobs = [{"W": torch.from_numpy(enc_gold[f"b{i}_W"]), "H": H} for i in range(2)]
    rs = oracle_search.encode_group(jobs, 3, seed=4321, max_batch=64)
    assert len(calls) == 1
    for i, r in enumerate(rs):
        assert np.array_equal(r["qweight"].numpy(), enc_gold[f"b{i}_qweight"])
    calls.clear()
    oracle_search.encode_group([{"W": jobs[0]["W"], "H": H}, {"W": jobs[1]["W"], "H": H.clone()}], 3, seed=4321, max_batch=64)
    assert len(calls) == 2


def test_sign_draws_and_hessian_preparation():
    from htr_amd import encode
    su, sv = encode.make_signs(256, 128, 99, 2, True)
    su2, sv2 = encode.make_signs(256, 128, 99, 5, True)
    assert torch.equal(su, su2) and not torch.equal(sv, sv2) and set(su.tolist()) == {-1.0, 1.0}
    a, b = encode.make_signs(256, 128, 99, 2, False)
    g = torch.Generator().manual_seed(99 + 7919 * 2)
    assert torch.equal(a, (torch.randint(0, 2, (256,), generator=g) * 2 - 1).float())
    assert torch.equal(b, (torch.randint(0, 2, (128,), generator=g) * 2 - 1).float())
    H = torch.diag(torch.tensor([2.0, 0.0, 4.0]))
    W = torch.ones(2, 3)
    Hp, Wp = encode.prep_H(H, W, damp=0.5)
    mean = (2.0 + 1.0 + 4.0) / 3                                             # dead diagonal entry becomes 1
    assert torch.allclose(torch.diag(Hp), torch.tensor([2.0, 1.0, 4.0], dtype=torch.float64) + 0.5 * mean)
    assert torch.equal(Wp, torch.tensor([[1.0, 0.0, 1.0], [1.0, 0.0, 1.0]]))


# ---------------------------------------------------------------------------------------------------------------- GPU
@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from htr_amd import _native
    _native.lib()
    return torch.device("cuda:0")


@pytest.mark.gpu
@pytest.mark.parametrize("K", [2, 3, 4, 5])
def test_gpu_search_matches_reference_vectors(dev, vit_gold, K):
    from htr_amd import encode
    print(f"viterbi golden K={K}", flush=True)
    x, w = torch.from_numpy(vit_gold[f"k{K}_x"]), torch.from_numpy(vit_gold[f"k{K}_w"])
    st = encode.viterbi(x.to(dev), w.to(dev), None, K).cpu().numpy()
    assert np.array_equal(st.astype(np.uint16), vit_gold[f"k{K}_states"])


@pytest.mark.gpu
@pytest.mark.parametrize("K,B,T,tailbite", [(2, 5, 256, True), (3, 7, 256, True), (4, 9, 256, True), (5, 6, 256, True),
                                            (6, 3, 256, True), (7, 2, 256, True), (8, 3, 256, True), (8, 2, 256, False), (8, 2, 9, True),
                                            (4, 3, 256, False), (3, 4, 100, True),
                                            (4, 2, 1, True), (2, 2, 17, False)])
def test_gpu_search_matches_oracle(dev, oracle, K, B, T, tailbite):
    from htr_amd import encode
    print(f"viterbi K={K} B={B} T={T} tailbite={tailbite}", flush=True)
    g = torch.Generator().manual_seed(1000 * K + B + T)
    x = torch.randn(B, T, generator=g) * 1.2
    w = torch.rand(B, T, generator=g) + 0.25
    x[0, : T // 2] = 0.0                                                     # long runs of equal costs
    st = encode.viterbi(x.to(dev), w.to(dev), None, K, tailbite=tailbite).cpu().numpy()
    want = oracle.c_viterbi(x.numpy(), w.numpy(), K, tailbite=tailbite)
    assert np.array_equal(st.astype(np.uint32), want)


@pytest.mark.gpu
def test_gpu_search_refuses_another_codebook(dev):
    from htr_amd import encode, wire
    print("viterbi: codebook check", flush=True)
    x, w = torch.zeros(1, 16), torch.ones(1, 16)
    cb = wire.codebook_f32(dev)
    assert encode.viterbi(x.to(dev), w.to(dev), cb, 4).shape == (1, 16)
    with pytest.raises(RuntimeError, match="not the HTR-W1 codebook"):
        encode.viterbi(x.to(dev), w.to(dev), cb * 2.0, 4)
    assert encode.viterbi(x, w, None, 4).shape == (1, 16)           # CPU tensors: the torch search


@pytest.mark.gpu
def test_gpu_encoder_round_trip(dev, enc_gold):
    """The reference's round-trip test on the device: encode the seed-12 matrix with the library's search, reopen, decode.
    torch's device linear algebra need not match the CPU's last bits, so the comparison with the CPU fixture is by
    share of identical tiles; the decode identity and the error bar are exact requirements."""
    from htr_amd import encode, ops, wire
    print("encoder round trip", flush=True)
    w = torch.from_numpy(enc_gold["a_W"]).to(dev)
    r = encode.encode_group([{"W": w, "H": torch.eye(128, device=dev)}], 4, max_batch=8)[0]
    assert tuple(r["qweight"].shape) == (8, 8, 32)
    d = [r[k].to(dev) for k in ("qweight", "scales", "su", "sv")]
    actual = wire.dequant(*d)
    assert torch.equal(actual, r["What"]) and bool(torch.isfinite(actual).all())
    assert float((actual - w).square().sum() / w.square().sum()) < 0.02
    same = float((r["qweight"].numpy() == enc_gold["a_qweight"]).all(axis=2).mean())
    assert same >= 0.9, same
    # the packed linear on the encoded matrix reproduces x @ What^T
    x = torch.randn(3, 128, generator=torch.Generator().manual_seed(1)).to(dev)
    y = ops.linear_f32out(x, *d)
    ref = x @ actual.T
    assert float((y - ref).abs().max() / ref.abs().max()) <= 1e-3
