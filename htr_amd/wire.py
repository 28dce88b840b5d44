"""HTR-W1 wire format helpers used by the host side of the gfx950 path.

Own statement of the format in the reference's docs/FORMAT.md.  The device kernels never
materialise a codebook; this module only carries the constants and the packing helpers the
host needs (shapes, payload accounting, sign packing, synthetic tensors for benchmarks).
Names mirror htr/wire.py of the reference where a function has a counterpart there.
"""
import math

import torch

L = 16
S = 1 << L
GEN_A, GEN_B = 0xDF6ADF, 0x34983
TILE = 16
RHT_BLOCK = 128
WIRE_NAME = "HTR-W1"
# sum over all 65536 states of v(s)^2: an integer, so the float64 mean is order-independent
SUM_V_SQ = 1433042863


def cbscale():
    """1 / sqrt(mean v^2) as a Python float (htr/wire.py:28-30 of the reference)."""
    return 1.0 / math.sqrt(SUM_V_SQ / S)


def gen_values(states):
    """Integer codebook value v(s) for integer states of any shape (htr/wire.py:10-13): the generator word
    s * A + B is reduced mod 2^32 and its four bytes are summed; the sum of four uniform bytes has mean 510."""
    word = torch.remainder(states.to(torch.int64) * GEN_A + GEN_B, 1 << 32)
    total = torch.zeros_like(word)
    for _ in range(4):
        total += torch.remainder(word, 256)
        word = word // 256
    return total - 510


_CACHE = {}


def codebook_f32(device="cpu"):
    """cb[s] = float32(v(s) / rms), rms = sqrt(mean v^2) in float64 (htr/wire.py:19-25 of the reference)."""
    key = ("cb", str(device))
    if key not in _CACHE:
        v = gen_values(torch.arange(S, dtype=torch.int64)).double()
        _CACHE[key] = (v / math.sqrt(SUM_V_SQ / S)).float().to(device)
    return _CACHE[key]


def hadamard(n, device="cpu"):
    """Sylvester Hadamard matrix / sqrt(n) (htr/wire.py:80-87): entry (i, j) is (-1)^popcount(i & j); the division is
    done in float64 and rounded once to float32, which is what the reference's recursion yields as well."""
    key = ("had", n, str(device))
    if key not in _CACHE:
        i = torch.arange(n, dtype=torch.int64)
        both = i[:, None] & i[None, :]
        parity = torch.zeros_like(both)
        while bool(both.any()):
            parity ^= both & 1
            both = both >> 1
        _CACHE[key] = ((1.0 - 2.0 * parity.double()) / math.sqrt(n)).float().to(device)
    return _CACHE[key]


def blk_had_cols_T(W, bs=RHT_BLOCK):
    """Every block of bs consecutive columns of W times H (htr/wire.py:90-92).  The batched float32 matmul, in this
    form, is the contract: the reference's encoder fixture (What) is reproduced bit for bit only with torch's own
    summation order."""
    m, n = W.shape
    return (W.reshape(m, n // bs, bs) @ hadamard(bs, W.device)).reshape(m, n)


def unpack_states(words, K):
    """int32 words [B, 8K] -> int64 states [B, 256]: state t = the 16 stream bits that end at bit (t + 1) K - 1,
    circular, MSB first (htr/wire.py:46-63).  Built from a doubled bit string instead of a 16-way gather."""
    B = words.shape[0]
    sh = torch.arange(31, -1, -1, device=words.device)
    bits = ((words.long()[:, :, None] >> sh) & 1).reshape(B, 256 * K)
    ext = torch.cat([bits[:, -16:], bits], 1)                      # position p of `bits` sits at p + 16
    pw = 1 << torch.arange(15, -1, -1, device=words.device)
    win = ext.unfold(1, 16, 1)                                      # window i covers bits i - 16 .. i - 1
    idx = (torch.arange(256, device=words.device) + 1) * K          # window that ends at bit (t + 1) K - 1
    return (win[:, idx, :] * pw).sum(-1)


def dequant_Q(qweight, scales):
    """Rotated-domain Q [m, n] float32 on the tensors' device, with torch (htr/wire.py:95-102).  Slow; the library's
    htr_dequant_q is the fast one."""
    mt, nt, W = qweight.shape
    st = unpack_states(qweight.reshape(-1, W), W // 8)
    R = codebook_f32(qweight.device)[st].reshape(mt, nt, 16, 16).permute(0, 2, 1, 3).reshape(mt * 16, nt * 16)
    return R * scales.float()[:, None]


def dequant(qweight, scales, su8, sv8):
    """Original-basis W [m, n] float32 = Sv . Ho . Q . Hi . Su with torch, in the reference's order of operations
    (htr/wire.py:105-113): rows first, then columns, then both signs.  The order is kept on purpose; any other one
    rounds differently and no longer matches the reference's What fixture bit for bit."""
    Q = dequant_Q(qweight, scales)
    m, n = Q.shape
    su = unpack_signs(su8, n).to(Q.device)
    sv = unpack_signs(sv8, m).to(Q.device)
    W = blk_had_cols_T(Q.T.contiguous()).T
    W = blk_had_cols_T(W.contiguous())
    return (W * sv[:, None] * su[None, :]).contiguous()


def pack_signs(s):
    """+-1 vector [N] (N % 8 == 0) -> uint8 [N/8]; bit j%8 (LSB first) of byte j/8 set means -1 (htr/wire.py:66-69)."""
    neg = (s < 0).to(torch.int32).view(-1, 8)
    w = (1 << torch.arange(8, dtype=torch.int32, device=s.device))
    return (neg * w).sum(-1).to(torch.uint8)


def unpack_signs(u8, N):
    """uint8 [N/8] -> float32 +-1 [N]: element j is -1 where bit j % 8 of byte j / 8 is set (htr/wire.py:72-74)."""
    j = torch.arange(N, device=u8.device)
    byte = u8.reshape(-1).to(torch.int64)[j // 8]
    minus = torch.remainder(byte // (1 << (j % 8)), 2) == 1
    return torch.where(minus, -1.0, 1.0).to(torch.float32)


def pack_states(states, K):
    """Tail-biting trellis path int64 [B, 256] -> int32 words [B, 8K], MSB first (htr/wire.py:33-43)."""
    B, T = states.shape
    if T != 256 or not 2 <= K <= 8:
        raise ValueError("pack_states wants [B, 256] states and 2 <= K <= 8")
    # the stream is the states' low K bits one after the other; bit p of it (MSB first) belongs to state p / K and is
    # that state's bit K - 1 - p % K; 32 consecutive stream bits make one big-endian word
    p = torch.arange(256 * K, device=states.device)
    fresh = torch.remainder(states.to(torch.int64), 1 << K)
    stream = torch.remainder(fresh[:, p // K] // (1 << (K - 1 - p % K)), 2)
    place = 1 << (31 - p % 32)
    words = torch.zeros(B, 8 * K, dtype=torch.int64, device=states.device)
    words.index_add_(1, p // 32, stream * place)
    return (words - (words >> 31) * (1 << 32)).to(torch.int32)          # two's complement view of the uint32 value


def bits_of(qweight):
    """K of a packed weight: last dim is 8K words (docs/FORMAT.md:30)."""
    return qweight.shape[-1] // 8


def payload_bytes(m, n, K):
    """W1 payload of one linear: streams + fp16 row scales + both sign vectors (docs/METHODOLOGY.md:87-90)."""
    return m * n * K // 8 + 2 * m + n // 8 + m // 8


def check_shapes(qweight, scales, su, sv):
    """Validate one HTR-W1 tensor set; returns (m, n, K)."""
    if qweight.dim() != 3 or qweight.dtype != torch.int32:
        raise RuntimeError("htr_qweight must be int32 [m/16, n/16, 8K]")
    mt, nt, W = qweight.shape
    K = W // 8
    if W % 8 or not 2 <= K <= 8:
        raise RuntimeError(f"unsupported K {W / 8}")
    m, n = mt * 16, nt * 16
    if m % RHT_BLOCK or n % RHT_BLOCK:
        raise RuntimeError("HTR-W1 needs m % 128 == 0 and n % 128 == 0")
    if scales.dtype != torch.float16 or scales.numel() != m:
        raise RuntimeError("htr_scales must be float16 [m]")
    if su.dtype != torch.uint8 or su.numel() != n // 8 or sv.dtype != torch.uint8 or sv.numel() != m // 8:
        raise RuntimeError("htr_su / htr_sv must be uint8 [n/8] / [m/8]")
    return m, n, K


def synth_linear(m, n, K, seed, device="cpu"):
    """Seeded synthetic HTR-W1 tensors.

    Every 256K-bit string is a valid circular trellis stream (states are derived from the
    bits), so uniform random words are uniform random trellis paths.  Row scales are
    lognormal(0, 0.25) in float16; sign bytes are uniform.
    """
    g = torch.Generator(device="cpu").manual_seed(seed)
    qweight = torch.randint(-(2 ** 31), 2 ** 31, (m // 16, n // 16, 8 * K), dtype=torch.int32, generator=g)
    scales = torch.exp(0.25 * torch.randn(m, generator=g)).half()
    su = torch.randint(0, 256, (n // 8,), dtype=torch.uint8, generator=g)
    sv = torch.randint(0, 256, (m // 8,), dtype=torch.uint8, generator=g)
    return tuple(t.to(device) for t in (qweight, scales, su, sv))


def synth_activation(M, n, seed, dtype=torch.bfloat16, device="cpu"):
    g = torch.Generator(device="cpu").manual_seed(seed)
    return torch.randn(M, n, generator=g).to(dtype).to(device)
