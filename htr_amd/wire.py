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
    """Integer codebook value v(s) for int64 states of any shape (htr/wire.py:10-13)."""
    x = (states.long() * GEN_A + GEN_B) & 0xFFFFFFFF
    return ((x & 0xFF) + ((x >> 8) & 0xFF) + ((x >> 16) & 0xFF) + ((x >> 24) & 0xFF)) - 510


_CACHE = {}


def codebook_f32(device="cpu"):
    """cb[s] = float32(v(s) / rms), rms = sqrt(mean v^2) in float64 (htr/wire.py:19-25 of the reference)."""
    key = ("cb", str(device))
    if key not in _CACHE:
        v = gen_values(torch.arange(S, dtype=torch.int64)).double()
        _CACHE[key] = (v / math.sqrt(SUM_V_SQ / S)).float().to(device)
    return _CACHE[key]


def hadamard(n, device="cpu"):
    """Sylvester Hadamard matrix / sqrt(n), built in float64 and rounded once to float32 (htr/wire.py:80-87)."""
    key = ("had", n, str(device))
    if key not in _CACHE:
        h = torch.ones(1, 1, dtype=torch.float64)
        while h.shape[0] < n:
            h = torch.cat([torch.cat([h, h], 1), torch.cat([h, -h], 1)], 0)
        _CACHE[key] = (h / math.sqrt(n)).float().to(device)
    return _CACHE[key]


def blk_had_cols_T(W, bs=RHT_BLOCK):
    """Every block of bs consecutive columns of W times H (htr/wire.py:90-92)."""
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
    (htr/wire.py:105-113)."""
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
    """uint8 [N/8] -> float32 +-1 [N] (htr/wire.py:72-74)."""
    bits = (u8.view(-1, 1).to(torch.int32) >> torch.arange(8, dtype=torch.int32, device=u8.device)) & 1
    return 1.0 - 2.0 * bits.reshape(-1)[:N].float()


def pack_states(states, K):
    """Tail-biting trellis path int64 [B, 256] -> int32 words [B, 8K], MSB first (htr/wire.py:33-43)."""
    B, T = states.shape
    if T != 256 or not 2 <= K <= 8:
        raise ValueError("pack_states wants [B, 256] states and 2 <= K <= 8")
    b = states.long() & ((1 << K) - 1)
    sh = torch.arange(K - 1, -1, -1, device=states.device)
    bits = ((b[:, :, None] >> sh) & 1).reshape(B, 8 * K, 32)
    wsh = torch.arange(31, -1, -1, device=states.device)
    words = (bits << wsh).sum(-1)
    return torch.where(words >= 2 ** 31, words - 2 ** 32, words).to(torch.int32)


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
