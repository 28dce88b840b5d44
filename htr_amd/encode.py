"""HTR-W1 matrix encoder on MI355X: block-LDLQ error feedback around the tail-biting trellis search.

Same algorithm and call surface as htr/encode.py of the reference (encode_group, make_signs, prep_H, the VITERBI
hook, htr/encode.py:1-110): rotate W and the Hessian with the randomized Hadamard transform, factor the damped
Hessian, walk the 16-column blocks from the last to the first, search each block's 256-weight tiles with the trellis
Viterbi, and feed the quantization error of a block forward into the columns not yet encoded.  The search runs in
libhtr_gfx950.so (htr_viterbi, one workgroup per tile) when the tensors are on the GPU; the linear algebra around it is
torch.  Results are HTR-W1 tensors plus the reconstruction `What`.
"""
import torch

from . import _native, wire

# callable(x[B, 256], w[B, 256], cb[65536], K) -> int64 states [B, 256]; None = the library's search on the GPU
VITERBI = None
# tiles per launch: bounds the backpointer scratch (tiles * 255 * (65536 >> K) bytes)
MAX_SCRATCH_BYTES = 1 << 30
_SCRATCH = {}


def viterbi(x, w, cb=None, K=4, tailbite=True):
    """Tail-biting bitshift-trellis Viterbi on the GPU (htr.reference.viterbi / htr.vit_v2.viterbi of the reference).

    x, w: float32 [B, T <= 256] on a ROCm device.  cb is accepted for signature compatibility and must be the HTR
    codebook (the kernel evaluates it procedurally).  Returns int64 states [B, T].
    """
    if not x.is_cuda:
        raise RuntimeError("htr_amd.encode.viterbi runs on a ROCm device only")
    x = x.float().contiguous()
    w = w.float().contiguous()
    B, T = x.shape
    if w.shape != x.shape or not 1 <= T <= 256:
        raise RuntimeError("viterbi wants x and w of one shape [B, T <= 256]")
    L = _native.lib()
    per_tile = L.htr_viterbi_workspace_bytes(1, T, K)
    if per_tile == 0:
        raise RuntimeError(f"viterbi: unsupported K {K} (2..7)")
    out = torch.empty((B, T), dtype=torch.int16, device=x.device)
    batch = max(1, min(B, MAX_SCRATCH_BYTES // per_tile))
    cus = torch.cuda.get_device_properties(x.device).multi_processor_count
    if B > batch >= cus:
        batch -= batch % cus        # one workgroup per tile: whole rounds over the CUs, no launch with a few stragglers
    with torch.cuda.device(x.device):
        stream = torch.cuda.current_stream(x.device)
        need = L.htr_viterbi_workspace_bytes(batch, T, K)
        key = (x.device.index, stream.cuda_stream)
        ws = _SCRATCH.get(key)
        if ws is None or ws.numel() < need:
            ws = torch.empty(need, dtype=torch.uint8, device=x.device)
            _SCRATCH[key] = ws
        for b0 in range(0, B, batch):
            nb = min(batch, B - b0)
            _native.check(L.htr_viterbi(x[b0:].data_ptr(), w[b0:].data_ptr(), nb, T, K, 1 if tailbite else 0,
                                        out[b0:].data_ptr(), ws.data_ptr(), ws.numel(), stream.cuda_stream))
    return out.long() & 0xFFFF


def block_rotate(W, bs=wire.RHT_BLOCK):
    """Blocks of bs columns times H^T (H is symmetric; kept as in htr/encode.py:15-17)."""
    m, n = W.shape
    return (W.reshape(m, n // bs, bs) @ wire.hadamard(bs, W.device).T).reshape(m, n)


def make_signs(n, m, seed, index, shared_su):
    """The reference's sign draws (htr/encode.py:20-32): with a shared input sign vector, su comes from generator(seed)
    for the whole input group and sv from generator(seed + 7919 (index + 1)); otherwise both from
    generator(seed + 7919 index), su first."""
    def draw(g, count):
        return (torch.randint(0, 2, (count,), generator=g) * 2 - 1).float()
    if shared_su:
        su = draw(torch.Generator().manual_seed(seed), n)
        sv = draw(torch.Generator().manual_seed(seed + 7919 * (index + 1)), m)
        return su, sv
    g = torch.Generator().manual_seed(seed + 7919 * index)
    su = draw(g, n)
    return su, draw(g, m)


def prep_H(H, W, damp=0.01):
    """Dead input columns get a unit diagonal and zero weights; the diagonal is damped by damp * mean(diag)
    (htr/encode.py:35-42).  float64."""
    H = H.clone().double()
    dead = torch.diag(H) == 0
    H[dead, dead] = 1.0
    W = W.clone()
    W[:, dead] = 0
    H += damp * torch.diag(H).mean() * torch.eye(H.shape[0], device=H.device, dtype=H.dtype)
    return H, W


class _Job:
    """One matrix of an input group in the rotated basis."""

    def __init__(self, W, H, su, sv, damp):
        n = W.shape[1]
        nb = n // 16
        Wt = block_rotate(W * sv[:, None] * su[None, :])
        Wt = block_rotate(Wt.T.contiguous()).T
        Ht = block_rotate(H * su[:, None] * su[None, :])
        Ht = block_rotate(Ht.T.contiguous()).T.contiguous()
        Ht, Wt = prep_H(Ht, Wt.contiguous(), damp)
        self.rs = Wt.pow(2).mean(dim=1).sqrt().half().float().clamp(min=1e-8)      # row scales, as stored (fp16)
        # block LDL feedback matrix: C = chol(H), normalised by its 16x16 diagonal blocks
        C = torch.linalg.cholesky(Ht)
        diag = C.view(nb, 16, nb, 16).diagonal(dim1=0, dim2=2).permute(2, 0, 1)
        self.Lb = torch.einsum("ikj,kjl->ikl", C.view(n, nb, 16), torch.linalg.inv(diag)).reshape(n, n).float()
        self.Wt = Wt.float()
        self.su, self.sv = su, sv
        self.Q = torch.zeros_like(self.Wt)
        self.F = torch.zeros_like(self.Wt)
        self.S = torch.zeros((W.shape[0] // 16, nb, 256), dtype=torch.int64, device=W.device)


@torch.no_grad()
def encode_group(jobs, K, seed=1234, shared_su=True, damp=0.01, max_batch=1024, log=None):
    """jobs: list of dict(W=[m, n], H=[n, n]) sharing n.  Returns a list of dict(qweight, scales, su, sv, What, Q)
    (htr/encode.py:45-110)."""
    search = VITERBI or (lambda x, w, cb, k: viterbi(x, w, cb, k))
    n = jobs[0]["W"].shape[1]
    if n % 128:
        raise RuntimeError("encode_group: n must be a multiple of 128")
    nb = n // 16
    dev = jobs[0]["W"].device
    cb = wire.codebook_f32(dev)
    P = []
    for index, jb in enumerate(jobs):
        W = jb["W"].float()
        if W.shape[0] % 128 or W.shape[1] != n:
            raise RuntimeError("encode_group: every matrix needs m % 128 == 0 and the group's n")
        su, sv = make_signs(n, W.shape[0], seed, index, shared_su)
        P.append(_Job(W, jb["H"].float().to(W.device), su.to(W.device), sv.to(W.device), damp))
    for k in range(nb - 1, -1, -1):                     # 16-column blocks, last first
        cols = slice(16 * k, 16 * k + 16)
        X = torch.cat([((p.Wt[:, cols] + p.F[:, cols]) / p.rs[:, None]).reshape(-1, 256) for p in P])
        Wg = torch.cat([(p.rs[:, None] ** 2).expand(-1, 16).contiguous().reshape(-1, 256) for p in P])
        Wg = Wg / Wg.mean(dim=1, keepdim=True)
        ST = torch.empty(X.shape, dtype=torch.int64, device=X.device)
        for b0 in range(0, X.shape[0], max_batch):
            ST[b0:b0 + max_batch] = search(X[b0:b0 + max_batch].contiguous(), Wg[b0:b0 + max_batch].contiguous(), cb, K)
        R = cb[ST]
        off = 0
        for p in P:
            m = p.Wt.shape[0]
            nt = m // 16
            p.S[:, k] = ST[off:off + nt]
            q = R[off:off + nt].reshape(m, 16) * p.rs[:, None]
            off += nt
            p.Q[:, cols] = q
            if k > 0:
                p.F[:, :16 * k] += (p.Wt[:, cols] - q) @ p.Lb[cols, :16 * k]
        if log and k % 32 == 0:
            log(f"  block {k}/{nb}")
    outs = []
    for p in P:
        mt = p.S.shape[0]
        qweight = wire.pack_states(p.S.reshape(-1, 256), K).reshape(mt, nb, 8 * K)
        W = wire.blk_had_cols_T(p.Q.T.contiguous()).T
        W = wire.blk_had_cols_T(W.contiguous())
        What = (W * p.sv[:, None] * p.su[None, :]).contiguous()
        outs.append(dict(qweight=qweight.cpu(), scales=p.rs.half().cpu(), su=wire.pack_signs(p.su).cpu(),
                         sv=wire.pack_signs(p.sv).cpu(), What=What, Q=p.Q))
    return outs
