"""HTR-W1 matrix encoder on MI355X: block-LDLQ error feedback around the tail-biting trellis search.

Same algorithm and call surface as htr/encode.py of the reference (encode_group, make_signs, prep_H, the VITERBI
hook, htr/encode.py:1-110): rotate W and the Hessian with the randomized Hadamard transform, factor the damped
Hessian, walk the 16-column blocks from the last to the first, search each block's 256-weight tiles with the trellis
Viterbi, and feed the quantization error of a block forward into the columns not yet encoded.  The search runs in
libhtr_gfx950.so (htr_viterbi, one workgroup per tile) when the tensors are on the GPU (a torch version of the same
formulation serves CPU tensors); the linear algebra around it is torch.  Results are HTR-W1 tensors plus the reconstruction `What`.
"""
import torch

from . import _native, wire

# callable(x[B, 256], w[B, 256], cb[65536], K) -> int64 states [B, 256]; None = the library's search on the GPU
VITERBI = None
# tiles per launch: bounds the backpointer scratch (tiles * 255 * (65536 >> K) bytes)
MAX_SCRATCH_BYTES = 1 << 30
_SCRATCH = {}
_CHECKED_CB = set()          # data pointers of codebook tensors already compared with the procedural codebook


def viterbi(x, w, cb=None, K=4, tailbite=True):
    """Tail-biting bitshift-trellis Viterbi on the GPU (htr.reference.viterbi / htr.vit_v2.viterbi of the reference).

    x, w: float32 [B, T <= 256] on a ROCm device.  cb is accepted for signature compatibility and must be the HTR
    codebook (the kernel evaluates it procedurally; another table is refused).  Returns int64 states [B, T].
    Costs that are NaN never win a comparison in the kernel, where torch.argmin in the reference returns the first NaN:
    inputs with NaN give different (meaningless either way) states.  CPU tensors take viterbi_cpu.
    """
    if not x.is_cuda:
        return viterbi_cpu(x, w, K, tailbite)                       # the reference falls back to its torch search too
    if cb is not None and cb.data_ptr() not in _CHECKED_CB:
        if cb.numel() != wire.S or not torch.equal(cb.detach().float().cpu().reshape(-1), wire.codebook_f32("cpu")):
            raise RuntimeError("viterbi: cb is not the HTR-W1 codebook; the GPU search evaluates that codebook only")
        _CHECKED_CB.add(cb.data_ptr())
    x = x.float().contiguous()
    w = w.float().contiguous()
    B, T = x.shape
    if w.shape != x.shape or not 1 <= T <= 256:
        raise RuntimeError("viterbi wants x and w of one shape [B, T <= 256]")
    L = _native.lib()
    per_tile = L.htr_viterbi_workspace_bytes(1, T, K)
    if per_tile == 0:
        raise RuntimeError(f"viterbi: unsupported K {K} (2..8)")
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


def viterbi_cpu(x, w, K=4, tailbite=True):
    """The same search with torch on the CPU, for tensors that are not on a GPU (the reference's fallback is its
    portable search, htr/reference.py:6-50; this is the formulation of the GPU kernel instead).  Per step only the
    minima over the 2^K predecessors are kept: M_t[low] = min_j cost_{t-1}[j Sj + low] with Sj = 65536 >> K, and
    cost_t[s] = M_t[s >> K] + w_t (x_t - cb[s])^2; arithmetic float32 and unfused, first index among equal values, two
    passes for tail-biting (free start, then start and end tied to the first pass's final low bits)."""
    x = x.float().contiguous()
    w = w.float().contiguous()
    B, T = x.shape
    if w.shape != x.shape or not 1 <= T <= 256 or not 2 <= K <= 8:
        raise RuntimeError("viterbi wants x and w of one shape [B, T <= 256] and K in 2..8")
    S, NB, SJ = wire.S, 1 << K, wire.S >> K
    cb = wire.codebook_f32("cpu")
    pred = torch.arange(S) >> K                                   # M entry that state s continues
    rows = torch.arange(B)
    j0 = None
    for constrained in ([False, True] if tailbite else [False]):
        M = torch.zeros(B, SJ)
        if constrained:
            M = torch.full((B, SJ), float("inf"))
            M[rows, j0] = 0.0
        back = torch.empty(B, max(T - 1, 0), SJ, dtype=torch.uint8)
        for t in range(T):
            d = x[:, t:t + 1] - cb[None, :]
            cost = M[:, pred] + w[:, t:t + 1] * (d * d)
            if t == T - 1:
                break
            M, arg = cost.view(B, NB, SJ).min(dim=1)              # over the top K bits j of s = j Sj + low
            back[:, t] = arg.to(torch.uint8)
        if constrained:
            cost = torch.where((torch.arange(S) & (SJ - 1))[None, :] == j0[:, None], cost, torch.full_like(cost, float("inf")))
        cost = torch.where(torch.isnan(cost), torch.full_like(cost, float("inf")), cost)       # NaN never wins, as in the kernel
        final = cost.argmin(dim=1)
        final = torch.where(torch.isinf(cost[rows, final]), torch.zeros_like(final), final)
        j0 = final & (SJ - 1)
    states = torch.empty(B, T, dtype=torch.int64)
    s_t = final
    states[:, T - 1] = s_t
    for t in range(T - 1, 0, -1):
        low = s_t >> K
        s_t = back[rows, t - 1, low].long() * SJ + low
        states[:, t - 1] = s_t
    return states


def block_rotate(W, bs=wire.RHT_BLOCK):
    """Blocks of bs columns times H^T (H is symmetric; htr/encode.py:15-17)."""
    m, n = W.shape
    return (W.reshape(m, n // bs, bs) @ wire.hadamard(bs, W.device).T).reshape(m, n)


def _rotate_both_sides(A, row_signs, col_signs):
    """diag(row_signs) A diag(col_signs) with the blockwise Hadamard applied to its columns, then to its rows."""
    B = block_rotate(A * row_signs[:, None] * col_signs[None, :])
    return block_rotate(B.T.contiguous()).T


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
    (htr/encode.py:35-42).  float64.  The order of these float64 operations (dead columns first, then the damping added
    to the whole matrix as damp * mean * I) is kept as the reference has it: the encoder's fixture is matched bit for
    bit, and damping the diagonal in place, or before the dead columns are fixed, rounds differently."""
    H = H.clone().double()
    dead = torch.diag(H) == 0
    H[dead, dead] = 1.0
    W = W.clone()
    W[:, dead] = 0
    H += damp * torch.diag(H).mean() * torch.eye(H.shape[0], device=H.device, dtype=H.dtype)
    return H, W


def _feedback_factor(Hd):
    """Block LDL feedback matrix of a damped, rotated Hessian (float64 in, float32 out): the Cholesky factor with every
    16-column block normalised by its own 16x16 diagonal block (htr/encode.py:64-67)."""
    n = Hd.shape[0]
    nb = n // 16
    C = torch.linalg.cholesky(Hd)
    diag_blocks = C.view(nb, 16, nb, 16).diagonal(dim1=0, dim2=2).permute(2, 0, 1)
    return torch.einsum("ikj,kjl->ikl", C.view(n, nb, 16), torch.linalg.inv(diag_blocks)).reshape(n, n).float()


class _Group:
    """The matrices of one input group in the rotated basis, stacked along the rows: every 16-column block of the whole
    group is one batch of 256-weight tiles for the search (one workgroup per tile on the GPU), and matrices that came
    with the same Hessian (gate and up of an expert, q / k / v of a layer) share one factorisation and one feedback
    product."""

    def __init__(self, jobs, seed, shared_su, damp):
        n = jobs[0]["W"].shape[1]
        if n % 128:
            raise RuntimeError("encode_group: n must be a multiple of 128")
        self.n, self.nb = n, n // 16
        dev = jobs[0]["W"].device
        self.signs, self.rows = [], []            # (su, sv) and the row range of every matrix in the stack
        self.factors = []                         # [first row, last row, feedback matrix]: consecutive matrices of one Hessian
        Wt, seen = [], {}
        r0 = 0
        for index, jb in enumerate(jobs):
            W = jb["W"].float()
            m = W.shape[0]
            if m % 128 or W.shape[1] != n:
                raise RuntimeError("encode_group: every matrix needs m % 128 == 0 and the group's n")
            su, sv = (s.to(W.device) for s in make_signs(n, m, seed, index, shared_su))
            Hr = _rotate_both_sides(jb["H"].float().to(W.device), su, su).contiguous()
            Hd, Wr = prep_H(Hr, _rotate_both_sides(W, sv, su).contiguous(), damp)
            Wt.append(Wr.float())
            # the damped Hessian depends on (H, su) only: the same H object under a shared su is factored once
            key = id(jb["H"]) if shared_su else None
            if key is not None and key in seen and self.factors[-1][2] is seen[key]:
                self.factors[-1][1] = r0 + m
            else:
                Lb = seen.get(key) if key is not None else None
                if Lb is None:
                    Lb = _feedback_factor(Hd)
                    if key is not None:
                        seen[key] = Lb
                self.factors.append([r0, r0 + m, Lb])
            self.signs.append((su, sv))
            self.rows.append((r0, r0 + m))
            r0 += m
        self.Wt = torch.cat(Wt)
        self.rs = self.Wt.pow(2).mean(dim=1).sqrt().half().float().clamp(min=1e-8)      # row scales, as stored (fp16)
        self.Q = torch.zeros_like(self.Wt)
        self.F = torch.zeros_like(self.Wt)                                              # error fed forward
        self.S = torch.zeros((r0 // 16, self.nb, 256), dtype=torch.int64, device=dev)
        # search weights: the squared row scales of a tile's 16 rows, normalised to mean 1 per tile; the same for every block
        wg = (self.rs[:, None] ** 2).expand(-1, 16).contiguous().reshape(-1, 256)
        self.wg = wg / wg.mean(dim=1, keepdim=True)


@torch.no_grad()
def encode_group(jobs, K, seed=1234, shared_su=True, damp=0.01, max_batch=1024, log=None):
    """jobs: list of dict(W=[m, n], H=[n, n]) sharing n.  Returns a list of dict(qweight, scales, su, sv, What, Q)
    (htr/encode.py:45-110): block LDLQ from the last 16-column block to the first, each block's tiles quantized by the
    trellis search against the row scales, the block's error fed forward through the feedback matrix."""
    search = VITERBI or (lambda x, w, cb, k: viterbi(x, w, cb, k))
    G = _Group(jobs, seed, shared_su, damp)
    cb = wire.codebook_f32(G.Wt.device)
    ntiles = G.wg.shape[0]
    for k in range(G.nb - 1, -1, -1):
        cols = slice(16 * k, 16 * k + 16)
        target = ((G.Wt[:, cols] + G.F[:, cols]) / G.rs[:, None]).reshape(-1, 256)
        for b0 in range(0, ntiles, max_batch):
            G.S[b0:b0 + max_batch, k] = search(target[b0:b0 + max_batch].contiguous(), G.wg[b0:b0 + max_batch].contiguous(), cb, K)
        q = cb[G.S[:, k]].reshape(-1, 16) * G.rs[:, None]
        G.Q[:, cols] = q
        if k > 0:
            err = G.Wt[:, cols] - q
            for first, last, Lb in G.factors:
                G.F[first:last, :16 * k] += err[first:last] @ Lb[cols, :16 * k]
        if log and k % 32 == 0:
            log(f"  block {k}/{G.nb}")
    outs = []
    for (first, last), (su, sv) in zip(G.rows, G.signs):
        Q = G.Q[first:last]
        S = G.S[first // 16:last // 16]
        qweight = wire.pack_states(S.reshape(-1, 256), K).reshape(S.shape[0], G.nb, 8 * K)
        W = wire.blk_had_cols_T(wire.blk_had_cols_T(Q.T.contiguous()).T.contiguous())
        What = (W * sv[:, None] * su[None, :]).contiguous()
        outs.append(dict(qweight=qweight.cpu(), scales=G.rs[first:last].half().cpu(), su=wire.pack_signs(su).cpu(),
                         sv=wire.pack_signs(sv).cpu(), What=What, Q=Q))
    return outs
