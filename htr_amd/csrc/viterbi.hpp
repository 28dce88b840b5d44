// Part of htr_gfx950.hip, included inside its anonymous namespace: k_viterbi: the encoder's trellis search.
// ------------------------------------------------------------------------------------------------ encoder search
// Tail-biting bitshift-trellis Viterbi over the 65536 codec states (htr/reference.py:6-50 of the reference; its GPU
// versions are htr/vit_v1.py and htr/vit_v2.py): per 256-weight tile, minimise sum_t w_t (x_t - cb[s_t])^2 with
// s_t = ((s_{t-1} << K) & 0xFFFF) | bits.  One workgroup per tile.  Only the minima over the 2^K predecessors,
// M_t[low] = min_j cost_{t-1}[j * Sj + low] (Sj = 65536 >> K entries), need to live between steps, and
// cost_t[s] = M_t[s >> K] + w_t (x_t - cb[s])^2, so two M arrays in LDS carry a whole tile (128 KB at K2, 32 KB at K4)
// and no cost array ever goes to memory.  The value of a state is the procedural codebook, cb[s] = f32(v(s) / rms) with
// 1021 distinct v, so a step's 65536 penalty terms are 1021 distinct numbers: they are computed once per step into an
// LDS table that every candidate indexes with v(s) (two integer instructions).
// Backpointers (one byte per M entry and step) go to global memory during the deciding pass only; thread 0 walks
// them back.  Arithmetic and tie-breaking are the reference's: float32, d = (x - cb)^2, m + w * d without fusing,
// the first index among equal values in every min / argmin.
template <int K> struct VitCfg {
  static constexpr int NB = 1 << K, SJ = 65536 >> K;
  static constexpr int THREADS = K == 2 ? 1024 : (K == 8 ? 256 : 512);   // at most one thread per M entry
  static constexpr int ITEMS = SJ / THREADS;         // M entries per thread
};

template <int K>
__global__ __launch_bounds__(VitCfg<K>::THREADS) void k_viterbi(const float* __restrict__ x, const float* __restrict__ w, int T,
                                                               int tailbite, uint8_t* __restrict__ bps, uint16_t* __restrict__ states,
                                                               double rms) {
  using C = VitCfg<K>;
  constexpr int NB = C::NB, SJ = C::SJ, THREADS = C::THREADS, ITEMS = C::ITEMS;
  extern __shared__ __align__(16) unsigned char lds[];
  float* M0 = (float*)lds;                 // [SJ]
  float* M1 = M0 + SJ;                     // [SJ]
  float* tl = M1 + SJ;                     // [2][1024] penalty of each v for the current / next step
  float* cbv = tl + 2048;                  // [1024] codebook value of each v
  float* xs = cbv + 1024;                  // [T] targets, then [T] weights (T <= 256)
  float* ws = xs + 256;
  float* red_v = ws + 256;                 // [32] reduction scratch
  uint32_t* red_i = (uint32_t*)(red_v + 32);
  const int tid = threadIdx.x;
  const size_t tile = blockIdx.x;
  const float* xg = x + tile * T;
  const float* wg = w + tile * T;
  uint8_t* bp = bps + tile * (size_t)(T - 1) * SJ;

  for (int i = tid; i < 1024; i += THREADS) cbv[i] = i <= 1020 ? (float)((double)(i - 510) / rms) : 0.f;
  for (int i = tid; i < T; i += THREADS) { xs[i] = xg[i]; ws[i] = wg[i]; }
  // table index v + 510 of state s: two integer instructions, cheaper to recompute than to keep
  auto vidx = [&](uint32_t s) { return __builtin_amdgcn_sad_u8(s * GEN_A + GEN_B, 0u, 0u); };
  __syncthreads();
  auto fill_terms = [&](int t, float* dst) {          // dst[v] = w_t * (x_t - cb(v))^2, unfused
    const float xt = xs[t], wt = ws[t];
    for (int i = tid; i < 1024; i += THREADS) {
      const float diff = __fsub_rn(xt, cbv[i]);
      dst[i] = __fmul_rn(wt, __fmul_rn(diff, diff));
    }
  };

  uint32_t j0 = 0;
  const int passes = tailbite ? 2 : 1;
  uint32_t final_state = 0;
  for (int pass = 0; pass < passes; ++pass) {
    const bool constrained = pass == 1;               // second pass: start and end tied to j0
    const bool record = pass == passes - 1;
    // cost_0[s] = M_0[s >> K] + term_0(s) with M_0 = 0 (free start) or 0 at j0 and infinity elsewhere
    for (int i = tid; i < SJ; i += THREADS) M0[i] = (!constrained || (uint32_t)i == j0) ? 0.f : __builtin_inff();
    fill_terms(0, tl);
    __syncthreads();
    float* Mold = M0;
    float* Mnew = M1;
    for (int t = 0; t < T - 1; ++t) {
      const float* tcur = tl + (t & 1) * 1024;
      fill_terms(t + 1, tl + ((t + 1) & 1) * 1024);   // the next step's table, behind this step's barrier
#pragma unroll 1
      for (int i = 0; i < ITEMS; ++i) {
        const int low = tid + i * THREADS;
        float best = 0.f;
        uint32_t bj = 0;
#pragma unroll 8
        for (int j = 0; j < NB; ++j) {
          // state s = j * SJ + low; its own predecessor minimum is M[s >> K]
          const float c = __fadd_rn(Mold[j * (SJ / NB) + (low >> K)], tcur[vidx((uint32_t)j * SJ + (uint32_t)low)]);
          if (j == 0 || c < best) { best = c; bj = j; }
        }
        Mnew[low] = best;
        if (record) bp[(size_t)t * SJ + low] = (uint8_t)bj;
      }
      __syncthreads();
      float* tmp = Mold; Mold = Mnew; Mnew = tmp;
    }
    // last step: argmin over all states of cost_{T-1}, first index among equals; second pass: only states whose
    // lower part is j0
    const float* tcur = tl + ((T - 1) & 1) * 1024;
    float best = __builtin_inff();
    uint32_t bs = 0xFFFFFFFFu;
#pragma unroll 1
    for (int i = 0; i < ITEMS; ++i) {
      const int low = tid + i * THREADS;
#pragma unroll 8
      for (int j = 0; j < NB; ++j) {
        const uint32_t s = (uint32_t)j * SJ + (uint32_t)low;
        float c = __fadd_rn(Mold[j * (SJ / NB) + (low >> K)], tcur[vidx(s)]);
        if (constrained && (uint32_t)low != j0) c = __builtin_inff();
        if (c < best || (c == best && s < bs)) { best = c; bs = s; }
      }
    }
    // wave, then workgroup reduction of (value, index)
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(best, off);
      const uint32_t oi = (uint32_t)__shfl_xor((int)bs, off);
      if (ov < best || (ov == best && oi < bs)) { best = ov; bs = oi; }
    }
    __syncthreads();
    if ((tid & 63) == 0) { red_v[tid >> 6] = best; red_i[tid >> 6] = bs; }
    __syncthreads();
    if (tid == 0) {
      float b = red_v[0]; uint32_t bi = red_i[0];
      for (int k = 1; k < THREADS / 64; ++k)
        if (red_v[k] < b || (red_v[k] == b && red_i[k] < bi)) { b = red_v[k]; bi = red_i[k]; }
      red_i[0] = bi == 0xFFFFFFFFu ? 0u : bi;         // every cost infinite or NaN: the reference's argmin gives 0
    }
    __syncthreads();
    final_state = red_i[0];
    j0 = final_state & (SJ - 1);
    __syncthreads();
  }
  // trace back (htr/reference.py:43-49): the backpointers of this tile were written by this workgroup; make them
  // visible to the reading thread
  __threadfence();
  __syncthreads();
  if (tid == 0) {
    uint16_t* st = states + tile * T;
    uint32_t s = final_state;
    st[T - 1] = (uint16_t)s;
    for (int t = T - 1; t > 0; --t) {
      const uint32_t low = s >> K;
      const uint32_t top = bp[(size_t)(t - 1) * SJ + low];
      s = top * SJ + low;
      st[t - 1] = (uint16_t)s;
    }
  }
}

