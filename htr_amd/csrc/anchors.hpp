// Part of htr_gfx950.hip, included inside its anonymous namespace: timing anchors of the fused linear (measurement only).
// ------------------------------------------------------------------------------------------------ timing anchors
// Measurement only: what a launch would cost if it did nothing but read its bytes, and what the decode costs on
// register data.  Neither produces results.

// The weight stream of k_linear and nothing else: same chunks, same descriptors, same order and depth of loads; every
// loaded word is folded into one register so that the loads cannot be dropped.
template <int K, int P>
__global__ __launch_bounds__(WG_THREADS) void k_anchor_read(const uint32_t* __restrict__ qw, int m, int n, int chunk, int flags,
                                                            unsigned long long nblk_magic, uint32_t* __restrict__ sink) {
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int nblk = n >> 7, vtotal = (m >> 7) * nblk;
  int cid = (int)blockIdx.x;
  if (flags & FLAG_LANES) cid = ((int)blockIdx.x & 7) * (flags >> FLAG_LANE_LEN_SHIFT) + ((int)blockIdx.x >> 3);
  const int v0 = cid * chunk, nsteps = min(vtotal, v0 + chunk) - v0;
  auto div_nblk = [&](int v) { return (int)(((unsigned long long)(unsigned)v * nblk_magic) >> 40); };
  const int rb_first = div_nblk(v0), c0 = v0 - rb_first * nblk;
  const int last_wraps = div_nblk(c0 + nsteps - 1);
  constexpr int STEP_BYTES = 256 * K;
  const uint32_t strip_bytes = (uint32_t)nblk * STEP_BYTES;
  const uint32_t* wave_base = qw + ((size_t)(rb_first * 8 + w) * nblk + (size_t)c0) * (STEP_BYTES / 4);
  const uint32_t extent = (uint32_t)nsteps * STEP_BYTES + (uint32_t)last_wraps * 7u * strip_bytes;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)wave_base, 0, (int)extent, 0x00020000);
  const int lane_off = lane * 4 * K;
  int pf_off = 0, pf_blk = c0;
  StreamRegs<K> buf[P];
  auto prefetch = [&](StreamRegs<K>& dst) {
    HTR_PIN();
    load_stream_buffer<K>(rsrc, lane_off + pf_off, dst);
    const bool wrap = pf_blk == nblk - 1;
    pf_off += STEP_BYTES + (wrap ? 7 * (int)strip_bytes : 0);
    pf_blk = wrap ? 0 : pf_blk + 1;
    HTR_PIN();
  };
#pragma unroll
  for (int p = 0; p < P; ++p) prefetch(buf[p]);
  uint32_t acc = 0u;
  for (int v = 0; v < nsteps; v += P) {
#pragma unroll
    for (int pp = 0; pp < P; ++pp) {
#pragma unroll
      for (int k = 0; k < K; ++k) acc ^= buf[pp].d[k];
      prefetch(buf[pp]);
    }
  }
  if (acc == 0x9E3779B9u && sink != nullptr) sink[0] = acc;      // practically never: keeps the loads alive
}

// The decode of k_linear's inner loop on register data, `iters` wave-steps per wave, timed with the shader clock
// (s_memtime) and the 100 MHz reference clock (s_memrealtime) around the loop.  WITH_MFMA adds the four matrix
// instructions of a step (constant B operands).  out[wave] = {shader cycles, reference ticks}.
template <int K, bool WITH_MFMA>
__global__ __launch_bounds__(WG_THREADS) void k_anchor_decode(int iters, unsigned long long* __restrict__ out, float* __restrict__ sink) {
  const int lane = threadIdx.x & 63;      // (the launch requests dynamic LDS it never touches: one workgroup per compute unit)
  const int hist = history_lane_byteaddr(lane);
  StreamRegs<K> r;
#pragma unroll
  for (int k = 0; k < K; ++k) r.d[k] = (uint32_t)(threadIdx.x * 2654435761u) ^ (uint32_t)(k * 40503u + blockIdx.x);
  h8 b0, b1;
#pragma unroll
  for (int i = 0; i < 8; ++i) { b0[i] = (_Float16)(0.25f + (float)((lane + i) & 3)); b1[i] = (_Float16)(0.5f - (float)((lane ^ i) & 1)); }
  f4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
  DecodedStep<K> d;
  __syncthreads();
  const unsigned long long c0 = __builtin_amdgcn_s_memtime(), t0 = __builtin_amdgcn_s_memrealtime();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int k = 0; k < K; ++k) asm volatile("" : "+v"(r.d[k]));          // opaque: the decode cannot be hoisted out of the loop
    decode_step<K>(r, hist, d);
    if constexpr (WITH_MFMA) {
      acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[0], b0, acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[2], b0, acc1, 0, 0, 0);
      acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[1], b1, acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[3], b1, acc1, 0, 0, 0);
    } else {
#pragma unroll
      for (int k = 0; k < 4; ++k) asm volatile("" : : "v"(d.a[k]));         // used: the decode cannot be dropped
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  if constexpr (WITH_MFMA) { asm volatile("" : "+v"(acc0)); asm volatile("" : "+v"(acc1)); }
  const unsigned long long c1 = __builtin_amdgcn_s_memtime(), t1 = __builtin_amdgcn_s_memrealtime();
  if (lane == 0) {
    const size_t wv = (size_t)blockIdx.x * WG_WAVES + (threadIdx.x >> 6);
    out[2 * wv] = c1 - c0;
    out[2 * wv + 1] = t1 - t0;
  }
  if constexpr (WITH_MFMA) { if (acc0.x + acc1.y == 12345.678f && sink != nullptr) sink[0] = acc0.x; }
}

