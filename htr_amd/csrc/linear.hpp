// Part of htr_gfx950.hip, included inside its anonymous namespace: k_rotate, k_rotate_mfma and k_linear: the fused packed linear for 1 to 8 activation rows (and grouped launches).
// ------------------------------------------------------------------------------------------------ fused linear
// The step space of one linear is (128-row block rb, 128-column block blk), row-major: virtual step v = rb * nblk + blk.
// It is cut into equal contiguous chunks, one per workgroup, so the workgroup count can be a multiple of the CU count
// whatever the shape.  A chunk may end inside a row block and continue in the next one; each piece of a row block a
// chunk covers is a "segment" and yields one partial.  The workgroup whose chunk holds the LAST step of a row block
// finishes that block: it adds the partials of the chunks before it (which can only concern its first segment) to
// its own and applies the output side.  Every other segment of a chunk is complete by itself; only a chunk's last
// segment can be a contribution to a later chunk's row block, so one partial slot per workgroup is enough.

// arguments the kernel needs late (epilogue) or only on the pre-rotated path
struct LinearTail {
  const uint16_t* scales;
  const uint8_t* sv;
  const void* bias;
  void* y;
  const _Float16* xt_g;   // pre-rotated activations [M][n] f16 (only when PREROT)
  const float* xs_g;      // their sums per (row, block) [M][n/128][4]: even tiles, odd tiles, columns 0..63, columns 64..127
  const float* sc_g;      // per-row activation scale [M]
  float* tiles;           // GEMM kernel: one 128 x 128 float tile per workgroup for the exchange between column splits
  uint32_t* status;       // workspace word that collects kernel-side failures (bit 0: a finisher gave up waiting)
  unsigned long long chunk_magic;   // ceil(2^40 / chunk): step index -> chunk index
  float cbscale;
  int spin_limit;         // polls of the contributors' slots before a finisher gives up
  // grouped launch (blockIdx.y = problem): per-problem pointers and row counts come from this device table, the
  // pre-rotated activations and the partial slots of problem p start p strides into their regions
  const htr_group_entry* group;
  unsigned long long group_prerot_stride;   // bytes
  unsigned long long group_part_stride;     // floats
};

constexpr int ROT_PAIRS = 32;      // (activation row, 128-column block) pairs a workgroup rotates in one pass: four per wave
constexpr int MAX_ROT_PASSES = 4;  // passes of the kernel variant for up to 8 rows over long chunks
constexpr int MAX_ROT_PAIRS = ROT_PAIRS * MAX_ROT_PASSES;

// LDS layout (dynamic): [xt: (M + 1) rows x row_halves f16][xs: M * nbl * 2 f32 (per tile parity)][sc: M f32][bs: 128 f32, scale per pair]
//                       [fin: segfin x M x 128 f32, partials of the row blocks this workgroup finishes]
// nbl = number of distinct column blocks a chunk touches = min(chunk, n / 128)
// One rotated 128-column block is stored as [columns 0..7 of tiles 0..7][columns 8..15 of tiles 0..7] (2 x 64 halves), and
// rows are padded by 16 halves: the 16-byte B-operand reads of 8 consecutive lanes (4 activation rows x 2 tile parities)
// then cover 128 contiguous-mod-128 bytes, i.e. every LDS bank once.
__host__ __device__ inline int xt_row_halves(int nbl) { return nbl * 128 + 16; }
__device__ __forceinline__ int xt_slot(int j) { return ((j >> 3) & 1) * 64 + (j >> 4) * 8 + (j & 7); }   // element j of a block
__host__ __device__ inline size_t lds_fin_offset(int M, int nbl) {
  return ((size_t)(M + 1) * xt_row_halves(nbl) * 2 + (size_t)M * nbl * 4 * 2 + (size_t)M * 4 + MAX_ROT_PAIRS * 4 + 15) / 16 * 16;
}
__host__ __device__ inline size_t lds_bytes(int M, int nbl, int segfin) {
  return lds_fin_offset(M, nbl) + (size_t)segfin * M * 128 * 4;
}

// power-of-two activation scale 2^e with sqrt(128) * amax / 2^e in (8192, 16384]: |H128 x| / sqrt(128) <= sqrt(128) * max|x|,
// so the rotated activations neither overflow f16 nor fall into its denormals
__device__ __forceinline__ int scale_exponent(float amax) {
  const int ex = (int)((__float_as_uint(amax * SQRT128) >> 23) & 0xFFu);
  if (ex == 0 || ex == 255) return 0;
  return max(-100, ex - 127 - 13);
}
__device__ __forceinline__ float pow2f(int e) { return __uint_as_float((uint32_t)(127 + e) << 23); }
// Scale exponent of one rotated 128-column block from the bit pattern of its largest |value| (after the 1/sqrt(128)):
// 0 while that lies in [2^-8, 2^15) -- no f16 overflow, and values down to 2^-6 of the largest stay normal -- else the
// exponent that brings it to [2^13, 2^14).  Zero, denormal, infinite and NaN maxima keep scale 1.
__device__ __forceinline__ int block_scale_exponent(uint32_t amax_bits) {
  const int ex = (int)((amax_bits >> 23) & 0xFFu);
  if (ex == 0 || ex == 255) return 0;
  const int l2 = ex - 127;
  if (l2 >= -8 && l2 <= 14) return 0;
  return max(-100, l2 - 13);
}

// ---- rotation of four 128-element blocks on the matrix unit: H128 = H4 (x) H32 over the element index i = 32 a + c, so
// a block is a 4 x 32 matrix X and H128 x = H4 . X . H32 (unnormalised).  The four blocks of a wave are the 16 rows
// (block p, a) of one MFMA A operand: lane (k-group gk = lane / 16, row = lane % 16 = 4 p + a) brings the 8
// consecutive 16-bit elements 32 a + 8 gk .. + 7 of block p (xr) and the su byte that holds their signs (sb).  The
// products are exact (operands are the activations themselves and +-1), accumulated in float32.  Result: lane
// (p = lane / 16, j = lane % 16) holds y[h][a'] = element 32 a' + 16 h + j of block p.
__device__ __forceinline__ void rotate4_mfma(const u4& xr, uint32_t sb, bool is_bf16, int lane, float (&y)[2][4]) {
  uint32_t xs4[4] = {xr.x, xr.y, xr.z, xr.w};
#pragma unroll
  for (int d = 0; d < 4; ++d)                                    // elements 2d (low half), 2d + 1 (high half): su bits 2d, 2d + 1
    xs4[d] ^= ((sb << (15 - 2 * d)) & 0x8000u) | ((sb << (30 - 2 * d)) & 0x80000000u);
  // B operand: H32[k][c'] = (-1)^popcount(k & c') for k = 8 gk + i (dword d holds i = 2d, 2d + 1) and
  // c' = 16 h + j, j = lane % 16; as 16-bit ones with the sign bit set where the parity is odd
  const int j = lane & 15, gk = lane >> 4;
  const uint32_t one2 = is_bf16 ? 0x3F803F80u : 0x3C003C00u;
  const uint32_t o1 = (j & 1) ? 0x80000000u : 0u;
  const uint32_t e1 = (j & 2) ? 0x80008000u : 0u;
  const uint32_t e2 = (j & 4) ? 0x80008000u : 0u;
  const uint32_t f3 = ((gk & 1) && (j & 8)) ? 0x80008000u : 0u;   // k bit 3 with c' bit 3
  const uint32_t f4m = (gk & 2) ? 0x80008000u : 0u;               // k bit 4 with c' bit 4 (h = 1)
  const uint32_t b0 = one2 ^ o1 ^ f3;
  const u4 hb0 = {b0, b0 ^ e1, b0 ^ e2, b0 ^ e1 ^ e2};
  const u4 hb1 = {hb0.x ^ f4m, hb0.y ^ f4m, hb0.z ^ f4m, hb0.w ^ f4m};
  const u4 xa = {xs4[0], xs4[1], xs4[2], xs4[3]};
  const f4 zero4 = {0.f, 0.f, 0.f, 0.f};
  f4 t0, t1;
  if (is_bf16) {
    t0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8, xa), __builtin_bit_cast(b8, hb0), zero4, 0, 0, 0);
    t1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8, xa), __builtin_bit_cast(b8, hb1), zero4, 0, 0, 0);
  } else {
    t0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, xa), __builtin_bit_cast(h8, hb0), zero4, 0, 0, 0);
    t1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(h8, xa), __builtin_bit_cast(h8, hb1), zero4, 0, 0, 0);
  }
  // D: lane (p = lane / 16, j), register a: T[p][a][16 h + j].  H4 over a gives element 32 a' + 16 h + j.
  const float u0 = t0.x + t0.y, u1 = t0.x - t0.y, u2 = t0.z + t0.w, u3 = t0.z - t0.w;
  y[0][0] = u0 + u2; y[0][1] = u1 + u3; y[0][2] = u0 - u2; y[0][3] = u1 - u3;
  const float w0 = t1.x + t1.y, w1 = t1.x - t1.y, w2 = t1.z + t1.w, w3 = t1.z - t1.w;
  y[1][0] = w0 + w2; y[1][1] = w1 + w3; y[1][2] = w0 - w2; y[1][3] = w1 - w3;
}

// Rotation of all activation rows ahead of the linear kernel (used where every workgroup rotating its own column
// blocks would repeat too much work, and for float32 activations).  Workgroup (g, row) rotates column blocks
// 8g .. 8g + 7 of one activation row, one block per wave; every workgroup scans the whole row for max|x| itself
// (n / 512 loads per thread), which is cheaper than a second launch or an exchange between workgroups.
__global__ __launch_bounds__(WG_THREADS) void k_rotate(const void* __restrict__ x, const uint8_t* __restrict__ su, int n, int x_dtype,
                                                       _Float16* __restrict__ xt_g, float* __restrict__ xs_g, float* __restrict__ sc_g,
                                                       const htr_group_entry* __restrict__ group, unsigned long long group_stride) {
  __shared__ float s_max[WG_WAVES];
  if (group != nullptr) {                  // grouped: blockIdx.z = problem, outputs shifted by the problem's stride
    const htr_group_entry& ge = group[blockIdx.z];
    if ((int)blockIdx.y >= ge.M) return;
    x = ge.x; su = (const uint8_t*)ge.su;
    const size_t shift = (size_t)blockIdx.z * group_stride;
    xt_g = (_Float16*)((unsigned char*)xt_g + shift);
    xs_g = (float*)((unsigned char*)xs_g + shift);
    sc_g = (float*)((unsigned char*)sc_g + shift);
  }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, mrow = blockIdx.y, nblk = n >> 7;
  const size_t row = (size_t)mrow * n;
  const int blk = blockIdx.x * WG_WAVES + w;
  const int col = blk * 128;
  // Every load of the kernel goes out back to back, through descriptors over the activation row and the sign bytes:
  // the wave's own block first (per element one 16-bit and one 32-bit load, the one that does not apply out of range:
  // zeros, no traffic, no branch), then the scan of the whole row for max|x|.  Conversions come after the last load
  // has been issued; a conversion between two loads makes the compiler wait for the first to return.
  const bool is32 = x_dtype == HTR_F32, own = blk < nblk;
  const int es = is32 ? 4 : 2;
  const unsigned char* xrow = (const unsigned char*)x + row * es;
  const __amdgpu_buffer_rsrc_t rrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)xrow, 0, n * es, 0x00020000);
  const __amdgpu_buffer_rsrc_t srsrc = __builtin_amdgcn_make_buffer_rsrc((void*)su, 0, n >> 3, 0x00020000);
  constexpr int OUT_OF_RANGE = 0x7FFFFF00;
  const int ea = col + lane, eb = ea + 64;
  const uint32_t a16 = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rrsrc, own && !is32 ? ea * 2 : OUT_OF_RANGE, 0, 0);
  const uint32_t b16 = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rrsrc, own && !is32 ? eb * 2 : OUT_OF_RANGE, 0, 0);
  const uint32_t a32 = __builtin_amdgcn_raw_buffer_load_b32(rrsrc, own && is32 ? ea * 4 : OUT_OF_RANGE, 0, 0);
  const uint32_t b32 = __builtin_amdgcn_raw_buffer_load_b32(rrsrc, own && is32 ? eb * 4 : OUT_OF_RANGE, 0, 0);
  const uint32_t sa = (uint8_t)__builtin_amdgcn_raw_buffer_load_b8(srsrc, own ? ea >> 3 : OUT_OF_RANGE, 0, 0);
  const uint32_t sb = (uint8_t)__builtin_amdgcn_raw_buffer_load_b8(srsrc, own ? eb >> 3 : OUT_OF_RANGE, 0, 0);
  // max|x| of the row.  |values| compare like their bit patterns, so the scan is integer: 16 bytes per thread and load
  // (pieces beyond the row's end read zeros), four loads in flight per thread.  Rows that are not 16-byte aligned are
  // scanned element by element.
  uint32_t m32 = 0u;            // float32: max of the sign-cleared words; 16-bit types: max of the sign-cleared halves
  if ((((size_t)xrow) & 15) == 0) {
    for (int base = threadIdx.x * 16; base < n * es; base += 4 * WG_THREADS * 16) {
      u4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = __builtin_amdgcn_raw_buffer_load_b128(rrsrc, base + u * WG_THREADS * 16, 0, 0);
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const uint32_t d[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          if (is32) m32 = max(m32, d[k] & 0x7FFFFFFFu);
          else m32 = max(m32, max(d[k] & 0x7FFFu, (d[k] >> 16) & 0x7FFFu));
        }
      }
    }
  } else if (is32) {
    for (int i = threadIdx.x; i < n; i += WG_THREADS)
      m32 = max(m32, (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rrsrc, i * 4, 0, 0) & 0x7FFFFFFFu);
  } else {
    for (int i = threadIdx.x; i < n; i += WG_THREADS)
      m32 = max(m32, (uint32_t)(uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rrsrc, i * 2, 0, 0) & 0x7FFFu);
  }
  float mx = is32 ? __uint_as_float(m32) : x_dtype == HTR_BF16 ? bf16_bits_to_float((uint16_t)m32) : f16_bits_to_float((uint16_t)m32);
  if (mx != mx) mx = __uint_as_float(0x7F800000u);     // a NaN anywhere: treat the row as unbounded (scale 1)
  // own elements: bits to float, input sign (bit j % 8 of byte j / 8 set: minus)
  uint32_t abits = is32 ? a32 : x_dtype == HTR_BF16 ? a16 << 16 : __float_as_uint(f16_bits_to_float((uint16_t)a16));
  uint32_t bbits = is32 ? b32 : x_dtype == HTR_BF16 ? b16 << 16 : __float_as_uint(f16_bits_to_float((uint16_t)b16));
  abits ^= ((sa >> (ea & 7)) & 1u) << 31;
  bbits ^= ((sb >> (eb & 7)) & 1u) << 31;
  float va = __uint_as_float(abits), vb = __uint_as_float(bbits);
  mx = wave_max(mx);
  if (lane == 0) s_max[w] = mx;
  __syncthreads();
  float amax = 0.f;
#pragma unroll
  for (int k = 0; k < WG_WAVES; ++k) amax = fmaxf(amax, s_max[k]);
  const int e = scale_exponent(amax);
  const float inv_sc = pow2f(-e);
  if (threadIdx.x == 0 && blockIdx.x == 0) sc_g[mrow] = pow2f(e);
  if (blk < nblk) {
    va *= inv_sc; vb *= inv_sc;
    fwht128_wave(va, vb, lane);
    const _Float16 ha = (_Float16)(va * INV_SQRT128), hb = (_Float16)(vb * INV_SQRT128);
    xt_g[row + col + lane] = ha;
    xt_g[row + col + lane + 64] = hb;
    // sums of the rounded values: the lane's first element lies in tile lane / 16, its second in tile 4 + lane / 16, so the
    // 16-lane row parity is the tile parity of both, and the two elements are the two halves of the block
    float ea, oa, eb, ob;
    wave_sum_by_row_parity((float)ha, ea, oa);
    wave_sum_by_row_parity((float)hb, eb, ob);
    if (lane == 0) *(f4*)(xs_g + ((size_t)mrow * nblk + blk) * 4) = f4{ea + eb, oa + ob, ea + oa, eb + ob};
  }
}

// The same for 16-bit activations whose rows start on 16-byte boundaries, on the matrix unit (rotate4_mfma): a wave
// rotates four blocks, a workgroup 32 blocks of one activation row; grid = (blocks / 32 rounded up, rows).  About a
// seventh of the vector instructions of the butterfly version per block, which shows where the rotation is not just
// latency: 128 rows of 14336 columns take 8.6 us there.
__global__ __launch_bounds__(WG_THREADS) void k_rotate_mfma(const void* __restrict__ x, const uint8_t* __restrict__ su, int n, int is_bf16,
                                                            _Float16* __restrict__ xt_g, float* __restrict__ xs_g, float* __restrict__ sc_g) {
  __shared__ uint32_t s_amax[WG_WAVES];
  const int lane = threadIdx.x & 63, w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int mrow = blockIdx.y, nblk = n >> 7;
  const int b0 = blockIdx.x * 4 * WG_WAVES + 4 * w;        // first of this wave's four blocks
  const int gk = lane >> 4, j = lane & 15;
  const unsigned char* xrow = (const unsigned char*)x + (size_t)mrow * n * 2;
  const __amdgpu_buffer_rsrc_t rrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)xrow, 0, n * 2, 0x00020000);
  const __amdgpu_buffer_rsrc_t srsrc = __builtin_amdgcn_make_buffer_rsrc((void*)su, 0, n >> 3, 0x00020000);
  constexpr int OUT_OF_RANGE = 0x7FFFFF00;
  // own elements first (lane (gk, row = 4 p + a) brings elements 32 a + 8 gk .. + 7 of block b0 + p), then the scan of
  // the row for max|x|, all loads back to back; blocks beyond the row read zeros
  const int col = (b0 + (j >> 2)) * 128 + 32 * (j & 3) + 8 * gk;
  const bool live = b0 + (j >> 2) < nblk;
  const u4 xr = __builtin_amdgcn_raw_buffer_load_b128(rrsrc, live ? col * 2 : OUT_OF_RANGE, 0, 0);
  const uint32_t sb = (uint32_t)(uint8_t)__builtin_amdgcn_raw_buffer_load_b8(srsrc, live ? col >> 3 : OUT_OF_RANGE, 0, 0);
  uint32_t m16 = 0u;                                       // max of the sign-cleared halves: |values| compare like their bits
  for (int base = (int)threadIdx.x * 16; base < n * 2; base += 4 * WG_THREADS * 16) {
    u4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = __builtin_amdgcn_raw_buffer_load_b128(rrsrc, base + u * WG_THREADS * 16, 0, 0);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint32_t d[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
      for (int k = 0; k < 4; ++k) m16 = max(m16, max(d[k] & 0x7FFFu, (d[k] >> 16) & 0x7FFFu));
    }
  }
  m16 = wave_max_u32(m16);
  if (lane == 0) s_amax[w] = m16;
  __syncthreads();
#pragma unroll
  for (int k = 0; k < WG_WAVES; ++k) m16 = max(m16, s_amax[k]);
  float amax = is_bf16 ? bf16_bits_to_float((uint16_t)m16) : f16_bits_to_float((uint16_t)m16);
  if (amax != amax) amax = __uint_as_float(0x7F800000u);   // a NaN anywhere: treat the row as unbounded (scale 1)
  const int e = scale_exponent(amax);
  const float f = pow2f(-e) * INV_SQRT128;
  if (threadIdx.x == 0 && blockIdx.x == 0) sc_g[mrow] = pow2f(e);
  if (b0 >= nblk) return;                                  // uniform per wave: none of its blocks exists
  float y[2][4];
  rotate4_mfma(xr, sb, is_bf16 != 0, lane, y);
  const int b_o = b0 + gk;                                 // lane (p = lane / 16, j) holds elements 32 a' + 16 h + j of block b0 + p
  const bool live_o = b_o < nblk;
  HTR_GLOBAL _Float16* dst = (HTR_GLOBAL _Float16*)xt_g + (size_t)mrow * n + b_o * 128 + j;
  float r[2][4];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const _Float16 hv = (_Float16)(y[h][a] * f);
      if (live_o) dst[32 * a + 16 * h] = hv;
      r[h][a] = (float)hv;
    }
  // sums of the rounded values: even tiles (h = 0), odd tiles (h = 1), columns 0..63 (a < 2), columns 64..127
  f4 sm = {(r[0][0] + r[0][1]) + (r[0][2] + r[0][3]), (r[1][0] + r[1][1]) + (r[1][2] + r[1][3]),
           (r[0][0] + r[0][1]) + (r[1][0] + r[1][1]), (r[0][2] + r[0][3]) + (r[1][2] + r[1][3])};
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    float v = sm[c];
    v += dpp_mov<0xB1>(v); v += dpp_mov<0x4E>(v); v += dpp_mov<0x141>(v); v += dpp_mov<0x140>(v);
    sm[c] = v;
  }
  if (live_o && j == 0) *(HTR_GLOBAL f4*)((HTR_GLOBAL float*)xs_g + ((size_t)mrow * nblk + b_o) * 4) = sm;
}

template <int K> struct DecodedStep { h8 a[4]; };   // MFMA A operands of one step: (row 2q | 2q+1) x (columns 0..7 | 8..15)

// NODECODE (timing anchors only): the operands are the raw stream words, no arithmetic at all; results are meaningless
template <int K, bool NODECODE = false> __device__ __forceinline__ void decode_step(const StreamRegs<K>& r, int hist, DecodedStep<K>& d) {
  if constexpr (NODECODE) {
    const u4 raw = {r.d[0], r.d[1 % K], r.d[2 % K], r.d[3 % K]};
#pragma unroll
    for (int k = 0; k < 4; ++k) d.a[k] = __builtin_bit_cast(h8, raw);
    return;
  }
  // The history dword travels through the LDS crossbar.  Only the first states of the lane reach into it, so their
  // group is decoded last, behind a scheduling fence: the crossbar latency hides behind the other three groups.
  const uint32_t prev = (uint32_t)__builtin_amdgcn_ds_bpermute(hist, (int)r.d[K - 1]);
  __builtin_amdgcn_sched_barrier(0);
  Window<K> win;
  win.build_tail(r);
  d.a[1] = win.template group8<8>();
  d.a[2] = win.template group8<16>();
  d.a[3] = win.template group8<24>();
  __builtin_amdgcn_sched_barrier(0);
  win.build_head(prev);
  d.a[0] = win.template group8<0>();
}

// The same with something to do at the fence between the two parts (a barrier and LDS reads, in the batched kernel)
template <int K, typename F> __device__ __forceinline__ void decode_step_mid(const StreamRegs<K>& r, int hist, DecodedStep<K>& d, F&& mid) {
  const uint32_t prev = (uint32_t)__builtin_amdgcn_ds_bpermute(hist, (int)r.d[K - 1]);
  __builtin_amdgcn_sched_barrier(0);
  Window<K> win;
  win.build_tail(r);
  d.a[1] = win.template group8<8>();
  d.a[2] = win.template group8<16>();
  __builtin_amdgcn_sched_barrier(0);
  mid();
  __builtin_amdgcn_sched_barrier(0);
  d.a[3] = win.template group8<24>();
  win.build_head(prev);
  d.a[0] = win.template group8<0>();
}

// Nothing may move across a weight-stream load: the loads of a wave must issue in program order, one per step, so
// that the number of loads in flight behind any buffer is the same on every path and the wait in front of a decode
// leaves the other P - 1 loads outstanding.
#define HTR_PIN() __builtin_amdgcn_sched_barrier(0)

// A finisher that gave up waiting: bit 0 of the workspace's status word (word 0 of the header), and, if the caller
// registered one (bytes 8..15 of the header: the address of a host-visible word), a flag in host memory, so that the
// host can see the failure without a device-to-host copy.  Rare path, one lane.
__device__ __forceinline__ void report_give_up(uint32_t* status) {
  __hip_atomic_fetch_or(status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const unsigned long long mirror = __hip_atomic_load((const unsigned long long*)(status + 2), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (mirror != 0ull) __hip_atomic_store((uint32_t*)mirror, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
// A workspace whose status word is set holds partials that nobody collected: every later launch on it marks all its
// outputs NaN (instead of adding stale partials to good ones) until the caller has cleared it (htr_workspace_init).
__device__ __forceinline__ uint32_t load_status(const uint32_t* status) {
  return __hip_atomic_load(status, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
constexpr int FLAG_LANES = 1 << 4;     // kernel flag: chunk ids are dealt to the XCDs in eight lanes (see k_linear)
constexpr int FLAG_LAST_FINISHES = 1 << 5;   // batched kernel: the last split of a row block finishes all of its rows (see there)
constexpr int FLAG_LANE_LEN_SHIFT = 8; // with FLAG_LANES: grid / 8 in the bits from here up (no read of the hidden grid-size argument)

// ANCHOR = 1 is the same kernel with the decode compiled out (stream, rotation, products, hand-over and output side stay;
// the results are meaningless): a timing anchor that tells how much of a launch is the decode.
template <int K, int MB, int P, int D, bool PREROT, int RP, int ANCHOR = 0, bool PACE = false>
__global__ __launch_bounds__(WG_THREADS) void k_linear(const uint32_t* __restrict__ qw_a, const void* __restrict__ x_a,
                                                       const uint8_t* __restrict__ su_a, float* __restrict__ part_a,
                                                       int m, int n, int M_a, int chunk, int flags,
                                                       unsigned long long nblk_magic, const LinearTail t_a) {
  extern __shared__ __align__(16) unsigned char lds[];
  const uint32_t* __restrict__ qw = qw_a;
  const void* __restrict__ x = x_a;
  const uint8_t* __restrict__ su = su_a;
  float* __restrict__ part = part_a;
  int M = M_a;
  LinearTail t = t_a;
  if constexpr (PREROT) {                    // grouped launches always come with pre-rotated activations
    if (t_a.group != nullptr) {              // uniform: one entry of the problem table per blockIdx.y
      const htr_group_entry& ge = t_a.group[blockIdx.y];
      M = ge.M;
      if (M <= 0) return;
      qw = (const uint32_t*)ge.qweight; x = ge.x; su = (const uint8_t*)ge.su;
      part = part_a + (size_t)blockIdx.y * t_a.group_part_stride;
      t.scales = (const uint16_t*)ge.scales; t.sv = (const uint8_t*)ge.sv; t.bias = ge.bias; t.y = ge.y;
      const size_t shift = (size_t)blockIdx.y * t_a.group_prerot_stride;
      t.xt_g = (const _Float16*)((const unsigned char*)t_a.xt_g + shift);
      t.xs_g = (const float*)((const unsigned char*)t_a.xs_g + shift);
      t.sc_g = (const float*)((const unsigned char*)t_a.sc_g + shift);
    }
  }
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));   // wave index, provably uniform: keeps the
                                                                           // strip addressing on the scalar unit
  const int nblk = n >> 7;
  const int vtotal = (m >> 7) * nblk;
  // Which chunk this workgroup takes.  Workgroups go to the eight XCDs round-robin; with FLAG_LANES (set by the host
  // when every XCD then holds whole row blocks) workgroup b takes chunk (b mod 8) * (grid / 8) + b / 8, so the chunks of
  // one row block run on one XCD and the partial hand-over between them stays on that XCD's side of the memory
  // system.  A finisher still waits only for chunks of its own row block, i.e. for workgroups b - 8, b - 16, ...
  int cid = (int)blockIdx.x;
  if (flags & FLAG_LANES) cid = ((int)blockIdx.x & 7) * (flags >> FLAG_LANE_LEN_SHIFT) + ((int)blockIdx.x >> 3);
  const int v0 = cid * chunk, nsteps = min(vtotal, v0 + chunk) - v0;
  // v / nblk for v < 2^24 by multiplication: nblk_magic = ceil(2^40 / nblk)
  auto div_nblk = [&](int v) { return (int)(((unsigned long long)(unsigned)v * nblk_magic) >> 40); };
  const int rb_first = div_nblk(v0), c0 = v0 - rb_first * nblk;  // first row block and first column block of the chunk
  const int last_wraps = div_nblk(c0 + nsteps - 1);              // row-block changes before the chunk's last step
  const int nfin = div_nblk(c0 + nsteps);                        // row blocks that end inside the chunk
  const bool all_blocks = nsteps >= nblk;                        // chunk touches every column block
  const int nbl = all_blocks ? nblk : nsteps;                    // distinct column blocks; LDS slot of block b:
  const int nblmax = min(chunk, nblk);                           //   b if all_blocks, else (b - c0) mod nblk
  const int rowh = xt_row_halves(nblmax);
  const int x_dtype = flags & 3, y_dtype = (flags >> 2) & 3;

  _Float16* xt = (_Float16*)lds;
  float* s_xs = (float*)(lds + (size_t)(M + 1) * rowh * 2);
  float* s_sc = s_xs + 2 * M * nblmax;                 // activation scale per row
  float* s_bs = s_sc + M;                              // power-of-two scale per (row, block) pair this workgroup rotated
  float* s_fin = (float*)(lds + lds_fin_offset(M, nblmax));

  const int npairs = M * nbl;
  // pair index -> activation row: pi / nbl for pi < 2^16 through the float reciprocal (the quotient's fraction is at
  // least 0.5 / nbl away from an integer, far more than the rounding error), instead of an integer division per use
  const float inv_nbl = __builtin_amdgcn_rcpf((float)nbl);
  auto row_of_pair = [&](int pi) { return M == 1 ? 0 : (int)(((float)pi + 0.5f) * inv_nbl); };
  auto pair_col = [&](int li) { int b = all_blocks ? li : c0 + li; if (b >= nblk) b -= nblk; return b * 128; };

  // ---- activations first: they head the longest dependency chain.  Wave w rotates the (row, block) pairs 4w .. 4w + 3
  // on the matrix unit: H128 = H4 (x) H32 over the element index i = 32 a + c, so a block is a 4 x 32 matrix X and
  // H128 x = H4 . X . H32.  The four pairs of a wave are the 16 rows (pair p, a) of one MFMA A operand: lane
  // (k-group gk = lane / 16, row = lane % 16 = 4 p + a) loads the 8 consecutive elements 32 a + 8 gk .. + 7 of its pair
  // (16 bytes) and the one su byte that holds their signs.  Descriptors over x and su: a pair beyond the chunk's last
  // one gets an out-of-range offset and reads zeros, so the loads issue back to back without branches.
  // RP passes of 32 pairs (template: 1, or MAX_ROT_PASSES for many rows over long chunks); all loads go out up front.
  u4 xr[RP];
  uint32_t sb[RP];
  constexpr int COPY_REGS = 4;
  u4 cp[COPY_REGS];
  int cdst[COPY_REGS];
  const int ncopy = npairs * 16;                 // 16 pieces of 8 halves per (row, block) pair
  if constexpr (!PREROT) {
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, M * n * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t srsrc = __builtin_amdgcn_make_buffer_rsrc((void*)su, 0, n >> 3, 0x00020000);
    constexpr int OUT_OF_RANGE = 0x7FFFFF00;
    // every offset first, then the loads back to back: with address arithmetic (and its branches) between two loads
    // the compiler waits for the first load to return before it issues the second one and the weight stream behind it
    const int a = lane & 3, gk = lane >> 4;
    int xoff[RP], soff[RP];
#pragma unroll
    for (int r = 0; r < RP; ++r) {
      const int pi = ROT_PAIRS * r + 4 * w + ((lane & 15) >> 2);
      const bool live = pi < npairs;
      const int prow = row_of_pair(pi), pli = pi - prow * nbl;
      const int col = pair_col(pli) + 32 * a + 8 * gk;
      xoff[r] = live ? (prow * n + col) * 2 : OUT_OF_RANGE;
      soff[r] = live ? col >> 3 : OUT_OF_RANGE;
    }
    HTR_PIN();
#pragma unroll
    for (int r = 0; r < RP; ++r) {
      xr[r] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, xoff[r], 0, 0);
      sb[r] = (uint32_t)(uint8_t)__builtin_amdgcn_raw_buffer_load_b8(srsrc, soff[r], 0, 0);
    }
    HTR_PIN();
  } else {
    // with pre-rotated activations: 16-byte pieces of this chunk's x~ slice, through a descriptor over x~ so that the
    // pieces beyond the slice need no branch; offsets first, then the loads back to back (a branch or address
    // arithmetic between two loads makes the compiler wait for the first one before it issues anything else)
    const __amdgpu_buffer_rsrc_t crsrc = __builtin_amdgcn_make_buffer_rsrc((void*)t.xt_g, 0, M * n * 2, 0x00020000);
    constexpr int OUT_OF_RANGE = 0x7FFFFF00;
    int coff[COPY_REGS];
#pragma unroll
    for (int tt = 0; tt < COPY_REGS; ++tt) {
      const int ci = threadIdx.x + tt * WG_THREADS;
      const int pi = ci >> 4, mrow = row_of_pair(pi), li = pi - mrow * nbl;
      coff[tt] = ci < ncopy ? (mrow * n + pair_col(li) + (ci & 15) * 8) * 2 : OUT_OF_RANGE;
      cdst[tt] = mrow * rowh + li * 128 + (ci & 1) * 64 + ((ci & 15) >> 1) * 8;      // where the piece goes in LDS
    }
    HTR_PIN();
#pragma unroll
    for (int tt = 0; tt < COPY_REGS; ++tt) cp[tt] = __builtin_amdgcn_raw_buffer_load_b128(crsrc, coff[tt], 0, 0);
    HTR_PIN();
  }

  // row constants of a finished row block (scale, output sign, bias).  The wave's first (segment, row) pair requests
  // them here, with the activation loads and ahead of the weight stream (loads return in order: behind the stream
  // they would hold up the first decode), and only keeps the raw bits, which the output side converts at the end.
  // (Only where the workgroup rotates its own activations: in the kernel for pre-rotated activations the six
  // registers, held through the loop, would cost a wave of occupancy; there the request goes out before the last
  // barrier.)
  struct RowRaw { uint32_t sc0, sc1, sv0, sv1, b0, b1; };
  auto row_load = [&](int rb, RowRaw& r) {
    const int r0 = rb * 128 + lane, r1 = r0 + 64;
    r.sc0 = ((const HTR_GLOBAL uint16_t*)t.scales)[r0];
    r.sc1 = ((const HTR_GLOBAL uint16_t*)t.scales)[r1];
    r.sv0 = ((const HTR_GLOBAL uint8_t*)t.sv)[r0 >> 3];
    r.sv1 = ((const HTR_GLOBAL uint8_t*)t.sv)[r1 >> 3];
    r.b0 = 0u; r.b1 = 0u;
    if (t.bias != nullptr) {
      if (y_dtype == HTR_F32) { r.b0 = ((const HTR_GLOBAL uint32_t*)t.bias)[r0]; r.b1 = ((const HTR_GLOBAL uint32_t*)t.bias)[r1]; }
      else { r.b0 = ((const HTR_GLOBAL uint16_t*)t.bias)[r0]; r.b1 = ((const HTR_GLOBAL uint16_t*)t.bias)[r1]; }
    }
  };
  auto row_finish = [&](const RowRaw& r, float& rs0, float& rs1, float& b0v, float& b1v) {
    rs0 = f16_bits_to_float((uint16_t)r.sc0) * t.cbscale * INV_SQRT128;
    rs1 = f16_bits_to_float((uint16_t)r.sc1) * t.cbscale * INV_SQRT128;
    // output sign of rows lane and lane + 64 (bit lane % 8 of their sv bytes) folded into the scale that is applied
    // after the rotation
    rs0 = ((r.sv0 >> (lane & 7)) & 1u) ? -rs0 : rs0;
    rs1 = ((r.sv1 >> (lane & 7)) & 1u) ? -rs1 : rs1;
    auto cvt = [&](uint32_t b) {
      return y_dtype == HTR_F32 ? __uint_as_float(b) : y_dtype == HTR_BF16 ? bf16_bits_to_float((uint16_t)b) : f16_bits_to_float((uint16_t)b);
    };
    b0v = cvt(r.b0); b1v = cvt(r.b1);
  };
  RowRaw first_raw = {0u, 0u, 0u, 0u, 0u, 0u};
  const bool early_rows = !PREROT && M == 1;       // more rows: requested before the last barrier (no division up here)
  if (early_rows && w < nfin) row_load(rb_first + w, first_raw);

  // ---- the weight stream.  This wave's strip of row block rb is tile row rb * 8 + w; its 8 tiles of column block blk
  // are 64 * K contiguous dwords; a strip is contiguous over blk, the same strip of the next row block starts 8 strips
  // later.  The stream is addressed through a buffer descriptor that covers exactly the wave's bytes of this chunk:
  // a load beyond the last step is out of range, returns zeros and costs no memory traffic, so every step can issue
  // its load unconditionally.
  constexpr int STEP_BYTES = 256 * K;
  const uint32_t strip_bytes = (uint32_t)nblk * STEP_BYTES;
  const uint32_t* wave_base = qw + ((size_t)(rb_first * 8 + w) * nblk + (size_t)c0) * (STEP_BYTES / 4);   // uniform
  const uint32_t extent = (uint32_t)nsteps * STEP_BYTES + (uint32_t)last_wraps * 7u * strip_bytes;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)wave_base, 0, (int)extent, 0x00020000);
  // the walk over the chunk's steps: a scalar byte offset (the lane adds its own), advanced without branches
  const int lane_off = lane * 4 * K;
  int pf_off = 0;
  int pf_blk = c0;
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

  for (int i = threadIdx.x; i < rowh / 2; i += WG_THREADS) ((uint32_t*)(xt + (size_t)M * rowh))[i] = 0u;   // zero row

  // ---- rotation (waves that have a pair): signs, X . H32 as two matrix instructions (exact: the operands are the
  // 16-bit activations themselves and +-1, accumulated in float32), H4 over the four accumulator registers, then the
  // block's own power-of-two scale, rounding to f16 and the sums per tile parity.  A block keeps scale 1 unless its
  // largest rotated value would leave f16's comfortable range (then 2^e brings it to [2^13, 2^14)): ordinary
  // activations have scale 1 in every block and the product accumulates across blocks inside the matrix unit; if any
  // block of the chunk has another scale, the products are scaled per block (see consume()).  No exchange between
  // waves, so one barrier between the rotation and the first product.
  if constexpr (!PREROT) {
#pragma unroll
    for (int r = 0; r < RP; ++r) {
    if (ROT_PAIRS * r + 4 * w < npairs) {                            // uniform
      const int j = lane & 15;
      float y[2][4];
      rotate4_mfma(xr[r], sb[r], x_dtype == HTR_BF16, lane, y);
      // largest |value| of the pair: 8 in the lane, then over the 16 lanes of the row
      float mx = fmaxf(fmaxf(fmaxf(fabsf(y[0][0]), fabsf(y[0][1])), fmaxf(fabsf(y[0][2]), fabsf(y[0][3]))),
                       fmaxf(fmaxf(fabsf(y[1][0]), fabsf(y[1][1])), fmaxf(fabsf(y[1][2]), fabsf(y[1][3]))));
      uint32_t mu = __float_as_uint(mx * INV_SQRT128);               // non-negative floats compare like their bit patterns
      mu = max(mu, dpp_mov_u32<0xB1>(mu)); mu = max(mu, dpp_mov_u32<0x4E>(mu));
      mu = max(mu, dpp_mov_u32<0x141>(mu)); mu = max(mu, dpp_mov_u32<0x140>(mu));
      const int e = block_scale_exponent(mu);
      const float f = pow2f(-e) * INV_SQRT128;
      const int po = ROT_PAIRS * r + 4 * w + (lane >> 4);
      const bool live_o = po < npairs;
      const int prow_o = row_of_pair(po), pli_o = po - prow_o * nbl;
      _Float16* dst = xt + (size_t)prow_o * rowh + pli_o * 128 + (j >> 3) * 64 + (j & 7);
      float sums[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const h2 p01 = __builtin_convertvector(f2{y[h][0] * f, y[h][1] * f}, h2);
        const h2 p23 = __builtin_convertvector(f2{y[h][2] * f, y[h][3] * f}, h2);
        if (live_o) {                                                // element 32 a' + 16 h + j: tile 2 a' + h, column j
          dst[(0 + h) * 8] = p01.x; dst[(2 + h) * 8] = p01.y; dst[(4 + h) * 8] = p23.x; dst[(6 + h) * 8] = p23.y;
        }
        // sum of the rounded values of tile parity h: in the lane, then over the row
        float sh = __builtin_amdgcn_fdot2(p23, h2{(_Float16)1.f, (_Float16)1.f}, __builtin_amdgcn_fdot2(p01, h2{(_Float16)1.f, (_Float16)1.f}, 0.f, false), false);
        sh += dpp_mov<0xB1>(sh); sh += dpp_mov<0x4E>(sh); sh += dpp_mov<0x141>(sh); sh += dpp_mov<0x140>(sh);
        sums[h] = sh;
      }
      if (live_o && j == 0) {
        s_xs[2 * po] = sums[0]; s_xs[2 * po + 1] = sums[1];
        s_bs[po] = pow2f(e);
      }
    }
    }
  }

  // ---- decode the first D steps into registers ahead of the barrier: they need no x~, and they fill the time the
  // rotating waves take (short chunks are decoded completely this way)
  static_assert(D >= 2 && D <= P && D % 2 == 0, "pre-decoded steps come out of the first D stream buffers");
  const int hist = history_lane_byteaddr(lane);
  DecodedStep<K> pre[D];
#pragma unroll
  for (int i = 0; i < D; ++i) {
    if (i == 0 || i < nsteps) decode_step<K, ANCHOR == 1>(buf[i], hist, pre[i]);
    prefetch(buf[i]);
  }
  // The decoded operands are first used behind the barrier, in conditional code, and the compiler would sink the
  // whole decode down there (after the barrier, where nothing overlaps it any more): pin the values here.
#pragma unroll
  for (int i = 0; i < D; ++i)
#pragma unroll
    for (int k = 0; k < 4; ++k) asm volatile("" : "+v"(pre[i].a[k]));

  if constexpr (PREROT) {
    // copy the slice into LDS; sums per (row, block, parity) come with it
#pragma unroll
    for (int tt = 0; tt < COPY_REGS; ++tt) {
      const int ci = threadIdx.x + tt * WG_THREADS;
      if (ci < ncopy) *(u4*)(xt + cdst[tt]) = cp[tt];
    }
    for (int ci = threadIdx.x + COPY_REGS * WG_THREADS; ci < ncopy; ci += WG_THREADS) {
      const int pi = ci >> 4, mrow = row_of_pair(pi), li = pi - mrow * nbl;
      *(u4*)(xt + (size_t)mrow * rowh + li * 128 + (ci & 1) * 64 + ((ci & 15) >> 1) * 8) =
          *(const u4*)(t.xt_g + (size_t)mrow * n + pair_col(li) + (ci & 15) * 8);
    }
    for (int i = threadIdx.x; i < npairs * 2; i += WG_THREADS) {
      const int pi = i >> 1, mrow = row_of_pair(pi), li = pi - mrow * nbl;
      s_xs[i] = t.xs_g[((size_t)mrow * nblk + (pair_col(li) >> 7)) * 4 + (i & 1)];
    }
  }
  __syncthreads();

  // ---- per-lane constants of the product and of the partial store
  // MFMA operands: row i = lane % 16 = (tile parity h = i / 8, row pair q = i % 8); B column c = lane % 16 carries
  // activation row c / 2 and tile parity c % 2; the 16-lane group g = lane / 16 supplies k-slots of tile 2g + parity.
  // D[i][c] sits in lane c + 16 * (i / 4), register i % 4.  MFMA rows 0..7 (even tiles) are valid in the even
  // columns c = 2r, rows 8..15 (odd tiles) in the odd columns c = 2r + 1; a valid lane (g', c) holds strip rows
  // 8 (g' & 1) .. + 7 of activation row c / 2 for parity g' / 2.
  const int g = lane >> 4, n16 = lane & 15;
  const int par = g >> 1;
  const bool mine = (n16 & 1) == par;
  int boff[MB];      // LDS half-index of this lane's B operand in LDS block 0
  int xsoff[MB];     // index of this lane's (row, parity) x~ sum in LDS block 0, or -1
  float sc[MB];      // the row's activation scale
  float offs[MB];    // running 1534 * sum(x~) over the blocks of the current segment
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int mrow = mb * 8 + (n16 >> 1);
    const bool live = mine && mrow < M;
    boff[mb] = (mrow < M ? mrow : M) * rowh + 8 * (2 * g + (n16 & 1));
    xsoff[mb] = live ? 2 * (mrow * nbl) + par : -1;
    offs[mb] = 0.f; sc[mb] = 0.f;
    if (live) {
      if constexpr (PREROT) sc[mb] = t.sc_g[mrow];
      else sc[mb] = 1.f;
    }
  }
  // does any block this workgroup rotated carry a scale other than 1?  (uniform; never with pre-rotated activations,
  // whose scale is one per row)
  bool scaled = false;
  if constexpr (!PREROT) {
    bool other = false;
#pragma unroll
    for (int r = 0; r < (RP * ROT_PAIRS + 63) / 64; ++r) other |= s_bs[min(lane + 64 * r, npairs - 1)] != 1.f;
    scaled = __any(other) != 0;
  }

  f4 acc[MB][2];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) { acc[mb][0] = f4{0.f, 0.f, 0.f, 0.f}; acc[mb][1] = f4{0.f, 0.f, 0.f, 0.f}; }

  int cur_blk = c0, cur_li = all_blocks ? c0 : 0, cur_seg = 0, done = 0;
  // B operands and x~ sums of the step about to be multiplied: read from LDS one step ahead, right after the
  // previous step's matrix instructions issue, so that their latency hides behind the decode
  h8 B0[MB], B1[MB];
  float xsv[MB];
  float bsv[MB];     // the block's scale (only read where some block's scale is not 1)
  float k1534[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) { k1534[mb] = xsoff[mb] >= 0 ? 1534.f : 0.f; bsv[mb] = 1.f; }
  auto load_b = [&](int li) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const _Float16* bp = xt + boff[mb] + li * 128;
      B0[mb] = *(const h8*)bp;
      B1[mb] = *(const h8*)(bp + 64);
      xsv[mb] = s_xs[max(xsoff[mb], 0) + 2 * li];
    }
    if constexpr (!PREROT) {
      if (scaled) {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) bsv[mb] = s_bs[(max(xsoff[mb], 0) >> 1) + li];
      }
    }
  };
  load_b(cur_li);
  // product of the decoded step with the chunk's rotated activations, and the end of a segment
  auto consume = [&](const DecodedStep<K>& d, bool maybe_last) {
    if (PREROT || !scaled) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[mb][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[0], B0[mb], acc[mb][0], 0, 0, 0);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[mb][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[2], B0[mb], acc[mb][1], 0, 0, 0);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[mb][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[1], B1[mb], acc[mb][0], 0, 0, 0);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) acc[mb][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[3], B1[mb], acc[mb][1], 0, 0, 0);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) offs[mb] = __builtin_fmaf(k1534[mb], xsv[mb], offs[mb]);
    } else {
      // blocks with different scales: the block's product on its own, then into the running sums in true units
      const f4 zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
          f4 pr = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[2 * rr], B0[mb], zero4, 0, 0, 0);
          pr = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[2 * rr + 1], B1[mb], pr, 0, 0, 0);
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) acc[mb][rr][jj] = __builtin_fmaf(pr[jj], bsv[mb], acc[mb][rr][jj]);
        }
        offs[mb] = __builtin_fmaf(k1534[mb] * xsv[mb], bsv[mb], offs[mb]);
      }
    }
    ++done; ++cur_blk; ++cur_li;
    const bool row_end = cur_blk == nblk;
    const bool last = maybe_last && done == nsteps;
    const bool seg_end = row_end || last;
    if (row_end) { cur_blk = 0; if (all_blocks) cur_li = 0; }
    if (!last) load_b(cur_li);          // next step's operands (the slot exists: not the last step)
    if (seg_end) {
      // End of a segment: this wave's strip partial per activation row, the 1534 offset removed, the activation scale
      // undone, the two tile parities added (the parity-1 lane of a value is lane ^ 33).  A segment that ends its
      // row block is finished by this workgroup and goes to LDS; a chunk that ends inside a row block leaves its
      // last partial in the workgroup's slot, stored with the lowest mantissa bit set (never the all-zero pattern),
      // device scope (written through), not waited for.
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int mrow = mb * 8 + (n16 >> 1);
        float tot[8];
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int rr = 0; rr < 2; ++rr) {
            const float v = xsoff[mb] >= 0 ? (acc[mb][rr][j] - offs[mb]) * sc[mb] : 0.f;
            float lo_half, hi_half;
            halves32(lane_xor_dpp<1>(v), lo_half, hi_half);
            tot[2 * j + rr] = v + hi_half;            // meaningful in lanes < 32 with an even column
          }
        if (lane < 32 && (n16 & 1) == 0 && mrow < M) {
          const int rowi = 16 * w + 8 * (g & 1);
          if (row_end) {
            float* dst = s_fin + ((size_t)cur_seg * M + mrow) * 128 + rowi;
            *(f4*)dst = f4{tot[0], tot[1], tot[2], tot[3]};
            *(f4*)(dst + 4) = f4{tot[4], tot[5], tot[6], tot[7]};
          } else {
            uint32_t* dst = (uint32_t*)(part + ((size_t)cid * M + mrow) * 128 + rowi);
#pragma unroll
            for (int i = 0; i < 8; ++i)
              __hip_atomic_store(dst + i, __float_as_uint(tot[i]) | 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
        acc[mb][0] = f4{0.f, 0.f, 0.f, 0.f}; acc[mb][1] = f4{0.f, 0.f, 0.f, 0.f};
        offs[mb] = 0.f;
      }
      if (row_end) ++cur_seg;
    }
  };

  // ---- main loop: one 128-column block (8 tiles of this wave's strip) per step.  Step v multiplies what the previous
  // step decoded, then decodes step v + 1 out of buffer (v + 1) % P while the matrix unit works, then refills it.
  // Groups of P steps that all have a successor run without bounds checks; the last steps are checked one by one.
#pragma unroll
  for (int i = 0; i < D - 1; ++i)
    if (i < nsteps) consume(pre[i], true);
  DecodedStep<K> cur = pre[D - 1];
  int v = D - 1;
  // The two waves that share a SIMD (w and w + 4) compete for its issue slots, and between equals the arbiter favours the
  // older one: left alone, waves 0..3 run ahead, leave the loop when the others have 40 % of their steps to go, and
  // those finish at the rate of one wave per SIMD (an instruction every five cycles instead of two waves' three).  In
  // the PACE instantiation the younger waves take the higher priority for two groups of P steps out of every four:
  // both keep pace, and the SIMD has two waves to issue from until the end (gate_up 28672x4096: 19.1 -> 17.7 us).  It
  // is a variant of its own, chosen by the launcher for long chunks, because it does not pay everywhere (short chunks,
  // many rows with many contributors per row block) and its mere presence in the code changed how the compiler laid
  // out the short-chunk kernels.
  for (; v + P < nsteps; v += P) {
    if constexpr (PACE) {
      if (w >= 4) {
        if ((v / P) & 2) __builtin_amdgcn_s_setprio(0); else __builtin_amdgcn_s_setprio(1);
      }
    }
#pragma unroll
    for (int pp = 0; pp < P; ++pp) {
      StreamRegs<K>& nxt = buf[(pp + D) % P];
      consume(cur, false);
      decode_step<K, ANCHOR == 1>(nxt, hist, cur);
      prefetch(nxt);
    }
  }
  if constexpr (PACE) __builtin_amdgcn_s_setprio(0);
#pragma unroll
  for (int pp = 0; pp < P; ++pp) {
    if (v + pp < nsteps) {
      consume(cur, true);
      if (v + pp + 1 < nsteps) decode_step<K, ANCHOR == 1>(buf[(pp + D) % P], hist, cur);
    }
  }

  // ---- output side of the row blocks that end in this chunk (nfin of them): wave w takes (segment, activation row)
  // pairs w, w + 8, ...
  const size_t slot_floats = (size_t)M * 128;
  if (nfin == 0) return;        // a pure contributor: its partial is on its way, nothing else to do (uniform)
  if (!early_rows && w < nfin * M) row_load(rb_first + (M == 1 ? w : w / M), first_raw);
  const uint32_t stale = load_status(t.status);     // non-zero: an earlier launch on this workspace gave up
  __syncthreads();
  for (int idx = w; idx < nfin * M; idx += WG_WAVES) {
    const int seg = M == 1 ? idx : idx / M, mrow = idx - seg * M, rb = rb_first + seg;
    const int r0 = rb * 128 + lane, r1 = r0 + 64;
    float rs0, rs1, b0v, b1v;
    if (idx == w) {
      row_finish(first_raw, rs0, rs1, b0v, b1v);
    } else {
      RowRaw rr;
      row_load(rb, rr);
      row_finish(rr, rs0, rs1, b0v, b1v);
    }
    float v0s = 0.f, v1s = 0.f;
    bool failed = false;
    if (seg == 0 && c0 != 0) {
      // earlier chunks hold the beginning of this row block: chunks j0 .. cid - 1, each in its own slot.  They
      // were dispatched before this workgroup, so waiting for them cannot deadlock; the wait is bounded all the same.
      // Eight contributors are read per round trip.
      const int j0 = (int)(((unsigned long long)(unsigned)(rb * nblk) * t.chunk_magic) >> 40), j1 = cid;
      int tries = 0;
      for (;;) {
        bool missing = false;
        v0s = 0.f; v1s = 0.f;
        for (int jb = j0; jb < j1; jb += 8) {
          uint32_t u0[8], u1[8];
#pragma unroll
          for (int k = 0; k < 8; ++k) {
            const int j = min(jb + k, j1 - 1);
            const uint32_t* pp = (const uint32_t*)(part + (size_t)j * slot_floats + (size_t)mrow * 128);
            u0[k] = __hip_atomic_load(pp + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            u1[k] = __hip_atomic_load(pp + lane + 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
#pragma unroll
          for (int k = 0; k < 8; ++k)
            if (jb + k < j1) {
              missing |= (u0[k] == 0u) | (u1[k] == 0u);
              v0s += __uint_as_float(u0[k]); v1s += __uint_as_float(u1[k]);
            }
        }
        if (!__any(missing)) break;
        if (++tries >= t.spin_limit) { failed = true; break; }
        __builtin_amdgcn_s_sleep(2);
      }
      if (!failed) {
        for (int j = j0; j < j1; ++j) {          // leave the workspace zero for the next call
          uint32_t* pp = (uint32_t*)(part + (size_t)j * slot_floats + (size_t)mrow * 128);
          __hip_atomic_store(pp + lane, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(pp + lane + 64, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      } else if (lane == 0) {
        report_give_up(t.status);
      }
    }
    failed |= stale != 0u;
    const float* own = s_fin + ((size_t)seg * M + mrow) * 128;
    v0s += own[lane]; v1s += own[lane + 64];
    // the row scale applies before the output rotation; the sign and 1/sqrt(128) after it
    v0s *= fabsf(rs0); v1s *= fabsf(rs1);
    fwht128_wave(v0s, v1s, lane);
    v0s = __builtin_fmaf(v0s, rs0 < 0.f ? -1.f : 1.f, b0v);
    v1s = __builtin_fmaf(v1s, rs1 < 0.f ? -1.f : 1.f, b1v);
    if (failed) { v0s = __builtin_nanf(""); v1s = v0s; }
    store_elem_g(t.y, y_dtype, (size_t)mrow * m + r0, v0s);
    store_elem_g(t.y, y_dtype, (size_t)mrow * m + r1, v1s);
  }
}

