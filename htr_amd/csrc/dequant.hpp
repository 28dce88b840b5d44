// Part of htr_gfx950.hip, included inside its anonymous namespace: k_decode_raw, k_dequant_q, k_dequant_w.
// ------------------------------------------------------------------------------------------------ debug decodes
template <int K, int U> struct ForEach32 {
  template <typename F> __device__ __forceinline__ static void run(const Window<K>& w, F&& f) {
    f(U, w.template value<U>());
    if constexpr (U + 1 < 32) ForEach32<K, U + 1>::run(w, f);
  }
};

template <int K>
__global__ __launch_bounds__(256) void k_decode_raw(const uint32_t* __restrict__ qw, int16_t* __restrict__ out, int64_t ntiles) {
  // thread = (tile, row pair q); the 8 threads of a tile are consecutive lanes
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int lane = threadIdx.x & 63;
  const bool live = gid < ntiles * 8;
  StreamRegs<K> r;
#pragma unroll
  for (int k = 0; k < K; ++k) r.d[k] = 0u;
  if (live) load_stream<K>(qw + gid * K, r);
  const uint32_t prev = (uint32_t)__builtin_amdgcn_ds_bpermute(history_lane_byteaddr(lane), (int)r.d[K - 1]);
  if (!live) return;
  Window<K> w;
  w.build(r, prev);
  int16_t vals[32];
  ForEach32<K, 0>::run(w, [&](int u, int v) { vals[u] = (int16_t)v; });
  u4* o = (u4*)(out + gid * 32);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    u4 pk;
    pk.x = (uint16_t)vals[8 * i + 0] | ((uint32_t)(uint16_t)vals[8 * i + 1] << 16);
    pk.y = (uint16_t)vals[8 * i + 2] | ((uint32_t)(uint16_t)vals[8 * i + 3] << 16);
    pk.z = (uint16_t)vals[8 * i + 4] | ((uint32_t)(uint16_t)vals[8 * i + 5] << 16);
    pk.w = (uint16_t)vals[8 * i + 6] | ((uint32_t)(uint16_t)vals[8 * i + 7] << 16);
    o[i] = pk;
  }
}

template <int K>
__global__ __launch_bounds__(256) void k_dequant_q(const uint32_t* __restrict__ qw, const uint16_t* __restrict__ scales,
                                                   float* __restrict__ Q, int mt, int nt, double rms) {
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int lane = threadIdx.x & 63;
  const int64_t ntiles = (int64_t)mt * nt;
  const bool live = gid < ntiles * 8;
  StreamRegs<K> r;
#pragma unroll
  for (int k = 0; k < K; ++k) r.d[k] = 0u;
  if (live) load_stream<K>(qw + gid * K, r);
  const uint32_t prev = (uint32_t)__builtin_amdgcn_ds_bpermute(history_lane_byteaddr(lane), (int)r.d[K - 1]);
  if (!live) return;
  Window<K> w;
  w.build(r, prev);
  const int64_t tile = gid >> 3;
  const int q = (int)(gid & 7);
  const int ti = (int)(tile / nt), tj = (int)(tile - (int64_t)ti * nt);
  const int64_t n = (int64_t)nt * 16;
  const int row0 = ti * 16 + 2 * q;
  const float sc0 = f16_bits_to_float(scales[row0]), sc1 = f16_bits_to_float(scales[row0 + 1]);
  float* o0 = Q + (int64_t)row0 * n + (int64_t)tj * 16;
  float* o1 = o0 + n;
  // cb[s] = float32(v / rms) with the division in float64, then one float32 multiply (htr/wire.py:24,102 of the reference)
  ForEach32<K, 0>::run(w, [&](int u, int v) {
    const float cb = (float)((double)v / rms);
    if (u < 16) o0[u] = cb * sc0; else o1[u - 16] = cb * sc1;
  });
}

// ------------------------------------------------------------------------------------------------ original-basis W
// W = Sv . Ho . Q . Hi . Su as bf16 [m, n] (htr/wire.py:105-113 of the reference), one workgroup of 512 threads per
// 128x128 block, 32 elements per thread.  The 14 butterfly stages of the two H128 (7 over the column index, 7 over the
// row index; they commute) run on register arrays, five or four stages at a time, with two trips through LDS that
// re-deal the elements so that the next stages' partners sit in one thread:
//   A  thread = (tile, row pair) as decoded: rows 2q, 2q + 1 x the tile's 16 columns -> column bits 0-3, row bit 0
//   B  thread = 8 column groups x rows +0, +2, +8                                   -> column bits 4-6, row bits 1, 3
//   C  thread = 16 rows (+4, +16, +32, +64) x 2 adjacent columns                    -> row bits 2, 4, 5, 6
// The row scale (times CBSCALE / 128, the two rotations' norms) is applied before the first stage, the signs after
// the last one, on the packed bf16 pairs.
constexpr int DQW_LD = 132;   // LDS leading dimension in floats: rows stay 16-byte aligned and shift by 4 banks

// in-place Walsh-Hadamard butterflies over the index bits [B0, B1) of a 32-element register array
template <int B0, int B1> __device__ __forceinline__ void fwht_regs(float (&v)[32]) {
#pragma unroll
  for (int b = B0; b < B1; ++b)
#pragma unroll
    for (int i = 0; i < 32; ++i)
      if (!(i & (1 << b))) {
        const float x = v[i], y = v[i | (1 << b)];
        v[i] = x + y; v[i | (1 << b)] = x - y;
      }
}

template <int K, int U> struct ForEach32Sum {     // f(u, bytesum of state u) for u = U .. 31
  template <typename F> __device__ __forceinline__ static void run(const Window<K>& w, F&& f) {
    f(U, __builtin_amdgcn_sad_u8(w.template genword<U>(), 0u, 0u));
    if constexpr (U + 1 < 32) ForEach32Sum<K, U + 1>::run(w, f);
  }
};

typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
typedef float fl2 __attribute__((ext_vector_type(2)));

template <int K>
__global__ __launch_bounds__(512) void k_dequant_w(const uint32_t* __restrict__ qw, const uint16_t* __restrict__ scales,
                                                   const uint8_t* __restrict__ su, const uint8_t* __restrict__ sv,
                                                   uint16_t* __restrict__ W, int nt, float cbscale) {
  extern __shared__ __align__(16) unsigned char lds[];
  float* blk = (float*)lds;                                  // [128][DQW_LD]
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int bj = blockIdx.x, bi = blockIdx.y;                // 128-column block, 128-row block
  const int n = nt * 16;
  float v[32];
  // ---- A: decode; v[16 rho + c] = row 2q + rho, column c of the tile
  {
    const int t64 = threadIdx.x >> 3, q = threadIdx.x & 7;
    const int ti = t64 >> 3, tj = t64 & 7;                   // tile row / column inside the block
    const size_t tile = (size_t)(bi * 8 + ti) * nt + (size_t)bj * 8 + tj;
    StreamRegs<K> r;
    load_stream<K>(qw + tile * (8 * K) + q * K, r);
    const int row0 = ti * 16 + 2 * q;
    const float s0 = f16_bits_to_float(scales[bi * 128 + row0]) * cbscale * (1.0f / 128.0f);
    const float s1 = f16_bits_to_float(scales[bi * 128 + row0 + 1]) * cbscale * (1.0f / 128.0f);
    Window<K> win;
    win.build(r, (uint32_t)__builtin_amdgcn_ds_bpermute(history_lane_byteaddr(lane), (int)r.d[K - 1]));
    const float o0 = -510.f * s0, o1 = -510.f * s1;          // v = bytesum - 510
    ForEach32Sum<K, 0>::run(win, [&](int u, uint32_t sum) {
      v[u] = __builtin_fmaf((float)sum, u < 16 ? s0 : s1, u < 16 ? o0 : o1);
    });
    fwht_regs<0, 5>(v);
    float* o = blk + row0 * DQW_LD + tj * 16;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *(f4*)(o + 4 * i) = f4{v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]};
      *(f4*)(o + DQW_LD + 4 * i) = f4{v[16 + 4 * i], v[16 + 4 * i + 1], v[16 + 4 * i + 2], v[16 + 4 * i + 3]};
    }
  }
  __syncthreads();
  // ---- B: v[kappa + 8 a] = row base + 2 a0 + 8 a1, column cl + 16 kappa.  Lanes: cl = lane & 15, row bit 2 = lane
  // bit 4 (4 rows = 16 banks further), row bit 0 = lane bit 5; waves: row bits 4, 5, 6.
  {
    const int cl = lane & 15;
    const int rbase = ((lane >> 5) & 1) + 4 * ((lane >> 4) & 1) + 16 * w;
    float* p = blk + rbase * DQW_LD + cl;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int kap = 0; kap < 8; ++kap) v[kap + 8 * a] = p[(2 * (a & 1) + 8 * (a >> 1)) * DQW_LD + 16 * kap];
    fwht_regs<0, 5>(v);
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int kap = 0; kap < 8; ++kap) p[(2 * (a & 1) + 8 * (a >> 1)) * DQW_LD + 16 * kap] = v[kap + 8 * a];
  }
  __syncthreads();
  // ---- C: v[c0 + 2 j] = row base + 4 j0 + 16 j1 + 32 j2 + 64 j3, column 2 (lane & 31) + 64 (lane >> 5) + c0; waves: row
  // bits 0, 1, 3.  Then signs and the bf16 pair store (a wave writes 256 contiguous bytes of a row).
  {
    const int col = 2 * (lane & 31) + 64 * (lane >> 5);
    const int rbase = (w & 1) + 2 * ((w >> 1) & 1) + 8 * (w >> 2);
    const float* p = blk + rbase * DQW_LD + col;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const fl2 t = *(const fl2*)(p + (4 * (j & 1) + 16 * ((j >> 1) & 1) + 32 * ((j >> 2) & 1) + 64 * (j >> 3)) * DQW_LD);
      v[2 * j] = t.x; v[2 * j + 1] = t.y;
    }
    fwht_regs<1, 5>(v);
    // sign masks: column pair from su (two adjacent bits), rows from the block's 128 sv bits (four uniform words)
    const uint32_t subits = (uint32_t)su[(bj * 128 + col) >> 3] >> (col & 7);
    const uint32_t colmask = ((subits & 1u) << 15) | ((subits & 2u) << 30);
    const uint32_t* svw = (const uint32_t*)(sv + bi * 16);
    uint16_t* dst = W + (size_t)(bi * 128 + rbase) * n + (size_t)bj * 128 + col;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int roff = 4 * (j & 1) + 16 * ((j >> 1) & 1) + 32 * ((j >> 2) & 1) + 64 * (j >> 3);   // compile-time per j
      const uint32_t sbit = (svw[roff >> 5] >> ((roff & 31) + rbase)) & 1u;      // rbase <= 11, roff & 31 <= 20: no carry
      const fl2 f = {v[2 * j], v[2 * j + 1]};
      const bf2 h = __builtin_convertvector(f, bf2);
      const uint32_t bits = __builtin_bit_cast(uint32_t, h) ^ colmask ^ (sbit * 0x80008000u);
      *(uint32_t*)(dst + (size_t)roff * n) = bits;
    }
  }
}

