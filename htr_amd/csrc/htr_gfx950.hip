// HTR-W1 packed-linear kernels for MI355X (gfx950, CDNA4, wave64) behind a plain C ABI.
//
//   y = sv . Ho( Q . Hi(su . x) ),   Q[i,j] = v(s_ij) * scale_i * CBSCALE,
//   v(s) = bytesum((s * 0xDF6ADF + 0x34983) mod 2^32) - 510              (docs/FORMAT.md:7-13 of the reference)
//
// Work decomposition of the fused linear kernel
//   workgroup = 8 waves = one 128-row output block (one H128 output block) x one split of the input columns
//   wave      = one 16-row strip of tiles; per step it streams the 8 consecutive tiles that cover one 128-column
//               input block (8 * 32K contiguous bytes: each lane loads its 4K contiguous bytes)
//   lane      = (tile-in-step = lane / 8, row pair q = lane % 8): the K dwords a lane loads are exactly the stream
//               bits of tile rows 2q and 2q+1 (32 steps); the 16-K history bits come from the previous lane's last
//               dword through the LDS crossbar (ds_bpermute), the tail-biting wrap is lane 7 -> lane 0 of the tile
//   decode    = per weight: one bit-field extract, one v_mad_u32_u24, one v_sad_u8 / v_sad_hi_u8.  The SAD pair
//               accumulates onto 0x64006400, which leaves two IEEE half floats 1024 + bytesum = 1534 + v packed in
//               one dword with no integer->float conversion and no pack instruction.
//   product   = v_mfma_f32_16x16x32_f16.  MFMA row i = lane % 16 = (tile parity h = i / 8, row pair q = i % 8), the
//               four 16-lane groups g supply the k-slots, so lane (g, h, q) feeds tile 2g + h.  Rows with h = 0 and
//               h = 1 need different activation columns; the B operand therefore carries, for activation row r,
//               the even tiles in MFMA column 2r and the odd tiles in column 2r + 1, and only D[i][2r + h(i)] is
//               kept.  Eight activation rows share one MFMA; more rows reuse the decoded A registers.
//   offset    = the constant 1534 is removed afterwards with 1534 * sum(x~) per activation row.
//   epilogue  = split partials meet in a workspace; the last workgroup of a row block (arrival counter) sums them in
//               a fixed order, applies scale * CBSCALE, the output H128, sv, bias and the cast.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include "../../include/htr_gfx950.h"

namespace {

constexpr uint32_t GEN_A = 0xDF6ADFu;
constexpr uint32_t GEN_B = 0x34983u;
constexpr float INV_SQRT128 = 0.08838834764831845f;
constexpr float SQRT128 = 11.313708498984761f;
// 1 / sqrt(mean v^2) over all 65536 states: sum v^2 = 1433042863 (htr/wire.py:28-30 of the reference)
constexpr double MEAN_SQ = 1433042863.0 / 65536.0;

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef uint32_t u4 __attribute__((ext_vector_type(4)));
typedef uint32_t u2 __attribute__((ext_vector_type(2)));

constexpr int WG_WAVES = 8;
constexpr int WG_THREADS = WG_WAVES * 64;
constexpr int LDS_BUDGET = 64 * 1024;

// ------------------------------------------------------------------------------------------------ small helpers
__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
__device__ __forceinline__ float f16_bits_to_float(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {   // round to nearest even
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
  return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float load_elem(const void* p, int dtype, size_t idx) {
  if (dtype == HTR_BF16) return bf16_bits_to_float(((const uint16_t*)p)[idx]);
  if (dtype == HTR_F16) return f16_bits_to_float(((const uint16_t*)p)[idx]);
  return ((const float*)p)[idx];
}
__device__ __forceinline__ void store_elem(void* p, int dtype, size_t idx, float v) {
  if (dtype == HTR_BF16) ((uint16_t*)p)[idx] = float_to_bf16_bits(v);
  else if (dtype == HTR_F16) ((uint16_t*)p)[idx] = __builtin_bit_cast(uint16_t, (_Float16)v);
  else ((float*)p)[idx] = v;
}
__device__ __forceinline__ float sign_of(const uint8_t* bits, int j) { return ((bits[j >> 3] >> (j & 7)) & 1) ? -1.f : 1.f; }
// ---- cross-lane exchange without LDS round trips: DPP for lane xor 1, 2, 4, 8; gfx950 row swaps for 16 and 32
template <int CTRL> __device__ __forceinline__ float dpp_mov(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
template <int H> __device__ __forceinline__ float lane_xor_dpp(float v) {
  if constexpr (H == 1) return dpp_mov<0xB1>(v);                   // quad_perm [1,0,3,2]
  else if constexpr (H == 2) return dpp_mov<0x4E>(v);              // quad_perm [2,3,0,1]
  else if constexpr (H == 4) return dpp_mov<0x141>(dpp_mov<0x1B>(v));   // quad reverse (xor 3) then row_half_mirror (xor 7)
  else return dpp_mov<0x128>(v);                                   // row_ror:8 == xor 8 inside a row of 16
}
// values of the two 16-lane (or 32-lane) halves that lane and lane ^ 16 (^ 32) belong to: first = even half's value,
// second = odd half's value, both seen from every lane of the pair
typedef uint32_t u2s __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void halves16(float v, float& even, float& odd) {
  const uint32_t u = __float_as_uint(v);
  const u2s r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  even = __uint_as_float(r.x); odd = __uint_as_float(r.y);
}
__device__ __forceinline__ void halves32(float v, float& even, float& odd) {
  const uint32_t u = __float_as_uint(v);
  const u2s r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  even = __uint_as_float(r.x); odd = __uint_as_float(r.y);
}
// One butterfly stage between lanes l and l ^ H: the lane with bit H clear gets a + partner, the other partner - a,
// i.e. a' = partner + s * a with s = +1 / -1 by that lane bit.
template <int H> __device__ __forceinline__ void butterfly_dpp(float& a, float s) {
  a = __builtin_fmaf(a, s, lane_xor_dpp<H>(a));
}
// rows / halves stages: both values of the pair are visible after the swap; a' = even + s * odd
__device__ __forceinline__ void butterfly16(float& a, float s) { float e, o; halves16(a, e, o); a = __builtin_fmaf(o, s, e); }
__device__ __forceinline__ void butterfly32(float& a, float s) { float e, o; halves32(a, e, o); a = __builtin_fmaf(o, s, e); }

// 128-point Walsh-Hadamard butterfly network over one wave: lane holds elements `lane` (a) and `lane + 64` (b).
// For the stages that fetch the partner (xor 1..8) the sign belongs to the lane's own value; for the swap stages
// (16, 32) both lanes see (even, odd) and the odd-side lane takes the difference.
__device__ __forceinline__ void fwht128_wave(float& a, float& b, int lane) {
  const float t = a + b; b = a - b; a = t;
  const float s1 = (lane & 1) ? -1.f : 1.f, s2 = (lane & 2) ? -1.f : 1.f, s4 = (lane & 4) ? -1.f : 1.f;
  const float s8 = (lane & 8) ? -1.f : 1.f, s16 = (lane & 16) ? -1.f : 1.f, s32 = (lane & 32) ? -1.f : 1.f;
  butterfly_dpp<1>(a, s1); butterfly_dpp<1>(b, s1);
  butterfly_dpp<2>(a, s2); butterfly_dpp<2>(b, s2);
  butterfly_dpp<4>(a, s4); butterfly_dpp<4>(b, s4);
  butterfly_dpp<8>(a, s8); butterfly_dpp<8>(b, s8);
  butterfly16(a, s16); butterfly16(b, s16);
  butterfly32(a, s32); butterfly32(b, s32);
}
// all-lanes reductions over the wave, fixed order
__device__ __forceinline__ float wave_sum(float v) {
  v += lane_xor_dpp<1>(v); v += lane_xor_dpp<2>(v); v += lane_xor_dpp<4>(v); v += lane_xor_dpp<8>(v);
  float e, o;
  halves16(v, e, o); v = e + o;
  halves32(v, e, o); return e + o;
}
// sums of v over the lanes with (lane & 16) == 0 and over those with (lane & 16) != 0, in every lane
__device__ __forceinline__ void wave_sum_by_row_parity(float v, float& even_rows, float& odd_rows) {
  v += lane_xor_dpp<1>(v); v += lane_xor_dpp<2>(v); v += lane_xor_dpp<4>(v); v += lane_xor_dpp<8>(v);   // per 16-lane row
  float lo, hi;
  halves32(v, lo, hi);          // lo: rows 0/1 as seen from the lane's position in its half, hi: rows 2/3
  const float s = lo + hi;      // row 0 + row 2 in even rows' lanes, row 1 + row 3 in odd rows' lanes
  float e, o;
  halves16(s, e, o);
  even_rows = e; odd_rows = o;
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, lane_xor_dpp<1>(v)); v = fmaxf(v, lane_xor_dpp<2>(v)); v = fmaxf(v, lane_xor_dpp<4>(v)); v = fmaxf(v, lane_xor_dpp<8>(v));
  float e, o;
  halves16(v, e, o); v = fmaxf(e, o);
  halves32(v, e, o); return fmaxf(e, o);
}

// ------------------------------------------------------------------------------------------------ stream loads
// The K dwords of lane `lane` start at dword lane*K of the wave's 64*K-dword step: contiguous across the wave.
template <int K> struct StreamRegs { uint32_t d[K]; };

template <int K> __device__ __forceinline__ void load_stream(const uint32_t* __restrict__ p, StreamRegs<K>& r) {
  if constexpr (K == 2) {
    u2 v = __builtin_nontemporal_load((const u2*)p); r.d[0] = v.x; r.d[1] = v.y;
  } else if constexpr (K == 4) {
    u4 v = __builtin_nontemporal_load((const u4*)p); r.d[0] = v.x; r.d[1] = v.y; r.d[2] = v.z; r.d[3] = v.w;
  } else if constexpr (K == 8) {
    u4 v = __builtin_nontemporal_load((const u4*)p), w = __builtin_nontemporal_load((const u4*)p + 1);
    r.d[0] = v.x; r.d[1] = v.y; r.d[2] = v.z; r.d[3] = v.w; r.d[4] = w.x; r.d[5] = w.y; r.d[6] = w.z; r.d[7] = w.w;
  } else if constexpr (K == 6) {
    const u2* q = (const u2*)p;
    u2 a = __builtin_nontemporal_load(q), b = __builtin_nontemporal_load(q + 1), c = __builtin_nontemporal_load(q + 2);
    r.d[0] = a.x; r.d[1] = a.y; r.d[2] = b.x; r.d[3] = b.y; r.d[4] = c.x; r.d[5] = c.y;
  } else {
#pragma unroll
    for (int k = 0; k < K; ++k) r.d[k] = __builtin_nontemporal_load(p + k);
  }
}

// ------------------------------------------------------------------------------------------------ decode core
// V[0] = the dword before the lane's first dword (history), V[1..K] = the lane's dwords.  Local step u (0..31) is
// trellis step t = 32q + u; its state is the 16 bits of V that start at bit 16 + (u + 1) * K (bit 0 = MSB of V[0]).
template <int K> struct Window {
  uint32_t V[K + 1];
  uint32_t mid[K];     // mid[w] = bits [32w + 16, 32w + 48) of V, for windows that straddle two dwords
  __device__ __forceinline__ void build(const StreamRegs<K>& r, uint32_t prev) {
    V[0] = prev;
#pragma unroll
    for (int k = 0; k < K; ++k) V[k + 1] = r.d[k];
#pragma unroll
    for (int k = 0; k < K; ++k) mid[k] = __builtin_amdgcn_alignbit(V[k], V[k + 1], 16);
  }
  template <int U> __device__ __forceinline__ uint32_t state() const {
    constexpr int b = 16 + (U + 1) * K, w = b >> 5, off = b & 31;
    if constexpr (off <= 16) return (V[w] >> (16 - off)) & 0xFFFFu;
    else return (mid[w] >> (32 - off)) & 0xFFFFu;
  }
  // generator word x = s*A + B; s < 2^16 and A < 2^24 so this is one v_mad_u32_u24
  template <int U> __device__ __forceinline__ uint32_t genword() const { return state<U>() * GEN_A + GEN_B; }
  // two consecutive weights as packed halves (1534 + v(u), 1534 + v(u + 1))
  template <int U> __device__ __forceinline__ uint32_t pair_f16() const {
    uint32_t r = __builtin_amdgcn_sad_u8(genword<U>(), 0u, 0x64006400u);
    return __builtin_amdgcn_sad_hi_u8(genword<U + 1>(), 0u, r);
  }
  template <int U> __device__ __forceinline__ int value() const {   // integer v(s)
    return (int)__builtin_amdgcn_sad_u8(genword<U>(), 0u, 0u) - 510;
  }
  template <int U0> __device__ __forceinline__ h8 group8() const {   // 8 consecutive weights as an MFMA operand
    u4 v = {pair_f16<U0>(), pair_f16<U0 + 2>(), pair_f16<U0 + 4>(), pair_f16<U0 + 6>()};
    return __builtin_bit_cast(h8, v);
  }
};

// lane that holds the dword preceding this lane's first dword: previous row pair of the same tile, circular
__device__ __forceinline__ int history_lane_byteaddr(int lane) { return ((lane & ~7) | ((lane - 1) & 7)) << 2; }

// ------------------------------------------------------------------------------------------------ fused linear
// The step space of one linear is (128-row block rb, 128-column block blk), row-major: virtual step v = rb * nblk + blk.
// It is cut into equal contiguous chunks, one per workgroup, so the workgroup count can be a multiple of the CU count
// whatever the shape.  A chunk may end inside a row block and continue in the next one; each piece of a row block a
// chunk covers is a "segment" and yields one partial.
struct LinearArgs {
  const uint32_t* qw;
  const uint16_t* scales;
  const uint8_t* su;
  const uint8_t* sv;
  const void* x;
  const void* bias;
  void* y;
  uint32_t* cnt;    // [m/128] arrival counters (election by counter only); zero on entry and on exit
  float* part;      // [workgroups][segmax][2][M][128] partials per segment and tile parity; all-zero on entry and on exit
  int m, n, M;
  const _Float16* xt_g;   // pre-rotated activations [M][n] f16 (only when prerot)
  const float* xs_g;      // their per-(row, block, tile parity) sums [M][n/128][2]
  const float* sc_g;      // per-row activation scale [M]
  int prerot;             // 1: x~ was produced by k_rotate; 0: this kernel rotates its own column blocks
  int chunk;        // virtual steps per workgroup
  int segmax;       // partial slots reserved per workgroup
  int by_counter;   // 1: elect the finisher of a row block with an arrival counter; 0: by reading every contributor's slot
  int x_dtype, y_dtype;
  float cbscale;
};

constexpr int MAX_SEG = 64;    // row-block segments one workgroup may produce
constexpr int PAIR_REGS = 4;   // (activation row, 128-column block) pairs a wave keeps in registers across the barrier

// LDS layout (dynamic): [xt: (M + 1) rows x row_halves f16][pmax: M * nbl f32][xs: M * nbl * 2 f32 (per tile parity)][sc: M f32]
// nbl = number of distinct column blocks a chunk touches = min(chunk, n / 128)
// One rotated 128-column block is stored as [columns 0..7 of tiles 0..7][columns 8..15 of tiles 0..7] (2 x 64 halves), and
// rows are padded by 16 halves: the 16-byte B-operand reads of 8 consecutive lanes (4 activation rows x 2 tile parities)
// then cover 128 contiguous-mod-128 bytes, i.e. every LDS bank once.
__host__ __device__ inline int xt_row_halves(int nbl) { return nbl * 128 + 16; }
__device__ __forceinline__ int xt_slot(int j) { return ((j >> 3) & 1) * 64 + (j >> 4) * 8 + (j & 7); }   // element j of a block
__host__ __device__ inline size_t lds_bytes(int M, int nbl) {
  return (size_t)(M + 1) * xt_row_halves(nbl) * 2 + (size_t)M * nbl * 4 * 3 + (size_t)M * 4;
}

// power-of-two activation scale 2^e with sqrt(128) * amax / 2^e in (8192, 16384]: |H128 x| / sqrt(128) <= sqrt(128) * max|x|,
// so the rotated activations neither overflow f16 nor fall into its denormals
__device__ __forceinline__ int scale_exponent(float amax) {
  const int ex = (int)((__float_as_uint(amax * SQRT128) >> 23) & 0xFFu);
  if (ex == 0 || ex == 255) return 0;
  return max(-100, ex - 127 - 13);
}
__device__ __forceinline__ float pow2f(int e) { return __uint_as_float((uint32_t)(127 + e) << 23); }

// Rotation of all activation rows ahead of the linear kernel (used from 3 rows up, where every workgroup rotating its
// own column blocks would repeat the same work hundreds of times): one workgroup per row.
__global__ __launch_bounds__(WG_THREADS) void k_rotate(const void* __restrict__ x, const uint8_t* __restrict__ su, int n, int x_dtype,
                                                       _Float16* __restrict__ xt_g, float* __restrict__ xs_g, float* __restrict__ sc_g) {
  __shared__ float s_max[WG_WAVES];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, mrow = blockIdx.x, nblk = n >> 7;
  const size_t row = (size_t)mrow * n;
  float mx = 0.f;
  for (int i = threadIdx.x; i < n; i += WG_THREADS) mx = fmaxf(mx, fabsf(load_elem(x, x_dtype, row + i)));
  mx = wave_max(mx);
  if (lane == 0) s_max[w] = mx;
  __syncthreads();
  float amax = 0.f;
#pragma unroll
  for (int k = 0; k < WG_WAVES; ++k) amax = fmaxf(amax, s_max[k]);
  const int e = scale_exponent(amax);
  const float inv_sc = pow2f(-e);
  if (threadIdx.x == 0) sc_g[mrow] = pow2f(e);
  for (int blk = w; blk < nblk; blk += WG_WAVES) {
    const int col = blk * 128;
    float va = load_elem(x, x_dtype, row + col + lane) * sign_of(su, col + lane) * inv_sc;
    float vb = load_elem(x, x_dtype, row + col + lane + 64) * sign_of(su, col + lane + 64) * inv_sc;
    fwht128_wave(va, vb, lane);
    const _Float16 ha = (_Float16)(va * INV_SQRT128), hb = (_Float16)(vb * INV_SQRT128);
    xt_g[row + col + lane] = ha;
    xt_g[row + col + lane + 64] = hb;
    float se, so;
    wave_sum_by_row_parity((float)ha + (float)hb, se, so);
    if (lane == 0) { xs_g[((size_t)mrow * nblk + blk) * 2] = se; xs_g[((size_t)mrow * nblk + blk) * 2 + 1] = so; }
  }
}

template <int K> struct DecodedStep { h8 a[4]; };   // MFMA A operands of one step: (row 2q | 2q+1) x (columns 0..7 | 8..15)

template <int K> __device__ __forceinline__ void decode_step(const StreamRegs<K>& r, int hist, DecodedStep<K>& d) {
  Window<K> win;
  win.build(r, (uint32_t)__builtin_amdgcn_ds_bpermute(hist, (int)r.d[K - 1]));
  d.a[0] = win.template group8<0>();
  d.a[1] = win.template group8<8>();
  d.a[2] = win.template group8<16>();
  d.a[3] = win.template group8<24>();
}

template <int K, int MB, int P, int PRE, bool PREROT>
__global__ __launch_bounds__(WG_THREADS) void k_linear(const LinearArgs a) {
  static_assert(PRE <= P, "pre-decoded steps come out of the prefetch registers");
  extern __shared__ __align__(16) unsigned char lds[];
  __shared__ int s_finish[MAX_SEG];
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));   // wave index, provably uniform: keeps the
                                                                           // strip addressing on the scalar unit
  const int nblk = a.n >> 7, rbs = a.m >> 7;
  const int M = a.M;
  const int vtotal = rbs * nblk;
  const int v0 = blockIdx.x * a.chunk, nsteps = min(vtotal, v0 + a.chunk) - v0;
  const int rb_first = v0 / nblk, c0 = v0 - rb_first * nblk;     // first row block and first column block of the chunk
  const bool all_blocks = nsteps >= nblk;                        // chunk touches every column block
  const int nbl = all_blocks ? nblk : nsteps;                    // distinct column blocks; LDS slot of block b:
  const int rowh = xt_row_halves(min(a.chunk, nblk));            //   b if all_blocks, else (b - c0) mod nblk

  _Float16* xt = (_Float16*)lds;
  float* s_pmax = (float*)(lds + (size_t)(M + 1) * rowh * 2);
  float* s_xs = s_pmax + M * min(a.chunk, nblk);
  float* s_sc = s_xs + 2 * M * min(a.chunk, nblk);     // activation scale per row

  // ---- input rotation of the chunk's column blocks: x~ = f16( H128(su . x) / sqrt(128) / sc ), sc a power of two per
  // activation row.  Pass 1 loads x (sign applied) and publishes max|x| per (row, block); pass 2 rotates, scales, converts.
  const int npairs = M * nbl;
  auto pair_col = [&](int li) { int b = all_blocks ? li : c0 + li; if (b >= nblk) b -= nblk; return b * 128; };
  float xa[PAIR_REGS], xb[PAIR_REGS];
  constexpr bool prerot = PREROT;   // x~ comes from k_rotate instead of being rotated here
  for (int i = threadIdx.x; i < rowh / 2; i += WG_THREADS) ((uint32_t*)(xt + (size_t)M * rowh))[i] = 0u;   // zero row
  // with pre-rotated activations: 16-byte pieces of this chunk's x~ slice, issued before the weight stream
  constexpr int COPY_REGS = 4;
  u4 cp[COPY_REGS];
  const int ncopy = npairs * 16;                 // 16 pieces of 8 halves per (row, block) pair
  if constexpr (prerot) {
#pragma unroll
    for (int t = 0; t < COPY_REGS; ++t) {
      const int ci = threadIdx.x + t * WG_THREADS;
      if (ci < ncopy) {
        const int pi = ci >> 4, mrow = pi / nbl, li = pi - mrow * nbl;
        cp[t] = *(const u4*)(a.xt_g + (size_t)mrow * a.n + pair_col(li) + (ci & 15) * 8);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < PAIR_REGS; ++t) {     // x first: loads return in order, and x heads the longest dependency chain
    const int pi = w + t * WG_WAVES;
    xa[t] = 0.f; xb[t] = 0.f;
    if (!prerot && pi < npairs) {
      const int mrow = pi / nbl, li = pi - mrow * nbl, col = pair_col(li);
      const size_t base = (size_t)mrow * a.n + col;
      xa[t] = load_elem(a.x, a.x_dtype, base + lane) * sign_of(a.su, col + lane);
      xb[t] = load_elem(a.x, a.x_dtype, base + lane + 64) * sign_of(a.su, col + lane + 64);
    }
  }

  // ---- start the weight stream.  This wave's strip of row block rb is tile row rb * 8 + w; its 8 tiles of column
  // block blk are 64 * K contiguous dwords; a strip is contiguous over blk, the same strip of the next row block
  // starts 8 strips later.
  constexpr int STEP_DWORDS = 64 * K;
  const size_t strip_dwords = (size_t)nblk * STEP_DWORDS;
  const uint32_t* pf_ptr = a.qw + (size_t)(rb_first * 8 + w) * strip_dwords + (size_t)c0 * STEP_DWORDS;   // uniform
  const int lane_dwords = lane * K;
  int pf_blk = c0;
  StreamRegs<K> buf[P];
  auto prefetch = [&](StreamRegs<K>& dst) {
    load_stream<K>(pf_ptr + lane_dwords, dst);
    pf_ptr += STEP_DWORDS;
    if (++pf_blk == nblk) { pf_blk = 0; pf_ptr += 7 * strip_dwords; }
  };
  const bool rotator = !prerot && w < npairs;      // this wave rotates at least one pair
  if constexpr (prerot) {
#pragma unroll
    for (int p = 0; p < P; ++p)
      if (p < nsteps) prefetch(buf[p]);
  }
  if constexpr (!prerot) {
#pragma unroll
  for (int t = 0; t < PAIR_REGS; ++t) {
    const int pi = w + t * WG_WAVES;
    if (pi < npairs) {
      const float mx = wave_max(fmaxf(fabsf(xa[t]), fabsf(xb[t])));
      if (lane == 0) s_pmax[pi] = mx;
    }
  }
  // The weight stream starts only now, after x has arrived: when every wave of the chip bursts its first weight loads
  // at once, an x load issued just before them takes about twice as long, and x heads the critical chain, while the
  // rotation below hides the weight latency anyway.
  asm volatile("" ::: "memory");
#pragma unroll
  for (int p = 0; p < P; ++p)
    if (p < nsteps) prefetch(buf[p]);
  for (int pi = w + PAIR_REGS * WG_WAVES; pi < npairs; pi += WG_WAVES) {   // more pairs than registers: max only, reload later
    const int mrow = pi / nbl, li = pi - mrow * nbl;
    const size_t base = (size_t)mrow * a.n + pair_col(li);
    const float mx = wave_max(fmaxf(fabsf(load_elem(a.x, a.x_dtype, base + lane)), fabsf(load_elem(a.x, a.x_dtype, base + lane + 64))));
    if (lane == 0) s_pmax[pi] = mx;
  }
  __syncthreads();
  // max|x| of activation row mrow over the chunk's blocks: lanes read the per-block maxima, one wave reduction
  auto row_amax = [&](int mrow) {
    float v = 0.f;
    for (int k = lane; k < nbl; k += 64) v = fmaxf(v, s_pmax[mrow * nbl + k]);
    return wave_max(v);
  };
  auto rotate_pair = [&](int pi, float va, float vb) {
    const int mrow = pi / nbl, li = pi - mrow * nbl;
    const int e = scale_exponent(row_amax(mrow));
    const float inv_sc = pow2f(-e);
    if (li == 0 && lane == 0) s_sc[mrow] = pow2f(e);
    va *= inv_sc; vb *= inv_sc;
    fwht128_wave(va, vb, lane);
    const _Float16 ha = (_Float16)(va * INV_SQRT128), hb = (_Float16)(vb * INV_SQRT128);
    xt[(size_t)mrow * rowh + li * 128 + xt_slot(lane)] = ha;
    xt[(size_t)mrow * rowh + li * 128 + xt_slot(lane + 64)] = hb;
    // sum of the rounded x~ per tile parity (element j sits in tile j / 16; lane and lane + 64 share the parity)
    float se, so;
    wave_sum_by_row_parity((float)ha + (float)hb, se, so);
    if (lane == 0) { s_xs[2 * pi] = se; s_xs[2 * pi + 1] = so; }
  };
  // The rotation is a long chain of dependent instructions that every wave of the workgroup waits for: run it at
  // raised priority so that decoding waves on the same SIMD do not starve it.
  __builtin_amdgcn_s_setprio(3);
#pragma unroll
  for (int t = 0; t < PAIR_REGS; ++t) {   // unrolled: the chains of a wave's pairs interleave
    const int pi = w + t * WG_WAVES;
    if (pi < npairs) rotate_pair(pi, xa[t], xb[t]);
  }
  for (int pi = w + PAIR_REGS * WG_WAVES; pi < npairs; pi += WG_WAVES) {
    const int mrow = pi / nbl, li = pi - mrow * nbl, col = pair_col(li);
    const size_t base = (size_t)mrow * a.n + col;
    rotate_pair(pi, load_elem(a.x, a.x_dtype, base + lane) * sign_of(a.su, col + lane),
                load_elem(a.x, a.x_dtype, base + lane + 64) * sign_of(a.su, col + lane + 64));
  }
  __builtin_amdgcn_s_setprio(0);

  } else {
    // copy the slice into LDS; sums per (row, block, parity) come with it
#pragma unroll
    for (int t = 0; t < COPY_REGS; ++t) {
      const int ci = threadIdx.x + t * WG_THREADS;
      if (ci < ncopy) {
        const int pi = ci >> 4, mrow = pi / nbl, li = pi - mrow * nbl;
        *(u4*)(xt + (size_t)mrow * rowh + li * 128 + (ci & 1) * 64 + ((ci & 15) >> 1) * 8) = cp[t];
      }
    }
    for (int ci = threadIdx.x + COPY_REGS * WG_THREADS; ci < ncopy; ci += WG_THREADS) {
      const int pi = ci >> 4, mrow = pi / nbl, li = pi - mrow * nbl;
      *(u4*)(xt + (size_t)mrow * rowh + li * 128 + (ci & 1) * 64 + ((ci & 15) >> 1) * 8) =
          *(const u4*)(a.xt_g + (size_t)mrow * a.n + pair_col(li) + (ci & 15) * 8);
    }
    for (int i = threadIdx.x; i < npairs * 2; i += WG_THREADS) {
      const int pi = i >> 1, mrow = pi / nbl, li = pi - mrow * nbl;
      s_xs[i] = a.xs_g[((size_t)mrow * nblk + (pair_col(li) >> 7)) * 2 + (i & 1)];
    }
  }
  // ---- decode the first steps into registers.  Waves that rotate nothing do it before the x~ barrier, while the
  // rotating waves sit in their dependency chains, so the rotation latency is not dead time; rotating waves go to
  // the barrier at once and decode the same steps after it.
  const int hist = history_lane_byteaddr(lane);
  DecodedStep<K> pre[PRE];
  auto predecode = [&]() {
#pragma unroll
    for (int p = 0; p < PRE; ++p)
      if (p < nsteps) {
        decode_step<K>(buf[p], hist, pre[p]);
        if (p + P < nsteps) prefetch(buf[p]);
      }
  };
  // (when most waves rotate, the few that do not would only delay the barrier by decoding first)
  const bool early = !rotator && npairs <= WG_WAVES / 2;
  if (early) predecode();
  __syncthreads();
  if (!early) predecode();

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
      if constexpr (prerot) sc[mb] = a.sc_g[mrow];
      else sc[mb] = s_sc[mrow];
    }
  }
  const size_t slot_floats = (size_t)2 * M * 128;          // one segment: [parity][M][128]
  float* myslot = a.part + (size_t)blockIdx.x * a.segmax * slot_floats + 16 * w + 8 * (g & 1);

  f4 acc[MB][2];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) { acc[mb][0] = f4{0.f, 0.f, 0.f, 0.f}; acc[mb][1] = f4{0.f, 0.f, 0.f, 0.f}; }

  int cur_blk = c0, cur_li = all_blocks ? c0 : 0, cur_seg = 0, done = 0;
  auto consume = [&](const DecodedStep<K>& d) {
    h8 B0[MB], B1[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const _Float16* bp = xt + boff[mb] + cur_li * 128;
      B0[mb] = *(const h8*)bp;
      B1[mb] = *(const h8*)(bp + 64);
      if (xsoff[mb] >= 0) offs[mb] += 1534.f * s_xs[xsoff[mb] + 2 * cur_li];
    }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[0], B0[mb], acc[mb][0], 0, 0, 0);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[1], B1[mb], acc[mb][0], 0, 0, 0);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[2], B0[mb], acc[mb][1], 0, 0, 0);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[mb][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[3], B1[mb], acc[mb][1], 0, 0, 0);
    ++done; ++cur_blk; ++cur_li;
    const bool row_end = cur_blk == nblk;
    if (row_end || done == nsteps) {
      // end of a segment: this wave's strip partials, one per tile parity, with the 1534 offset removed and the
      // activation scale undone.  Stored with the lowest mantissa bit set (never the all-zero pattern), device scope
      // (written through), not waited for here.
      float* dst0 = myslot + (size_t)cur_seg * slot_floats;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int mrow = mb * 8 + (n16 >> 1);
        if (xsoff[mb] >= 0) {
          uint32_t* dst = (uint32_t*)(dst0 + (size_t)(par * M + mrow) * 128);
#pragma unroll
          for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int rr = 0; rr < 2; ++rr)
              __hip_atomic_store(dst + 2 * j + rr, __float_as_uint((acc[mb][rr][j] - offs[mb]) * sc[mb]) | 1u,
                                 __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        acc[mb][0] = f4{0.f, 0.f, 0.f, 0.f}; acc[mb][1] = f4{0.f, 0.f, 0.f, 0.f};
        offs[mb] = 0.f;
      }
      ++cur_seg;
      if (row_end) { cur_blk = 0; if (all_blocks) cur_li = 0; }
    }
  };

#pragma unroll
  for (int p = 0; p < PRE; ++p)
    if (p < nsteps) consume(pre[p]);

  // ---- main loop: one 128-column block (8 tiles of this wave's strip) per step; buffer p holds step v with v % P == p
  for (int vb = PRE; vb < nsteps; vb += P) {
#pragma unroll
    for (int pp = 0; pp < P; ++pp) {
      constexpr int dummy = 0; (void)dummy;
      const int p = (PRE + pp) % P;
      const int v = vb + pp;
      if (v < nsteps) {
        DecodedStep<K> d;
        decode_step<K>(buf[p], hist, d);
        if (v + P < nsteps) prefetch(buf[p]);
        consume(d);
      }
    }
  }

  // ---- cross-workgroup reduction.  The workspace is all-zero between calls.  Device-scope stores are acknowledged
  // once written through, so after the wait and the barrier every partial of this workgroup is visible device-wide
  // (a cache-wide writeback would also do, at many times the cost).
  //   election by slots:   for each row block it touched the workgroup reads the slots of every contributing chunk;
  //                        if none is zero all have arrived and it finishes the row block.  Several workgroups may
  //                        see a complete set; they compute bit-identical results (fixed summation order) and store
  //                        the same values.
  //   election by counter: one arrival per workgroup and row block; the last one finishes.  Same-address atomics
  //                        serialise, so this is used only where re-reading the slots would cost more.
  // Either way the finisher zeroes what it consumed.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  const int nseg = cur_seg;
  if (a.by_counter) {
    if ((int)threadIdx.x < nseg) {
      const int rb = rb_first + threadIdx.x;
      const int j0 = (rb * nblk) / a.chunk, j1 = (rb * nblk + nblk - 1) / a.chunk;
      s_finish[threadIdx.x] = __hip_atomic_fetch_add(&a.cnt[rb], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (uint32_t)(j1 - j0);
    }
    __syncthreads();
    if ((int)threadIdx.x < nseg && s_finish[threadIdx.x])
      __hip_atomic_store(&a.cnt[rb_first + threadIdx.x], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  for (int idx = w; idx < nseg * M; idx += WG_WAVES) {
    const int seg = idx / M, mrow = idx - seg * M, rb = rb_first + seg;
    if (a.by_counter && !s_finish[seg]) continue;
    const int r0 = rb * 128 + lane, r1 = r0 + 64;
    const float rs0 = f16_bits_to_float(a.scales[r0]) * a.cbscale, rs1 = f16_bits_to_float(a.scales[r1]) * a.cbscale;
    const float sg0 = sign_of(a.sv, r0), sg1 = sign_of(a.sv, r1);
    float b0v = 0.f, b1v = 0.f;
    if (a.bias != nullptr) { b0v = load_elem(a.bias, a.y_dtype, r0); b1v = load_elem(a.bias, a.y_dtype, r1); }
    // contributors: chunks j0..j1 overlap row block rb; chunk j holds it in its segment rb - (first row block of j)
    const int j0 = (rb * nblk) / a.chunk, j1 = (rb * nblk + nblk - 1) / a.chunk;
    const int sj0 = rb - (j0 * a.chunk) / nblk;              // every later contributor starts inside rb: segment 0
    float v0s = 0.f, v1s = 0.f;
    bool missing = false;
    auto slot_of = [&](int j) {
      return (uint32_t*)(a.part + ((size_t)j * a.segmax + (j == j0 ? sj0 : 0)) * slot_floats + (size_t)mrow * 128);
    };
#pragma unroll 8
    for (int j = j0; j <= j1; ++j) {
      const uint32_t* pp = slot_of(j);
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        const uint32_t u0 = __hip_atomic_load(pp + (size_t)pr * M * 128 + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t u1 = __hip_atomic_load(pp + (size_t)pr * M * 128 + lane + 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        missing |= (u0 == 0u) | (u1 == 0u);
        v0s += __uint_as_float(u0); v1s += __uint_as_float(u1);
      }
    }
    if (__any(missing)) continue;             // some contributor has not arrived yet: a later workgroup finishes this row
    for (int j = j0; j <= j1; ++j) {          // leave the workspace zero for the next call
      uint32_t* pp = slot_of(j);
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        __hip_atomic_store(pp + (size_t)pr * M * 128 + lane, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(pp + (size_t)pr * M * 128 + lane + 64, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    v0s *= rs0; v1s *= rs1;
    fwht128_wave(v0s, v1s, lane);
    v0s = v0s * INV_SQRT128 * sg0 + b0v;
    v1s = v1s * INV_SQRT128 * sg1 + b1v;
    store_elem(a.y, a.y_dtype, (size_t)mrow * a.m + r0, v0s);
    store_elem(a.y, a.y_dtype, (size_t)mrow * a.m + r1, v1s);
  }
}

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
// W = Sv . Ho . Q . Hi . Su as bf16 [m, n] (htr/wire.py:105-113 of the reference), one workgroup per 128x128 block:
// decode the 64 tiles into LDS as float32 (row scale * CBSCALE applied), H128 down the columns (Ho), H128 along the
// rows (Hi), signs, 1/128, round to bf16.  The row pass is last so that the stores are row-contiguous.
constexpr int DQW_LD = 129;   // LDS leading dimension in floats: odd, so column walks hit distinct banks

template <int K>
__global__ __launch_bounds__(512) void k_dequant_w(const uint32_t* __restrict__ qw, const uint16_t* __restrict__ scales,
                                                   const uint8_t* __restrict__ su, const uint8_t* __restrict__ sv,
                                                   uint16_t* __restrict__ W, int nt, float cbscale) {
  extern __shared__ __align__(16) unsigned char lds[];
  float* blk = (float*)lds;                                  // [128][DQW_LD]
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int bj = blockIdx.x, bi = blockIdx.y;                // 128-column block, 128-row block
  const int n = nt * 16;
  // thread = (tile in block, row pair q): 64 tiles x 8 = 512 threads; a tile's 8 threads are consecutive lanes
  {
    const int t64 = threadIdx.x >> 3, q = threadIdx.x & 7;
    const int ti = t64 >> 3, tj = t64 & 7;                   // tile row / column inside the block
    const size_t tile = (size_t)(bi * 8 + ti) * nt + (size_t)bj * 8 + tj;
    StreamRegs<K> r;
    load_stream<K>(qw + tile * (8 * K) + q * K, r);
    Window<K> win;
    win.build(r, (uint32_t)__builtin_amdgcn_ds_bpermute(history_lane_byteaddr(lane), (int)r.d[K - 1]));
    const int row0 = ti * 16 + 2 * q;
    const float s0 = f16_bits_to_float(scales[bi * 128 + row0]) * cbscale;
    const float s1 = f16_bits_to_float(scales[bi * 128 + row0 + 1]) * cbscale;
    float* o0 = blk + row0 * DQW_LD + tj * 16;
    float* o1 = o0 + DQW_LD;
    ForEach32<K, 0>::run(win, [&](int u, int v) {
      if (u < 16) o0[u] = (float)v * s0; else o1[u - 16] = (float)v * s1;
    });
  }
  __syncthreads();
  // Ho: transform every column (wave w takes columns w, w + 8, ...; lane holds rows lane and lane + 64)
  for (int c = w; c < 128; c += 8) {
    float a = blk[lane * DQW_LD + c], b = blk[(lane + 64) * DQW_LD + c];
    fwht128_wave(a, b, lane);
    blk[lane * DQW_LD + c] = a;
    blk[(lane + 64) * DQW_LD + c] = b;
  }
  __syncthreads();
  // Hi along every row, then signs and 1/128 (both rotations' 1/sqrt(128)), bf16 store
  const float su0 = sign_of(su, bj * 128 + lane), su1 = sign_of(su, bj * 128 + lane + 64);
  for (int r = w; r < 128; r += 8) {
    float a = blk[r * DQW_LD + lane], b = blk[r * DQW_LD + lane + 64];
    fwht128_wave(a, b, lane);
    const float sg = sign_of(sv, bi * 128 + r) * (1.0f / 128.0f);
    uint16_t* dst = W + (size_t)(bi * 128 + r) * n + (size_t)bj * 128;
    dst[lane] = float_to_bf16_bits(a * sg * su0);
    dst[lane + 64] = float_to_bf16_bits(b * sg * su1);
  }
}

// ------------------------------------------------------------------------------------------------ host side
thread_local int g_last_hip_error = 0;

struct Plan { int chunk, wgs, segmax, nbl, mb, by_counter, prerot; size_t lds; };

constexpr int PREROT_MIN_M = 6;   // from this many rows on the activations are rotated once by k_rotate
// The pre-rotated activations live in a fixed region between the counters and the partial slots: partial slots must be
// all-zero between calls, and no call may leave other data where a later call of another shape expects such slots.
constexpr size_t PREROT_REGION = (size_t)4 << 20;
inline size_t align256(size_t v) { return (v + 255) / 256 * 256; }
// bytes of the pre-rotated activations, their block sums and the row scales
inline size_t prerot_bytes(int n, int M) { return align256((size_t)M * n * 2) + align256((size_t)M * (n / 128) * 8) + align256((size_t)M * 4); }

constexpr int NUM_CU = 256;
constexpr int MAX_ROW_BLOCKS = 16384;                       // counter region: one word per 128-row block
inline size_t counters_bytes() { return (size_t)MAX_ROW_BLOCKS * 4; }

inline bool plan_for_chunk(int m, int n, int M, int chunk, Plan& pl) {
  const int nblk = n / 128, rbs = m / 128;
  const long vtotal = (long)rbs * nblk;
  if (chunk < 1 || chunk > vtotal) return false;
  pl.chunk = chunk;
  pl.wgs = (int)((vtotal + chunk - 1) / chunk);
  pl.segmax = chunk == 1 ? 1 : (chunk + nblk - 2) / nblk + 1;
  pl.nbl = chunk < nblk ? chunk : nblk;
  pl.lds = lds_bytes(M, pl.nbl);
  if (pl.segmax > MAX_SEG || pl.lds > (size_t)LDS_BUDGET) return false;
  // bytes a workgroup re-reads when finishers are elected by slots: per segment, every contributor's two parities
  const int contributors = chunk >= nblk ? 2 : (nblk + chunk - 1) / chunk + 1;
  const double slot_kb = (double)pl.segmax * contributors * 2 * M * 0.5;
  pl.by_counter = slot_kb > 96.0 ? 1 : 0;
  // pre-rotation also pays for few rows when every wave would otherwise rotate four or more (row, block) pairs in
  // each of very many workgroups (output heads: 152064x4096 runs 9 % faster with it)
  const bool redundant = (M * pl.nbl + 7) / 8 >= 4 && pl.wgs >= 3 * NUM_CU;
  pl.prerot = ((M >= PREROT_MIN_M || redundant) && prerot_bytes(n, M) <= PREROT_REGION) ? 1 : 0;
  return true;
}

// Picks the chunk length (virtual steps per workgroup) with a cost model in microseconds fitted to chunk-length sweeps
// on MI355X (K4, batch 1): a fixed latency chain of ~6 us (launch, x fetch, rotation, store acknowledgement, slot reads,
// output rotation); ~0.8 us per step while every CU holds at most one workgroup, 0.7 us per step and resident
// workgroup beyond that, plus contention when workgroups share a CU; chunks that do not divide a row of column blocks
// (or are not whole rows) cost ~35 % more; every extra contributor to a row block adds slot reads.
inline bool make_plan(int m, int n, int M, int nsplit, Plan& pl) {
  const int nblk = n / 128, rbs = m / 128;
  const long vtotal = (long)rbs * nblk;
  pl.mb = M <= 8 ? 1 : (M <= 16 ? 2 : 4);
  if (nsplit > 0) {                                                 // explicit plan (tuning): chunk length in the low
    const int chunk = nsplit & 0xFFFFF;                             // 20 bits, bit 30 / 29 = force pre-rotation on / off
    bool ok = chunk > 0 ? plan_for_chunk(m, n, M, chunk, pl) : false;
    if (ok && (nsplit & (1 << 30)) && prerot_bytes(n, M) <= PREROT_REGION) pl.prerot = 1;
    if (ok && (nsplit & (1 << 29))) pl.prerot = 0;
    return ok;
  }
  if (vtotal >= (long)64 * NUM_CU && nblk <= 64 && plan_for_chunk(m, n, M, nblk, pl)) return true;
  double best = 1e30;
  bool found = false;
  const int max_chunk = (int)(vtotal < 4096 ? vtotal : 4096);
  for (int chunk = 1; chunk <= max_chunk; ++chunk) {
    Plan c;
    c.mb = pl.mb;
    if (!plan_for_chunk(m, n, M, chunk, c)) continue;
    const double k = (double)c.wgs / NUM_CU;
    const double step = (k <= 1.0 ? 0.8 : 0.7 * k) * (1.0 + 0.25 * (pl.mb - 1));
    const bool aligned = (nblk % chunk == 0) || (chunk % nblk == 0);
    const int pairs_per_wave = c.prerot ? 1 : (M * c.nbl + 7) / 8;
    const int contributors = chunk >= nblk ? 1 : (nblk + chunk - 1) / chunk;
    const double t = 6.0 + (k > 1.0 ? 1.5 : 0.0) + 0.15 * (pairs_per_wave - 1) + step * chunk * (aligned ? 1.0 : 1.35)
                     + 0.1 * contributors + (c.by_counter ? 0.4 * contributors + 1.0 : 0.0);
    if (t < best) { best = t; pl = c; found = true; }
  }
  return found;
}

// The dispatcher places workgroups wherever resources allow, not evenly: with 512 equal workgroups some CUs receive
// three and others one, and the kernel ends with the most loaded CU.  Requesting 1/k of a CU's 160 KB of LDS per
// workgroup (k = workgroups per CU when spread evenly) makes exactly k fit, so the spread is even.
constexpr size_t CU_LDS_BYTES = 160 * 1024;
inline size_t balanced_lds_request(size_t needed, int grid) {
  const int k = (grid + NUM_CU - 1) / NUM_CU;
  if (k > 4) return needed;
  const size_t share = (CU_LDS_BYTES / k) / 1024 * 1024 - 1024;      // room for the kernel's static LDS
  return share > needed ? share : needed;
}

template <int K, int MB, int PRE, bool PREROT> int launch_linear_v(const LinearArgs& a, int grid, size_t lds, hipStream_t st) {
  constexpr int P = K <= 4 ? 4 : (K <= 6 ? 3 : 2);          // wave-steps of weights in flight
  auto kern = k_linear<K, MB, P, (PRE < P ? PRE : P), PREROT>;
  lds = balanced_lds_request(lds, grid);
  if (lds > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) { g_last_hip_error = (int)e; return HTR_ERR_LAUNCH; }
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(WG_THREADS), lds, st, a);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { g_last_hip_error = (int)e; return HTR_ERR_LAUNCH; }
  return HTR_OK;
}
// Steps decoded ahead of the x~ barrier: deep (more registers, fewer resident waves) only for short chunks, where the
// prologue latency is a large part of the kernel; long chunks prefer occupancy.
template <int K, bool PREROT> int launch_linear_kr(const LinearArgs& a, int mb, int grid, size_t lds, hipStream_t st) {
  const bool deep = a.chunk <= 8;
  switch (mb) {
    case 1: return deep ? launch_linear_v<K, 1, 4, PREROT>(a, grid, lds, st) : launch_linear_v<K, 1, 1, PREROT>(a, grid, lds, st);
    case 2: return deep ? launch_linear_v<K, 2, 2, PREROT>(a, grid, lds, st) : launch_linear_v<K, 2, 1, PREROT>(a, grid, lds, st);
    default: return launch_linear_v<K, 4, 1, PREROT>(a, grid, lds, st);
  }
}
template <int K> int launch_linear_k(const LinearArgs& a, int mb, int grid, size_t lds, hipStream_t st) {
  return a.prerot ? launch_linear_kr<K, true>(a, mb, grid, lds, st) : launch_linear_kr<K, false>(a, mb, grid, lds, st);
}

#define HTR_FOR_K(K, EXPR)                 \
  switch (K) {                             \
    case 2: { constexpr int KK = 2; EXPR; } break; \
    case 3: { constexpr int KK = 3; EXPR; } break; \
    case 4: { constexpr int KK = 4; EXPR; } break; \
    case 5: { constexpr int KK = 5; EXPR; } break; \
    case 6: { constexpr int KK = 6; EXPR; } break; \
    case 7: { constexpr int KK = 7; EXPR; } break; \
    case 8: { constexpr int KK = 8; EXPR; } break; \
    default: return HTR_ERR_K;             \
  }

inline bool dtype_ok(int d) { return d == HTR_BF16 || d == HTR_F16 || d == HTR_F32; }

}  // namespace

// ================================================================================================ C ABI
extern "C" {

const char* htr_strerror(int status) {
  switch (status) {
    case HTR_OK: return "ok";
    case HTR_ERR_NULL: return "a required pointer is NULL";
    case HTR_ERR_K: return "unsupported K (HTR-W1 allows 2..8)";
    case HTR_ERR_SHAPE: return "m and n must be positive multiples of 128";
    case HTR_ERR_BATCH: return "M must be in 1..32 for one launch";
    case HTR_ERR_DTYPE: return "dtype must be bf16 (0), f16 (1) or f32 (2)";
    case HTR_ERR_WORKSPACE: return "workspace too small or not 256-byte aligned";
    case HTR_ERR_ALIGN: return "tensor pointer not aligned (qweight 16 B, others natural)";
    case HTR_ERR_LAUNCH: return "HIP launch failed";
    case HTR_ERR_SPLIT: return "explicit split count does not fit this shape";
    case HTR_ERR_COUNT: return "problem count out of range";
    default: return "unknown status";
  }
}

int htr_last_hip_error(void) { return g_last_hip_error; }
int htr_abi_version(void) { return 1; }
float htr_cbscale(void) { return (float)(1.0 / __builtin_sqrt(MEAN_SQ)); }

size_t htr_workspace_bytes(int m, int n, int K, int M, int nsplit) {
  if (K < 2 || K > 8 || m <= 0 || n <= 0 || m % 128 || n % 128 || m / 128 > MAX_ROW_BLOCKS || M < 1 || M > HTR_MAX_BATCH) return 0;
  Plan pl;
  if (!make_plan(m, n, M, nsplit, pl)) return 0;
  return counters_bytes() + PREROT_REGION + (size_t)pl.wgs * pl.segmax * 2 * M * 128 * sizeof(float);
}

int htr_linear_plan(int m, int n, int K, int M, int nsplit, int* out6) {
  if (!out6) return HTR_ERR_NULL;
  if (K < 2 || K > 8) return HTR_ERR_K;
  if (m <= 0 || n <= 0 || m % 128 || n % 128 || m / 128 > MAX_ROW_BLOCKS) return HTR_ERR_SHAPE;
  if (M < 1 || M > HTR_MAX_BATCH) return HTR_ERR_BATCH;
  Plan pl;
  if (!make_plan(m, n, M, nsplit, pl)) return HTR_ERR_SPLIT;
  out6[0] = pl.chunk; out6[1] = pl.wgs; out6[2] = pl.segmax; out6[3] = pl.nbl; out6[4] = pl.by_counter; out6[5] = (int)pl.lds;
  return HTR_OK;
}

int htr_linear(const void* qweight, const void* scales, const void* su, const void* sv, const void* x, const void* bias,
               void* y, int m, int n, int K, int M, int x_dtype, int y_dtype, int nsplit, void* workspace,
               size_t workspace_bytes, void* stream) {
  if (!qweight || !scales || !su || !sv || !x || !y) return HTR_ERR_NULL;
  if (K < 2 || K > 8) return HTR_ERR_K;
  if (m <= 0 || n <= 0 || m % 128 || n % 128 || m / 128 > MAX_ROW_BLOCKS) return HTR_ERR_SHAPE;
  if (M < 1 || M > HTR_MAX_BATCH) return HTR_ERR_BATCH;
  if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return HTR_ERR_DTYPE;
  if (((uintptr_t)qweight & 15) || ((uintptr_t)scales & 1) || ((uintptr_t)x & (x_dtype == HTR_F32 ? 3 : 1)) ||
      ((uintptr_t)y & (y_dtype == HTR_F32 ? 3 : 1)) || (bias && ((uintptr_t)bias & (y_dtype == HTR_F32 ? 3 : 1))))
    return HTR_ERR_ALIGN;
  Plan pl;
  if (!make_plan(m, n, M, nsplit, pl)) return HTR_ERR_SPLIT;
  const size_t need = htr_workspace_bytes(m, n, K, M, nsplit);
  if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return HTR_ERR_WORKSPACE;

  LinearArgs a;
  a.qw = (const uint32_t*)qweight; a.scales = (const uint16_t*)scales; a.su = (const uint8_t*)su; a.sv = (const uint8_t*)sv;
  a.x = x; a.bias = bias; a.y = y;
  a.cnt = (uint32_t*)workspace;
  unsigned char* wsp = (unsigned char*)workspace + counters_bytes();
  a.prerot = pl.prerot; a.xt_g = nullptr; a.xs_g = nullptr; a.sc_g = nullptr;
  if (pl.prerot) {
    a.xt_g = (const _Float16*)wsp;
    a.xs_g = (const float*)(wsp + align256((size_t)M * n * 2));
    a.sc_g = (const float*)(wsp + align256((size_t)M * n * 2) + align256((size_t)M * (n / 128) * 8));
  }
  a.part = (float*)(wsp + PREROT_REGION);
  a.m = m; a.n = n; a.M = M; a.chunk = pl.chunk; a.segmax = pl.segmax; a.by_counter = pl.by_counter;
  a.x_dtype = x_dtype; a.y_dtype = y_dtype;
  a.cbscale = htr_cbscale();
  const int grid = pl.wgs;
  hipStream_t st = (hipStream_t)stream;
  if (pl.prerot) {
    hipLaunchKernelGGL(k_rotate, dim3(M), dim3(WG_THREADS), 0, st, x, (const uint8_t*)su, n, x_dtype, (_Float16*)a.xt_g,
                       (float*)a.xs_g, (float*)a.sc_g);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { g_last_hip_error = (int)e; return HTR_ERR_LAUNCH; }
  }
  HTR_FOR_K(K, return launch_linear_k<KK>(a, pl.mb, grid, pl.lds, st));
  return HTR_OK;
}

int htr_decode_raw(const void* qweight, void* out_i16, int64_t ntiles, int K, void* stream) {
  if (!qweight || !out_i16) return HTR_ERR_NULL;
  if (K < 2 || K > 8) return HTR_ERR_K;
  if (ntiles <= 0) return HTR_ERR_SHAPE;
  if (((uintptr_t)qweight & 15) || ((uintptr_t)out_i16 & 15)) return HTR_ERR_ALIGN;
  const int64_t blocks = (ntiles * 8 + 255) / 256;
  hipStream_t st = (hipStream_t)stream;
  HTR_FOR_K(K, hipLaunchKernelGGL(k_decode_raw<KK>, dim3((unsigned)blocks), dim3(256), 0, st, (const uint32_t*)qweight,
                                  (int16_t*)out_i16, ntiles));
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { g_last_hip_error = (int)e; return HTR_ERR_LAUNCH; }
  return HTR_OK;
}

int htr_dequant_w(const void* qweight, const void* scales, const void* su, const void* sv, void* out_bf16, int m, int n,
                  int K, void* stream) {
  if (!qweight || !scales || !su || !sv || !out_bf16) return HTR_ERR_NULL;
  if (K < 2 || K > 8) return HTR_ERR_K;
  if (m <= 0 || n <= 0 || m % 128 || n % 128 || m / 128 > 65535) return HTR_ERR_SHAPE;
  if (((uintptr_t)qweight & 15) || ((uintptr_t)out_bf16 & 1) || ((uintptr_t)scales & 1)) return HTR_ERR_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(n / 128, m / 128);
  const size_t lds = (size_t)128 * DQW_LD * sizeof(float);
  const float cb = htr_cbscale();
#define HTR_LAUNCH_DQW(KK_)                                                                                              \
  {                                                                                                                      \
    auto kern = k_dequant_w<KK_>;                                                                                        \
    hipError_t e0 = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);       \
    if (e0 != hipSuccess) { g_last_hip_error = (int)e0; return HTR_ERR_LAUNCH; }                                         \
    hipLaunchKernelGGL(kern, grid, dim3(512), lds, st, (const uint32_t*)qweight, (const uint16_t*)scales,                \
                       (const uint8_t*)su, (const uint8_t*)sv, (uint16_t*)out_bf16, n / 16, cb);                         \
  }
  HTR_FOR_K(K, HTR_LAUNCH_DQW(KK));
#undef HTR_LAUNCH_DQW
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { g_last_hip_error = (int)e; return HTR_ERR_LAUNCH; }
  return HTR_OK;
}

int htr_dequant_q(const void* qweight, const void* scales, void* out_f32, int mt, int nt, int K, void* stream) {
  if (!qweight || !scales || !out_f32) return HTR_ERR_NULL;
  if (K < 2 || K > 8) return HTR_ERR_K;
  if (mt <= 0 || nt <= 0) return HTR_ERR_SHAPE;
  if (((uintptr_t)qweight & 15) || ((uintptr_t)out_f32 & 3) || ((uintptr_t)scales & 1)) return HTR_ERR_ALIGN;
  const int64_t blocks = ((int64_t)mt * nt * 8 + 255) / 256;
  hipStream_t st = (hipStream_t)stream;
  const double rms = __builtin_sqrt(MEAN_SQ);
  HTR_FOR_K(K, hipLaunchKernelGGL(k_dequant_q<KK>, dim3((unsigned)blocks), dim3(256), 0, st, (const uint32_t*)qweight,
                                  (const uint16_t*)scales, (float*)out_f32, mt, nt, rms));
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) { g_last_hip_error = (int)e; return HTR_ERR_LAUNCH; }
  return HTR_OK;
}

}  // extern "C"
