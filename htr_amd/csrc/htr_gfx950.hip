// HTR-W1 packed-linear kernels for MI355X (gfx950, CDNA4, wave64) behind a plain C ABI.
//
//   y = sv . Ho( Q . Hi(su . x) ),   Q[i,j] = v(s_ij) * scale_i * CBSCALE,
//   v(s) = bytesum((s * 0xDF6ADF + 0x34983) mod 2^32) - 510              (docs/FORMAT.md:7-13 of the reference)
//
// Work decomposition of the fused linear kernel
//   step      = one 128-row x 128-column block of the weight; the steps of a linear, row-major, are cut into equal
//               contiguous chunks, one workgroup each, so the workgroup count does not depend on the shape
//   workgroup = 8 waves = the 8 strips of a 128-row block (one H128 output block)
//   wave      = one 16-row strip of tiles; per step it streams the 8 consecutive tiles that cover one 128-column
//               input block (8 * 32K contiguous bytes: each lane loads its 4K contiguous bytes) through a buffer
//               descriptor that covers exactly its bytes of the chunk, so loads beyond the end cost nothing
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
//   epilogue  = the workgroup whose chunk holds the last step of a row block finishes it: it adds the partials the
//               earlier chunks of that row block left in their workspace slots (fixed order) to its own, applies
//               scale * CBSCALE, the output H128, sv, bias and the cast.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>
#include <stdlib.h>
#include <atomic>
#include <type_traits>

#include "../../include/htr_gfx950.h"

namespace {

constexpr uint32_t GEN_A = 0xDF6ADFu;
constexpr uint32_t GEN_B = 0x34983u;
constexpr float INV_SQRT128 = 0.08838834764831845f;
constexpr float SQRT128 = 11.313708498984761f;
// 1 / sqrt(mean v^2) over all 65536 states: sum v^2 = 1433042863 (htr/wire.py:28-30 of the reference)
constexpr double MEAN_SQ = 1433042863.0 / 65536.0;

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));
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
// The same through pointers that are known to be global memory (kernel-argument structs lose that, and generic
// accesses compile to flat instructions, which also count against the LDS counter)
#define HTR_GLOBAL __attribute__((address_space(1)))
__device__ __forceinline__ float load_elem_g(const void* p, int dtype, size_t idx) {
  if (dtype == HTR_BF16) return bf16_bits_to_float(((const HTR_GLOBAL uint16_t*)p)[idx]);
  if (dtype == HTR_F16) return f16_bits_to_float(((const HTR_GLOBAL uint16_t*)p)[idx]);
  return ((const HTR_GLOBAL float*)p)[idx];
}
__device__ __forceinline__ void store_elem_g(void* p, int dtype, size_t idx, float v) {
  if (dtype == HTR_BF16) ((HTR_GLOBAL uint16_t*)p)[idx] = float_to_bf16_bits(v);
  else if (dtype == HTR_F16) ((HTR_GLOBAL uint16_t*)p)[idx] = __builtin_bit_cast(uint16_t, (_Float16)v);
  else ((HTR_GLOBAL float*)p)[idx] = v;
}
__device__ __forceinline__ float sign_of_g(const uint8_t* bits, int j) {
  return ((((const HTR_GLOBAL uint8_t*)bits)[j >> 3] >> (j & 7)) & 1) ? -1.f : 1.f;
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
  // own value with the sign of s, added to the partner's: an xor and an add whose DPP operand fetches the partner
  const float own = __uint_as_float(__float_as_uint(a) ^ (__float_as_uint(s) & 0x80000000u));
  a = lane_xor_dpp<H>(a) + own;
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

typedef uint16_t us2 __attribute__((ext_vector_type(2)));
typedef uint32_t u3 __attribute__((ext_vector_type(3)));
template <int CTRL> __device__ __forceinline__ uint32_t dpp_mov_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, false);
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  v = max(v, dpp_mov_u32<0xB1>(v)); v = max(v, dpp_mov_u32<0x4E>(v));
  v = max(v, dpp_mov_u32<0x141>(dpp_mov_u32<0x1B>(v))); v = max(v, dpp_mov_u32<0x128>(v));
  u2s r = __builtin_amdgcn_permlane16_swap(v, v, false, false); v = max(r.x, r.y);
  r = __builtin_amdgcn_permlane32_swap(v, v, false, false); return max(r.x, r.y);
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

// The same K dwords through a buffer descriptor: byte offset `off` from the descriptor's base; out-of-range lanes read
// zeros without touching memory.  Streaming data: non-temporal.
template <int K> __device__ __forceinline__ void load_stream_buffer(__amdgpu_buffer_rsrc_t rsrc, int off, StreamRegs<K>& r) {
  constexpr int NT = 2;
  if constexpr (K == 2) {
    u2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, off, 0, NT); r.d[0] = v.x; r.d[1] = v.y;
  } else if constexpr (K == 3) {
    u3 v = __builtin_amdgcn_raw_buffer_load_b96(rsrc, off, 0, NT); r.d[0] = v.x; r.d[1] = v.y; r.d[2] = v.z;
  } else if constexpr (K == 4) {
    u4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, NT); r.d[0] = v.x; r.d[1] = v.y; r.d[2] = v.z; r.d[3] = v.w;
  } else {
    u4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, NT); r.d[0] = v.x; r.d[1] = v.y; r.d[2] = v.z; r.d[3] = v.w;
    if constexpr (K == 5) {
      r.d[4] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, off + 16, 0, NT);
    } else if constexpr (K == 6) {
      u2 t = __builtin_amdgcn_raw_buffer_load_b64(rsrc, off + 16, 0, NT); r.d[4] = t.x; r.d[5] = t.y;
    } else if constexpr (K == 7) {
      u3 t = __builtin_amdgcn_raw_buffer_load_b96(rsrc, off + 16, 0, NT); r.d[4] = t.x; r.d[5] = t.y; r.d[6] = t.z;
    } else {
      u4 t = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off + 16, 0, NT); r.d[4] = t.x; r.d[5] = t.y; r.d[6] = t.z; r.d[7] = t.w;
    }
  }
}
// ------------------------------------------------------------------------------------------------ decode core
// V[0] = the dword before the lane's first dword (history), V[1..K] = the lane's dwords.  Local step u (0..31) is
// trellis step t = 32q + u; its state is the 16 bits of V that start at bit 16 + (u + 1) * K (bit 0 = MSB of V[0]).
template <int K> struct Window {
  uint32_t V[K + 1];
  uint32_t mid[K];     // mid[w] = bits [32w + 16, 32w + 48) of V, for windows that straddle two dwords
  // the same in two parts: everything that does not involve the history dword, then the rest
  __device__ __forceinline__ void build_tail(const StreamRegs<K>& r) {
#pragma unroll
    for (int k = 0; k < K; ++k) V[k + 1] = r.d[k];
#pragma unroll
    for (int k = 1; k < K; ++k) mid[k] = __builtin_amdgcn_alignbit(V[k], V[k + 1], 16);
  }
  __device__ __forceinline__ void build_head(uint32_t prev) {
    V[0] = prev;
    mid[0] = __builtin_amdgcn_alignbit(V[0], V[1], 16);
  }
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

// ------------------------------------------------------------------------------------------------ batched linear
// Variant for 9 .. 128 activation rows.  With that many rows the rotated activations of a whole chunk no longer fit in
// LDS next to useful chunk lengths, and short chunks mean that every workgroup copies a large activation slice and
// hands over a large partial for little weight traffic.  Here a workgroup owns one 128-row block and 1/S of its
// column blocks (grid = S x row blocks), and the activations (rotated ahead by a launch of their own) are staged through
// LDS one 128-column block at a time, double-buffered, one barrier per step; with few rows over few column blocks the
// workgroup rotates its own slice instead and keeps it in LDS (ROT, below).  The split S along the columns is only as large
// as filling the chip needs; S = 1 needs no exchange.
//   wave    = two adjacent 16-row strips (pair sp = w / 2) x one half (ch = w % 2) of the block's columns: 2 x 4 tiles
//             per step, two runs of 128 K contiguous bytes
//   lane    = (tile column g = lane / 16, strip h = lane / 8 % 2, row pair q = lane % 8); a tile is still 8 consecutive
//             lanes, so the decode is the one of k_linear
//   product = MFMA row i = lane % 16 = (h, q): rows 2q (or 2q + 1) of both strips, all of them over the same 32 columns
//             (k-slot g = columns 0..7, or 8..15, of tile column 4 ch + g).  So every one of the 16 MFMA columns carries
//             an activation row: 16 rows per matrix instruction, and a wave reads only its half of the block from LDS.
//             D[i][c] sits in lane c + 16 * (i / 4), register i % 4: lane (g', c) ends up with rows 32 sp + 8 g' .. + 7
//             of the row block for activation row c.
//   The two waves of a strip pair leave their column halves side by side in LDS when the split is done; whoever reads
//   the workgroup's partial adds the two.
constexpr int BATCH_ROWH = 128 + 8;          // halves per staged activation row: 16 rows x 16 bytes then cover every bank once
constexpr int BATCH_FIN_STRIDE = 128 + 4;    // floats per activation row of the workgroup's partial
// position of output row r (0..127) in a row of the partial: [r % 8][r / 8], so that the lanes of a wave (16 activation
// rows x 4 groups of 8 output rows) hit 64 different banks with each of their 8 values
__device__ __forceinline__ int batch_fin_pos(int r) { return (r & 7) * 16 + (r >> 3); }

template <int K, int MG, int P, bool ROT>
__global__ __launch_bounds__(WG_THREADS, MG <= 2 && !ROT ? 4 : 2) void k_linear_batch(const uint32_t* __restrict__ qw, float* __restrict__ part,
                                                             const void* __restrict__ x, const uint8_t* __restrict__ su,
                                                             int m, int n, int M, int S, int flags, const LinearTail t) {
  static_assert(!ROT || MG <= 2, "the variant that rotates its own activations holds up to 32 rows");
  extern __shared__ __align__(16) unsigned char lds[];
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int sp = w >> 1, ch = w & 1;
  const int nblk = n >> 7;
  const int s_idx = blockIdx.x, rb = blockIdx.y;
  const int cb = (nblk + S - 1) / S;                               // column blocks per split
  const int c_begin = s_idx * cb, c_end = min(nblk, c_begin + cb);
  const int nsteps = c_end - c_begin;                              // >= 1: the host picks S so that no split is empty
  const int y_dtype = (flags >> 2) & 3;

  // LDS: [2 buffers][16 MG rows][136 halves] x~ blocks, [2][16 MG][2] sums, [16 MG] activation scales,
  // [2 column halves][M][132] partial of the workgroup.  Rows M .. 16 MG - 1 are staged like the others (they read out of
  // range: zeros), so every group of 16 rows is addressed alike.  With more than 64 rows the partial does not fit
  // behind the blocks and takes their place once the last step is done.
  // ROT (up to 16 rows over up to 16 column blocks per split, or up to 32 rows over up to 8): no rotation launch; the
  // workgroup rotates the activations of its own column blocks at the start (wave w: rows 2 MG w .. 2 MG w + 2 MG - 1,
  // four blocks per pass on the matrix unit, eight passes, one power-of-two scale per row from max|x| over the split's
  // columns) and keeps all of them in LDS, [cb blocks][16 MG rows][136 halves] + [cb][16 MG][2] sums: no staging and no
  // barrier inside the loop.
  constexpr int ROWH = BATCH_ROWH, ROWS = 16 * MG, BUFH = ROWS * ROWH;
  constexpr bool FIN_OVER_BLOCKS = MG > 4;
  _Float16* xt = (_Float16*)lds;
  float* s_xs = (float*)(lds + (size_t)(ROT ? cb : 2) * BUFH * 2);
  float* s_sc = s_xs + (ROT ? cb * 2 * ROWS : 4 * ROWS);
  float* s_fin = FIN_OVER_BLOCKS ? (float*)lds : s_sc + ROWS;

  // ---- activation staging in 16-byte pieces (8 halves): piece pi of the block is row pi / 16, columns 8 (pi % 16) .. + 7;
  // a thread takes pieces tid, tid + 512, ...
  constexpr int NPT = MG >= 2 ? MG / 2 : 1;      // pieces per thread
  const int tid = threadIdx.x;
  const bool has_piece = MG >= 2 || tid < ROWS * 16, has_sum = tid < 2 * ROWS;
  const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)t.xt_g, 0, M * n * 2, 0x00020000);
  const __amdgpu_buffer_rsrc_t srsrc = __builtin_amdgcn_make_buffer_rsrc((void*)t.xs_g, 0, M * nblk * 16, 0x00020000);
  constexpr int OUT_OF_RANGE = 0x7FFFFF00;
  int piece_lds[NPT], piece_src[NPT];            // halves inside a buffer; byte offset in x~ of the piece in block 0
#pragma unroll
  for (int i = 0; i < NPT; ++i) {
    const int pi = tid + i * WG_THREADS, p_row = pi >> 4, p_idx = pi & 15;
    piece_lds[i] = p_row * ROWH + (p_idx & 1) * 64 + (p_idx >> 1) * 8;
    piece_src[i] = p_row < M ? (p_row * n + p_idx * 8) * 2 : -1;
  }
  const int sum_src = (tid >> 1) < M ? (((tid >> 1) * nblk) * 4 + 2 + (tid & 1)) * 4 : -1;   // sums over columns 0..63 | 64..127
  // Blocks travel ahead of their use in registers: two steps (two register sets, by block parity) up to 32 rows, because
  // loads return in order, so that waiting for a block also waits for every weight load issued before it, and one step
  // of distance would cut the weight stream's run-ahead to a single step; with more rows a step is long enough for one.
  constexpr int DIST = MG <= 2 ? 2 : 1;
  u4 xg[DIST][NPT];
  float xsg[DIST];
  auto stage_load = [&](int blk, int q) {    // block index in the row; beyond the split: zeros, no traffic
    HTR_PIN();
    const bool live = blk < c_end;
    const int set = DIST == 2 ? q : 0;
#pragma unroll
    for (int i = 0; i < NPT; ++i)
      xg[set][i] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, live && piece_src[i] >= 0 ? piece_src[i] + blk * 256 : OUT_OF_RANGE, 0, 0);
    xsg[set] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(srsrc, live && sum_src >= 0 ? sum_src + blk * 16 : OUT_OF_RANGE, 0, 0));
    HTR_PIN();
  };
  auto stage_store = [&](int q) {            // the block of parity q goes to buffer q
    const int set = DIST == 2 ? q : 0;
#pragma unroll
    for (int i = 0; i < NPT; ++i)
      if (has_piece) *(u4*)(xt + q * BUFH + piece_lds[i]) = xg[set][i];
    if (has_sum) s_xs[q * 2 * ROWS + tid] = xsg[set];
  };
  // ROT: the raw activations of this wave's rows, eight passes of four blocks, all loads back to back
  constexpr int RPASS = ROT ? 8 : 1;
  constexpr int ROTR = 2 * MG, PPR = 8 / ROTR;          // rows a wave rotates, passes (of four blocks) per row
  u4 rx[RPASS];
  uint32_t rsb[RPASS];
  if constexpr (ROT) {
    const __amdgpu_buffer_rsrc_t rawsrc = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, M * n * 2, 0x00020000);
    const __amdgpu_buffer_rsrc_t sgnsrc = __builtin_amdgcn_make_buffer_rsrc((void*)su, 0, n >> 3, 0x00020000);
    int xo[RPASS], so[RPASS];
#pragma unroll
    for (int r = 0; r < RPASS; ++r) {
      const int row = ROTR * w + r / PPR, bl = 4 * (r % PPR) + ((lane & 15) >> 2);      // block within the split
      const int col = (c_begin + bl) * 128 + 32 * (lane & 3) + 8 * (lane >> 4);
      const bool live = row < M && bl < nsteps;
      xo[r] = live ? (row * n + col) * 2 : OUT_OF_RANGE;
      so[r] = live ? col >> 3 : OUT_OF_RANGE;
    }
    HTR_PIN();
#pragma unroll
    for (int r = 0; r < RPASS; ++r) {
      rx[r] = __builtin_amdgcn_raw_buffer_load_b128(rawsrc, xo[r], 0, 0);
      rsb[r] = (uint32_t)(uint8_t)__builtin_amdgcn_raw_buffer_load_b8(sgnsrc, so[r], 0, 0);
    }
    HTR_PIN();
  } else {
    if (tid < ROWS) s_sc[tid] = tid < M ? t.sc_g[tid] : 0.f;
    stage_load(c_begin, 0);
    if constexpr (DIST == 2) stage_load(c_begin + 1, 1);
  }

  // row constants of the output side (scale, sign, bias of rows lane and lane + 64), requested ahead of the weight stream by
  // the workgroups that finish rows of the row block, so that they have long arrived when they are needed
  const int RG = (M + 7) >> 3;               // groups of eight activation rows
  // the splits share the output side (below), unless the host found that the grid does not fit the chip at once: splits
  // that wait for each other must all be resident, a last split that waits for the earlier ones need not be
  const bool spread = (M > 16 || (M > 8 && S > 2)) && !(flags & FLAG_LAST_FINISHES);
  const bool finisher = spread ? s_idx < RG : s_idx == S - 1;
  const int r0 = rb * 128 + lane, r1 = r0 + 64;
  uint32_t raw_sc0 = 0u, raw_sc1 = 0u, raw_sv0 = 0u, raw_sv1 = 0u, raw_b0 = 0u, raw_b1 = 0u;   // bits only: converted at the end
  if (finisher) {
    raw_sc0 = ((const HTR_GLOBAL uint16_t*)t.scales)[r0];
    raw_sc1 = ((const HTR_GLOBAL uint16_t*)t.scales)[r1];
    raw_sv0 = ((const HTR_GLOBAL uint8_t*)t.sv)[r0 >> 3];
    raw_sv1 = ((const HTR_GLOBAL uint8_t*)t.sv)[r1 >> 3];
    if (t.bias != nullptr) {
      if (y_dtype == HTR_F32) { raw_b0 = ((const HTR_GLOBAL uint32_t*)t.bias)[r0]; raw_b1 = ((const HTR_GLOBAL uint32_t*)t.bias)[r1]; }
      else { raw_b0 = ((const HTR_GLOBAL uint16_t*)t.bias)[r0]; raw_b1 = ((const HTR_GLOBAL uint16_t*)t.bias)[r1]; }
    }
  }

  // ---- the weight stream of this wave: per step, tiles 4 ch .. 4 ch + 3 of strips 2 sp and 2 sp + 1.  One descriptor
  // from the first strip's first byte of the split to the second strip's last: lanes of the second strip that run past
  // the split are out of range (zeros, no traffic); lanes of the first strip would land in later column blocks, so a
  // request beyond the last step is sent out of range as a whole.
  constexpr int STEP_BYTES = 256 * K;
  const uint32_t strip_bytes = (uint32_t)nblk * STEP_BYTES;
  const uint32_t* wave_base = qw + ((size_t)(rb * 8 + 2 * sp) * nblk + (size_t)c_begin) * (STEP_BYTES / 4);
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)wave_base, 0, (int)(strip_bytes + (uint32_t)nsteps * STEP_BYTES), 0x00020000);
  const int g = lane >> 4, n16 = lane & 15;
  int pf_off = ((lane >> 3) & 1) * (int)strip_bytes + ((4 * ch + g) * 8 + (lane & 7)) * 4 * K;
  int pf_left = nsteps;                      // steps not yet requested (uniform)
  StreamRegs<K> buf[P];
  auto prefetch = [&](StreamRegs<K>& dst) {
    HTR_PIN();
    load_stream_buffer<K>(rsrc, pf_left > 0 ? pf_off : OUT_OF_RANGE, dst);
    pf_off += STEP_BYTES;
    --pf_left;
    HTR_PIN();
  };
#pragma unroll
  for (int p = 0; p < P; ++p) prefetch(buf[p]);

  // ---- the product.  This lane's B operands and sums belong to activation rows 16 mg + lane % 16: group mg sits
  // 16 mg rows behind group 0 in LDS, a constant offset
  const _Float16* b_lane = xt + n16 * ROWH + 8 * (4 * ch + g);
  const float* xs_lane = s_xs + 2 * n16 + ch;
  float offs[MG];      // running 1534 * sum(x~) over the wave's half of the blocks
  f4 acc[MG][2];
#pragma unroll
  for (int mg = 0; mg < MG; ++mg) { offs[mg] = 0.f; acc[mg][0] = f4{0.f, 0.f, 0.f, 0.f}; acc[mg][1] = f4{0.f, 0.f, 0.f, 0.f}; }

  // B operands and sums: up to 32 rows they are read one step ahead, right behind the barrier, and their latency hides
  // behind the second half of the decode; with more rows they would hold too many registers, and each pair of 16-row
  // groups is read while the matrix instructions of the pair before it run
  constexpr bool AHEAD = MG <= 2;
  constexpr int NB = AHEAD ? MG : 4;               // B register sets
  h8 B0[NB], B1[NB];
  float xsv[NB];
  auto fetch_b = [&](int bsel, int mg, int set) {       // bsel: staging buffer (0 / 1), or with ROT the block within the split
    const _Float16* bp = b_lane + bsel * BUFH + mg * 16 * ROWH;
    B0[set] = *(const h8*)bp;
    B1[set] = *(const h8*)(bp + 64);
    xsv[set] = xs_lane[bsel * 2 * ROWS + mg * 32];
  };
  auto load_b = [&](int bsel) {
    if constexpr (AHEAD) {
#pragma unroll
      for (int mg = 0; mg < MG; ++mg) fetch_b(bsel, mg, mg);
    }
  };
  auto multiply = [&](const DecodedStep<K>& d, int bsel) {
    if constexpr (AHEAD) {
#pragma unroll
      for (int mg = 0; mg < MG; ++mg) acc[mg][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[0], B0[mg], acc[mg][0], 0, 0, 0);
#pragma unroll
      for (int mg = 0; mg < MG; ++mg) acc[mg][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[2], B0[mg], acc[mg][1], 0, 0, 0);
#pragma unroll
      for (int mg = 0; mg < MG; ++mg) acc[mg][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[1], B1[mg], acc[mg][0], 0, 0, 0);
#pragma unroll
      for (int mg = 0; mg < MG; ++mg) acc[mg][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[3], B1[mg], acc[mg][1], 0, 0, 0);
#pragma unroll
      for (int mg = 0; mg < MG; ++mg) offs[mg] = __builtin_fmaf(1534.f, xsv[mg], offs[mg]);
    } else {
      fetch_b(bsel, 0, 0); fetch_b(bsel, 1, 1);
#pragma unroll
      for (int pr = 0; pr < MG / 2; ++pr) {
        const int cs = (pr & 1) * 2;
        if (pr + 1 < MG / 2) { fetch_b(bsel, 2 * pr + 2, cs ^ 2); fetch_b(bsel, 2 * pr + 3, (cs ^ 2) + 1); }
#pragma unroll
        for (int u = 0; u < 2; ++u) acc[2 * pr + u][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[0], B0[cs + u], acc[2 * pr + u][0], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < 2; ++u) acc[2 * pr + u][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[2], B0[cs + u], acc[2 * pr + u][1], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < 2; ++u) acc[2 * pr + u][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[1], B1[cs + u], acc[2 * pr + u][0], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < 2; ++u) acc[2 * pr + u][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.a[3], B1[cs + u], acc[2 * pr + u][1], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < 2; ++u) offs[2 * pr + u] = __builtin_fmaf(1534.f, xsv[cs + u], offs[2 * pr + u]);
      }
    }
  };

  static_assert(P % 2 == 0, "the block parity of a step must be static in the unrolled loop");
  const int hist = history_lane_byteaddr(lane);
  DecodedStep<K> cur;
  if constexpr (ROT) {
    // ---- rotation of this wave's rows.  Row scale from the raw values: |H128 x| / sqrt(128) <= sqrt(128) max|x|.
    const bool is_bf16 = (flags & 3) == HTR_BF16;
    const int j = lane & 15, gk = lane >> 4;
#pragma unroll
    for (int rr = 0; rr < ROTR; ++rr) {
      uint32_t m16 = 0u;
#pragma unroll
      for (int q = 0; q < PPR; ++q) {
        const uint32_t d[4] = {rx[PPR * rr + q].x, rx[PPR * rr + q].y, rx[PPR * rr + q].z, rx[PPR * rr + q].w};
#pragma unroll
        for (int k = 0; k < 4; ++k) m16 = max(m16, max(d[k] & 0x7FFFu, (d[k] >> 16) & 0x7FFFu));
      }
      m16 = wave_max_u32(m16);
      float amax = is_bf16 ? bf16_bits_to_float((uint16_t)m16) : f16_bits_to_float((uint16_t)m16);
      if (amax != amax) amax = __uint_as_float(0x7F800000u);      // a NaN anywhere: treat the row as unbounded (scale 1)
      const int e = scale_exponent(amax);
      const float f = pow2f(-e) * INV_SQRT128;
      const int row = ROTR * w + rr;
      if (lane == 0) s_sc[row] = row < M ? pow2f(e) : 0.f;
#pragma unroll
      for (int q = 0; q < PPR; ++q) {
        if (4 * q >= nsteps) continue;                             // uniform: none of the pass's blocks exists
        float y[2][4];
        rotate4_mfma(rx[PPR * rr + q], rsb[PPR * rr + q], is_bf16, lane, y);
        const int bl = 4 * q + gk;                                 // lane (p = lane / 16, j) holds elements 32 a' + 16 h + j of block 4 q + p
        const bool live_o = bl < nsteps;
        _Float16* dst = xt + (size_t)(bl * ROWS + row) * ROWH + (j >> 3) * 64 + (j & 7);
        float lo = 0.f, hi = 0.f;                                  // sums of the rounded values: columns 0..63 | 64..127
        const h2 ones = {(_Float16)1.f, (_Float16)1.f};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const h2 p01 = __builtin_convertvector(f2{y[h][0] * f, y[h][1] * f}, h2);
          const h2 p23 = __builtin_convertvector(f2{y[h][2] * f, y[h][3] * f}, h2);
          if (live_o) { dst[(0 + h) * 8] = p01.x; dst[(2 + h) * 8] = p01.y; dst[(4 + h) * 8] = p23.x; dst[(6 + h) * 8] = p23.y; }
          lo = __builtin_amdgcn_fdot2(p01, ones, lo, false);
          hi = __builtin_amdgcn_fdot2(p23, ones, hi, false);
        }
        lo += dpp_mov<0xB1>(lo); lo += dpp_mov<0x4E>(lo); lo += dpp_mov<0x141>(lo); lo += dpp_mov<0x140>(lo);
        hi += dpp_mov<0xB1>(hi); hi += dpp_mov<0x4E>(hi); hi += dpp_mov<0x141>(hi); hi += dpp_mov<0x140>(hi);
        if (live_o && j == 0) { s_xs[(bl * ROWS + row) * 2] = lo; s_xs[(bl * ROWS + row) * 2 + 1] = hi; }
      }
    }
    decode_step<K>(buf[0], hist, cur);
    prefetch(buf[0]);
    __syncthreads();
    load_b(0);
    // the loop: multiply step v, read the operands of step v + 1, decode it; no barrier, every block is in LDS
    // (no barrier keeps the two waves of a SIMD in step here, and the arbiter favours the older one: as in k_linear's
    // PACE variant the younger waves take the higher priority every other group of P steps, so that both reach the end
    // of the loop together; 16 rows on 14336x4096: 15.6 -> 14.9 us.  In the staged loop below the barrier of every step
    // does that, and finer alternation inside a step only cost time.)
    int v = 0;
    for (; v + P < nsteps; v += P) {
      if (w >= 4) { if ((v / P) & 1) __builtin_amdgcn_s_setprio(0); else __builtin_amdgcn_s_setprio(1); }
#pragma unroll
      for (int pp = 0; pp < P; ++pp) {
        multiply(cur, 0);
        load_b(v + pp + 1);
        decode_step<K>(buf[(pp + 1) % P], hist, cur);
        prefetch(buf[(pp + 1) % P]);
      }
    }
    __builtin_amdgcn_s_setprio(0);
#pragma unroll
    for (int pp = 0; pp < P; ++pp) {
      if (v + pp < nsteps) {
        multiply(cur, 0);
        if (v + pp + 1 < nsteps) {
          load_b(v + pp + 1);
          decode_step<K>(buf[(pp + 1) % P], hist, cur);
          prefetch(buf[(pp + 1) % P]);
        }
      }
    }
  } else {
  // step 0: its block goes to buffer 0, the next block to come is requested, the first weights are decoded meanwhile
  stage_store(0);
  stage_load(c_begin + DIST, 0);
  decode_step<K>(buf[0], hist, cur);
  prefetch(buf[0]);
  __syncthreads();
  load_b(0);

  // One step with a successor: multiply step v, put the block of step v + 1 (in registers) into the other buffer,
  // request the next block to come, decode step v + 1; between the two halves of the decode the workgroup meets, after
  // which the B operands of step v + 1 may be read.
  auto step_with_next = [&](int v, int q, StreamRegs<K>& nxt) {      // q = (v + 1) & 1, static
    multiply(cur, q ^ 1);
    stage_store(q);
    stage_load(c_begin + v + 1 + DIST, q);
    decode_step_mid<K>(nxt, hist, cur, [&]() { __syncthreads(); load_b(q); });
    prefetch(nxt);
  };
  int v = 0;
  for (; v + P < nsteps; v += P) {
#pragma unroll
    for (int pp = 0; pp < P; ++pp) step_with_next(v + pp, (pp + 1) & 1, buf[(pp + 1) % P]);
  }
#pragma unroll
  for (int pp = 0; pp < P; ++pp) {
    if (v + pp + 1 < nsteps) step_with_next(v + pp, (pp + 1) & 1, buf[(pp + 1) % P]);
    else if (v + pp < nsteps) multiply(cur, pp & 1);
  }
  }   // staged path

  // ---- this wave's partial (offset removed, activation scale undone) goes to its column half's copy in LDS
  float scl[MG];
#pragma unroll
  for (int mg = 0; mg < MG; ++mg) scl[mg] = s_sc[mg * 16 + n16];
  if constexpr (FIN_OVER_BLOCKS) __syncthreads();          // every wave has read its last B operands
#pragma unroll
  for (int mg = 0; mg < MG; ++mg) {
    const int mrow = mg * 16 + n16;
    if (mrow < M) {
      float* dst = s_fin + (ch * M + mrow) * BATCH_FIN_STRIDE + 4 * sp + g;       // row 32 sp + 8 g + i sits at i * 16 + 4 sp + g
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int rr = 0; rr < 2; ++rr)
          dst[(2 * j + rr) * 16] = (acc[mg][rr][j] - offs[mg]) * scl[mg];
    }
  }
  __syncthreads();
  const int pos0 = batch_fin_pos(lane), pos1 = batch_fin_pos(lane + 64);
  // ---- exchange between the splits of the row block.  The activation rows are dealt to the splits in groups of eight
  // (group rg = rows 8 rg .. 8 rg + 7, one row per wave): split rg mod S finishes group rg, every other split leaves
  // its partial of those rows in its slot.  So the output side of many rows is spread over the splits instead of
  // falling to one workgroup (32 rows on 4096x14336, 8 splits: 23.0 -> 19.7 us; 128 rows: 56.6 -> 38.5).  The
  // workgroups of one row block are neighbours in dispatch order and the grid fits the chip (the host checks it against
  // the device's CU count and otherwise sets FLAG_LAST_FINISHES), so they run together; the wait is bounded all the same.  Up to 8 rows (one group), and up to 16 rows with two splits, the last split
  // finishes everything, as in k_linear: two workgroups that wait for each other cost 0.3 us more than one that waits.
  for (int rg = 0, owner = spread ? 0 : S - 1; rg < RG; ++rg, owner = !spread ? owner : (owner + 1 == S ? 0 : owner + 1)) {
    const int mrow = 8 * rg + w;
    if (owner != s_idx && mrow < M) {
      const float* own = s_fin + mrow * BATCH_FIN_STRIDE;
      const float* oth = own + M * BATCH_FIN_STRIDE;
      uint32_t* dst = (uint32_t*)(part + (((size_t)rb * S + s_idx) * M + mrow) * 128);
      __hip_atomic_store(dst + lane, __float_as_uint(own[pos0] + oth[pos0]) | 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(dst + lane + 64, __float_as_uint(own[pos1] + oth[pos1]) | 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (!finisher) return;
  const uint32_t stale = load_status(t.status);     // non-zero: an earlier launch on this workspace gave up

  // ---- output side of this split's row groups: add the other splits' partials (fixed order), finish
  const float rs0 = f16_bits_to_float((uint16_t)raw_sc0) * t.cbscale * INV_SQRT128;
  const float rs1 = f16_bits_to_float((uint16_t)raw_sc1) * t.cbscale * INV_SQRT128;
  const float sg0 = ((raw_sv0 >> (lane & 7)) & 1u) ? -1.f : 1.f, sg1 = ((raw_sv1 >> (lane & 7)) & 1u) ? -1.f : 1.f;
  auto cvt_bias = [&](uint32_t b) {
    return y_dtype == HTR_F32 ? __uint_as_float(b) : y_dtype == HTR_BF16 ? bf16_bits_to_float((uint16_t)b) : f16_bits_to_float((uint16_t)b);
  };
  const float b0v = cvt_bias(raw_b0), b1v = cvt_bias(raw_b1);
  // slot of the k-th other split (k = 0 .. S - 2, own split skipped) for activation row mrow
  auto slot_of = [&](int k, int mrow) { return (uint32_t*)(part + (((size_t)rb * S + (k + (k >= s_idx ? 1 : 0))) * M + mrow) * 128); };
  // waits (bounded) until every other split's partial of activation row mrow is there; their sum in fixed order
  auto wait_for_row = [&](int mrow, float& v0s, float& v1s) {
    int tries = 0;
    for (;;) {
      bool missing = false;
      v0s = 0.f; v1s = 0.f;
      for (int jb = 0; jb < S - 1; jb += 8) {
        uint32_t u0[8], u1[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const uint32_t* pp = slot_of(min(jb + k, S - 2), mrow);
          u0[k] = __hip_atomic_load(pp + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          u1[k] = __hip_atomic_load(pp + lane + 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k)
          if (jb + k < S - 1) {
            missing |= (u0[k] == 0u) | (u1[k] == 0u);
            v0s += __uint_as_float(u0[k]); v1s += __uint_as_float(u1[k]);
          }
      }
      if (!__any(missing)) return false;
      if (++tries >= t.spin_limit) return true;
      __builtin_amdgcn_s_sleep(2);
    }
  };
  // the rest of a row: slots back to zero for the next call (or the failure noted), own partial, output side
  auto finish_row = [&](int mrow, float v0s, float v1s, bool failed) {
    if (S > 1) {
      if (!failed) {
        for (int k = 0; k < S - 1; ++k) {
          uint32_t* pp = slot_of(k, mrow);
          __hip_atomic_store(pp + lane, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          __hip_atomic_store(pp + lane + 64, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      } else if (lane == 0) {
        report_give_up(t.status);
      }
    }
    failed |= stale != 0u;
    const float* own = s_fin + mrow * BATCH_FIN_STRIDE;
    const float* oth = own + M * BATCH_FIN_STRIDE;
    v0s += own[pos0] + oth[pos0]; v1s += own[pos1] + oth[pos1];
    v0s *= rs0; v1s *= rs1;
    fwht128_wave(v0s, v1s, lane);
    v0s = __builtin_fmaf(v0s, sg0, b0v);
    v1s = __builtin_fmaf(v1s, sg1, b1v);
    if (failed) { v0s = __builtin_nanf(""); v1s = v0s; }
    store_elem_g(t.y, y_dtype, (size_t)mrow * m + r0, v0s);
    store_elem_g(t.y, y_dtype, (size_t)mrow * m + r1, v1s);
  };
  // Wave w finishes row w of this split's groups s_idx, s_idx + S, ...: its i-th row is 8 (s_idx + i S) + w (all groups
  // if the last split finishes everything).
  constexpr int RPW = MG * 2;                    // rows per wave at most (a single split finishes all groups)
  auto my_row = [&](int i) { return spread ? 8 * (s_idx + i * S) + w : 8 * i + w; };
  // With up to eight other splits the slots of several of the wave's rows are requested together (at most 2 x 32
  // registers of them), so that the rows behind the first cost no memory round trip of their own.  JW = slots
  // requested per row (the next power of two from S - 1; the surplus repeats the last slot).
  auto finish_rows_together = [&](auto jw) {
    constexpr int JW = decltype(jw)::value;
    constexpr int RB = RPW * JW <= 32 ? RPW : 32 / JW;      // rows per request
#pragma unroll
    for (int rbase = 0; rbase < RPW; rbase += RB) {
      if (my_row(rbase) >= M) break;
      float a0[RB], a1[RB];
      int tries = 0;
      bool failed = false;
      for (;;) {
        uint32_t u0[RB][JW], u1[RB][JW];
#pragma unroll
        for (int r = 0; r < RB; ++r) {
          // a row beyond M repeats the request of the batch's first row and is not looked at
          const int mrow = my_row(rbase + r) < M ? my_row(rbase + r) : my_row(rbase);
#pragma unroll
          for (int k = 0; k < JW; ++k) {
            const uint32_t* pp = slot_of(min(k, S - 2), mrow);
            u0[r][k] = __hip_atomic_load(pp + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            u1[r][k] = __hip_atomic_load(pp + lane + 64, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
        bool missing = false;
#pragma unroll
        for (int r = 0; r < RB; ++r) {
          a0[r] = 0.f; a1[r] = 0.f;
          const bool real = my_row(rbase + r) < M;
#pragma unroll
          for (int k = 0; k < JW; ++k)
            if (real && k < S - 1) {
              missing |= (u0[r][k] == 0u) | (u1[r][k] == 0u);
              a0[r] += __uint_as_float(u0[r][k]); a1[r] += __uint_as_float(u1[r][k]);
            }
        }
        if (!__any(missing)) break;
        if (++tries >= t.spin_limit) { failed = true; break; }
        __builtin_amdgcn_s_sleep(2);
      }
#pragma unroll
      for (int r = 0; r < RB; ++r)
        if (my_row(rbase + r) < M) finish_row(my_row(rbase + r), a0[r], a1[r], failed);
    }
  };
  if (my_row(0) >= M) return;
  if (S > 1 && S - 1 <= 8 && my_row(1) < M) {
    if (S - 1 <= 1) finish_rows_together(std::integral_constant<int, 1>{});
    else if (S - 1 <= 2) finish_rows_together(std::integral_constant<int, 2>{});
    else if (S - 1 <= 4) finish_rows_together(std::integral_constant<int, 4>{});
    else finish_rows_together(std::integral_constant<int, 8>{});
    return;
  }
  for (int i = 0; my_row(i) < M; ++i) {
    float v0s = 0.f, v1s = 0.f;
    const bool failed = S > 1 ? wait_for_row(my_row(i), v0s, v1s) : false;
    finish_row(my_row(i), v0s, v1s, failed);
  }
}

// ------------------------------------------------------------------------------------------------ fused GEMM
// More than 128 activation rows: the product is bound by the matrix unit and by what feeds it, not by the decode.  A
// workgroup owns one 128-row block of the weight, one tile of 128 activation rows and 1/S of the column blocks (grid =
// S x row blocks x row tiles).  Per 128-column block, wave w = (row half rh = w % 2, column quarter cq = w / 2) decodes 64
// rows x 32 columns: its lanes take the (tile, row pair) granules of strips 4 rh .. 4 rh + 3 in tile columns 2 cq (lanes
// 0..31) and 2 cq + 1 (lanes 32..63).  A granule is rows 2q, 2q + 1 x the tile's 16 columns; the 32x32x16 matrix
// instruction wants lane (row i = lane % 32, k-group lane / 32) to bring 8 consecutive columns of ONE row, the two
// k-groups of a row in lanes l and l + 32.  One v_permlane32_swap per register moves "columns 8..15 of the lower lanes'
// granule" up and "columns 0..7 of the upper lanes' granule" down, after which the decode registers ARE the A operands:
// (even rows | odd rows) x (tile column 2 cq | 2 cq + 1), 32 weight rows each.  The weights never pass through LDS.
// The B operands are the block's rotated activations (rotated ahead by a launch of their own), staged through LDS in
// three buffers; each B read (32 activation rows x 16 columns) serves two matrix instructions (even and odd rows), 0.5 KB
// of LDS traffic per instruction: half of what a design with both operands in LDS needs, which is what the LDS can
// sustain next to the staging.  The decode of the next block is interleaved with the matrix instructions of this one.
// Output side: every wave has the partial of its 64 rows over its 32 columns; the four column quarters meet in LDS, the
// offset (1534 x the activation row's sum over the split's columns) is removed by the first quarter, the activation scale
// is undone; with S > 1 the last split of a row block collects the others' tiles and finishes: row scale, output H128,
// sign, bias, cast.
constexpr int GEMM_THREADS = WG_THREADS;
// activation rows per tile = 32 JB, JB = 3 or 4: with 96 rows the weight is decoded once more per 96 rows but a step is
// shorter and the activations travel two steps ahead in two register sets; 128 rows need the registers (one set, one
// step ahead, two stream buffers) and pay where they save a round of workgroups.  The planner chooses.
constexpr int GEMM_LD = 128 + 8;                               // halves per row of a staged activation block: 16-byte rows, 4 banks of shift
constexpr int GEMM_XBUFS = 3;
constexpr int GEMM_FIN_LD = 128 + 4;                           // floats per activation row of the output in LDS
constexpr size_t gemm_lds_bytes(int jb) {
  const size_t rows = (size_t)32 * jb;
  const size_t fin = 2 * rows * GEMM_FIN_LD * 4;               // two copies of the output (column quarters 0, 2 | 1, 3)
  const size_t xb = GEMM_XBUFS * rows * GEMM_LD * 2 + GEMM_XBUFS * rows * 4;
  return (fin > xb ? fin : xb) + 16;
}
typedef float f16v __attribute__((ext_vector_type(16)));

template <int K, int P, int JB>
__global__ __launch_bounds__(GEMM_THREADS) void k_linear_gemm(const uint32_t* __restrict__ qw, float* __restrict__ part,
                                                                 int m, int n, int M, int S, int flags, const LinearTail t) {
  extern __shared__ __align__(16) unsigned char lds[];
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int rh = w & 1, cq = w >> 1;
  const int nblk = n >> 7;
  const int s_idx = blockIdx.x, rb = blockIdx.y, mt = blockIdx.z;
  constexpr int GEMM_ROWS = 32 * JB, GEMM_TILE_HALVES = GEMM_ROWS * GEMM_LD;
  constexpr size_t GEMM_LDS_BYTES = gemm_lds_bytes(JB);
  constexpr int XSETS = JB <= 3 ? 2 : 1;                         // register sets of activations in flight = steps ahead
  const int j0 = mt * GEMM_ROWS, rows = min(GEMM_ROWS, M - j0);  // this tile's activation rows
  const int cb = (nblk + S - 1) / S;
  const int c_begin = s_idx * cb, c_end = min(nblk, c_begin + cb);
  const int nsteps = c_end - c_begin;                            // >= 1: the host picks S so that no split is empty
  const int y_dtype = (flags >> 2) & 3;
  _Float16* x_tile = (_Float16*)lds;                             // [3][128][GEMM_LD]
  float* s_xs = (float*)(x_tile + GEMM_XBUFS * GEMM_TILE_HALVES);   // [3][128]: sum of the block's rotated activations per row
  float* s_fin = (float*)lds;                                    // [2][128][GEMM_FIN_LD], over the blocks once the products are done
  uint32_t& s_failed = *(uint32_t*)(lds + GEMM_LDS_BYTES - 16);  // the finisher's wait gave up
  constexpr int OUT_OF_RANGE = 0x7FFFF000;
  const int l32 = lane & 31, kg = lane >> 5;

  // ---- staging of the rotated activations: 16-byte pieces, piece pi = activation row pi / 16, columns 8 (pi % 16) .. + 7;
  // a thread takes pieces tid, tid + 512, ...; rows beyond M read zeros.  A block is requested three steps before its use, in
  // two register sets: loads return in order, so behind the weight requests of the steps ahead (which take a trip to
  // memory) a block needs as long as they do, however close it sits in the L2.
  constexpr int NPT = GEMM_ROWS * 16 / GEMM_THREADS;               // pieces per thread
  const int tid = (int)threadIdx.x;
  const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc((void*)t.xt_g, 0, M * n * 2, 0x00020000);
  const __amdgpu_buffer_rsrc_t srsrc = __builtin_amdgcn_make_buffer_rsrc((void*)t.xs_g, 0, M * nblk * 16, 0x00020000);
  int piece_src[NPT], piece_lds[NPT];
#pragma unroll
  for (int i = 0; i < NPT; ++i) {
    const int pi = tid + i * GEMM_THREADS, prow = pi >> 4, pg = pi & 15;
    piece_src[i] = prow < rows ? ((j0 + prow) * n + pg * 8) * 2 : -1;
    piece_lds[i] = prow * GEMM_LD + pg * 8;
  }
  const int sum_src = tid < rows ? ((j0 + tid) * nblk) * 16 : -1;          // {even tiles, odd tiles, ...} of block 0
  u4 xg[XSETS][NPT];
  u2 xsg[XSETS];
  auto stage_load = [&](int blk, int set) {    // block index in the row; beyond the split: zeros, no traffic
    HTR_PIN();
    const bool live = blk < c_end;
#pragma unroll
    for (int i = 0; i < NPT; ++i)
      xg[set][i] = __builtin_amdgcn_raw_buffer_load_b128(xrsrc, live && piece_src[i] >= 0 ? piece_src[i] + blk * 256 : OUT_OF_RANGE, 0, 0);
    xsg[set] = __builtin_amdgcn_raw_buffer_load_b64(srsrc, live && sum_src >= 0 ? sum_src + blk * 16 : OUT_OF_RANGE, 0, 0);
    HTR_PIN();
  };
  auto stage_store = [&](int xb, int set) {
#pragma unroll
    for (int i = 0; i < NPT; ++i) *(u4*)(x_tile + xb * GEMM_TILE_HALVES + piece_lds[i]) = xg[set][i];
    if (tid < GEMM_ROWS) s_xs[xb * GEMM_ROWS + tid] = __uint_as_float(xsg[set].x) + __uint_as_float(xsg[set].y);
  };
  stage_load(c_begin, 0);
  if constexpr (XSETS == 2) stage_load(c_begin + 1, 1);

  // ---- the weight stream: lane = (tile column 2 cq + lane / 32, strip 4 rh + lane % 32 / 8, row pair q = lane % 8); the 8
  // lanes of a tile are consecutive, so the history exchange is the one of k_linear.  One descriptor over the row block's
  // eight strips from the split's first byte on; a request beyond the split's last block is sent out of range.
  constexpr int STEP_BYTES = 256 * K;
  const uint32_t strip_bytes = (uint32_t)nblk * STEP_BYTES;
  const uint32_t* base = qw + ((size_t)(rb * 8) * nblk + (size_t)c_begin) * (STEP_BYTES / 4);
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, (int)(7u * strip_bytes + (uint32_t)nsteps * STEP_BYTES), 0x00020000);
  const int lane_off = (4 * rh + (l32 >> 3)) * (int)strip_bytes + ((2 * cq + kg) * 8 + (lane & 7)) * 4 * K;
  int pf_off = 0, pf_left = nsteps;
  StreamRegs<K> buf[P];
  auto prefetch = [&](StreamRegs<K>& dst) {
    HTR_PIN();
    load_stream_buffer<K>(rsrc, pf_left > 0 ? lane_off + pf_off : OUT_OF_RANGE, dst);
    pf_off += STEP_BYTES;
    --pf_left;
    HTR_PIN();
  };
#pragma unroll
  for (int p = 0; p < P; ++p) prefetch(buf[p]);
  const int hist = history_lane_byteaddr(lane);

  // A operands of one step: [even | odd rows][columns 0..7 | 8..15 of the lane's tile].  The matrix instruction sums over
  // 16 k-slots, lanes 0..31 bringing slots 0..7 and lanes 32..63 slots 8..15 of row lane % 32; which weight columns the
  // slots stand for is free as long as the B operand agrees.  So the decode registers are used as they are: in the
  // first instruction of a pair the slots are columns 0..7 of tile column 2 cq (lower lanes) and columns 0..7 of tile
  // column 2 cq + 1 (upper lanes), in the second columns 8..15 of both, and the B operand reads the activations of
  // exactly those columns.  No lane exchange.
  struct Operands { h8 a[2][2]; };
  auto form = [&](const DecodedStep<K>& d, Operands& o) {
    // d.a[0], d.a[1] = row 2q columns 0..7, 8..15; d.a[2], d.a[3] = row 2q + 1 columns 0..7, 8..15 of the lane's tile
#pragma unroll
    for (int par = 0; par < 2; ++par) { o.a[par][0] = d.a[2 * par]; o.a[par][1] = d.a[2 * par + 1]; }
  };

  // activation scale of this lane's column of each 32-row block of the output (activation row 32 jb + lane % 32)
  f16v acc[JB][2];
#pragma unroll
  for (int jb = 0; jb < JB; ++jb)
#pragma unroll
    for (int par = 0; par < 2; ++par)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[jb][par][r] = 0.f;
  float offs[JB];      // running 1534 x sum(x~) of the lane's activation rows over whole blocks (first column quarter only)
#pragma unroll
  for (int jb = 0; jb < JB; ++jb) offs[jb] = 0.f;
  const float k1534 = cq == 0 ? 1534.f : 0.f;
  // B operands: lane (activation row l32 of the 32-row block, k-group kg) reads columns 0..7 (then 8..15) of tile column
  // 2 cq + kg of the block
  const _Float16* b_lane = x_tile + l32 * GEMM_LD + 32 * cq + 16 * kg;

  // products of one decoded step with the staged block in buffer xb
  auto multiply = [&](const Operands& o, int xb) {
    const _Float16* bp = b_lane + xb * GEMM_TILE_HALVES;
#pragma unroll
    for (int jb = 0; jb < JB; ++jb) {
      const h8 b0 = *(const h8*)(bp + jb * 32 * GEMM_LD), b1 = *(const h8*)(bp + jb * 32 * GEMM_LD + 8);
      acc[jb][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(o.a[0][0], b0, acc[jb][0], 0, 0, 0);
      acc[jb][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(o.a[1][0], b0, acc[jb][1], 0, 0, 0);
      acc[jb][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(o.a[0][1], b1, acc[jb][0], 0, 0, 0);
      acc[jb][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(o.a[1][1], b1, acc[jb][1], 0, 0, 0);
      offs[jb] = __builtin_fmaf(k1534, s_xs[xb * GEMM_ROWS + 32 * jb + l32], offs[jb]);
    }
  };
  Operands cur;
  auto decode_next = [&](StreamRegs<K>& sr) {
    DecodedStep<K> d;
    decode_step<K>(sr, hist, d);
    prefetch(sr);
    form(d, cur);
    // the operands exist HERE, in the half in which this wave decodes: without the pin the compiler sinks the whole
    // decode (it touches no memory) across the barrier to its first use, into the half in which the wave multiplies
#pragma unroll
    for (int par = 0; par < 2; ++par) { asm volatile("" : "+v"(cur.a[par][0])); asm volatile("" : "+v"(cur.a[par][1])); }
  };

  // ---- A step has two halves and ONE barrier, at its end.  The two waves that share a SIMD work in opposite order:
  // waves 0..3 multiply block v in the first half and decode block v + 1 in the second, waves 4..7 decode block v
  // first and multiply it second.  So most of the time each SIMD has one wave on the matrix unit and one on the vector
  // unit, and the two run side by side (matrix instructions of one wave do not hold up the vector instructions of
  // another); between barriers the waves run freely, which costs nothing: the loop is as fast as with no barrier at all
  // (a second barrier between the halves cost 7 %).  Block v's activations are in buffer v % 3, stored by every wave
  // during step v - 1 (so complete at that step's barrier); block v + 1's go from registers to their buffer during
  // step v, whose previous content (block v - 2) was last read two barriers ago; block v + 3 is requested then.
  // (Two copies of the loop, chosen once per wave: with the choice inside the loop the compiler keeps the registers of
  // both kinds of half alive side by side and spills.)
  static_assert(P == 2 || P == 4, "stream buffers rotate with the unrolled loop");
  auto run = [&](auto lag_c) {
    constexpr bool LAG = decltype(lag_c)::value;
    if constexpr (!LAG) decode_next(buf[0]);
    stage_store(0, 0);                                           // block 0 (set 0) to buffer 0; the next block not yet requested into set 0
    stage_load(c_begin + XSETS, 0);
    __syncthreads();
    int xb = 0, vstep = 0;                                       // buffer of the step being multiplied, its index
    auto step = [&](StreamRegs<K>& mine, StreamRegs<K>& ahead, bool more, int set) {      // set: register set of block v + 1
      // every wave moves its pieces of block v + 1 to their buffer, and requests those of block v + 2, at the start of
      // the half in which it multiplies: the matrix instructions queue up behind and hide it
      const int xn = xb == GEMM_XBUFS - 1 ? 0 : xb + 1;
      // (scheduling fences between the halves and around the barrier: the halves stay in the order written)
      if constexpr (!LAG) { stage_store(xn, set % XSETS); stage_load(c_begin + vstep + 1 + XSETS, set % XSETS); multiply(cur, xb); } else decode_next(mine);
      HTR_PIN();
      if constexpr (LAG) { stage_store(xn, set % XSETS); stage_load(c_begin + vstep + 1 + XSETS, set % XSETS); multiply(cur, xb); } else { if (more) decode_next(ahead); }
      xb = xn;
      ++vstep;
      HTR_PIN();
      __syncthreads();
      HTR_PIN();
    };
    int v = 0;
    for (; v + P < nsteps; v += P) {
#pragma unroll
      for (int pp = 0; pp < P; ++pp) step(buf[pp], buf[(pp + 1) % P], true, (pp + 1) & 1);
    }
#pragma unroll
    for (int pp = 0; pp < P; ++pp)
      if (v + pp < nsteps) step(buf[pp], buf[(pp + 1) % P], v + pp + 1 < nsteps, (pp + 1) & 1);
  };
  if (w >= 4) run(std::true_type{}); else run(std::false_type{});

  // ---- the four column quarters meet in LDS (the staged blocks are no longer needed: the loop ended with a barrier).
  // D[i][j]: lane holds column j = lane % 32, register r row i = 8 (r / 4) + 4 (lane / 32) + r % 4 of the 32 x 32 piece, and
  // row i of an A operand is strip 4 rh + i / 8, row pair i % 8: weight row 64 rh + 16 (r / 4) + 8 (lane / 32) + 2 (r % 4) + parity,
  // so a lane's values for r = 4 rq .. 4 rq + 3, both parities interleaved, are 8 consecutive rows.
  float scl[JB];
#pragma unroll
  for (int jb = 0; jb < JB; ++jb) {
    const int j = 32 * jb + l32;
    scl[jb] = j < rows ? ((const HTR_GLOBAL float*)t.sc_g)[j0 + j] : 0.f;
  }
#pragma unroll
  for (int phase = 0; phase < 2; ++phase) {
    if ((cq >> 1) == phase) {
      float* copy = s_fin + (cq & 1) * (GEMM_ROWS * GEMM_FIN_LD);
#pragma unroll
      for (int jb = 0; jb < JB; ++jb) {
        float* dst = copy + (32 * jb + l32) * GEMM_FIN_LD + 64 * rh + 8 * kg;
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          f4 lo = {(acc[jb][0][4 * rq] - offs[jb]) * scl[jb], (acc[jb][1][4 * rq] - offs[jb]) * scl[jb],
                   (acc[jb][0][4 * rq + 1] - offs[jb]) * scl[jb], (acc[jb][1][4 * rq + 1] - offs[jb]) * scl[jb]};
          f4 hi = {(acc[jb][0][4 * rq + 2] - offs[jb]) * scl[jb], (acc[jb][1][4 * rq + 2] - offs[jb]) * scl[jb],
                   (acc[jb][0][4 * rq + 3] - offs[jb]) * scl[jb], (acc[jb][1][4 * rq + 3] - offs[jb]) * scl[jb]};
          if (phase == 1) {
            const f4 plo = *(const f4*)(dst + 16 * rq), phi = *(const f4*)(dst + 16 * rq + 4);
            lo += plo; hi += phi;
          }
          *(f4*)(dst + 16 * rq) = lo;
          *(f4*)(dst + 16 * rq + 4) = hi;
        }
      }
    }
    __syncthreads();
  }
  // one copy: the output of the workgroup
  for (int idx = threadIdx.x; idx < GEMM_ROWS * 32; idx += GEMM_THREADS) {
    float* p0 = s_fin + (idx >> 5) * GEMM_FIN_LD + 4 * (idx & 31);
    *(f4*)p0 += *(const f4*)(p0 + GEMM_ROWS * GEMM_FIN_LD);
  }
  __syncthreads();

  // ---- exchange between the splits of a row block.  A split's 128 x 128 partial is too large to hand over word by word
  // with in-band markers (the finisher would pay a memory round trip per row): the partial goes to the workgroup's tile
  // in the scratch half of the workspace with device-scope stores, and ONE flag word per workgroup, set after every
  // thread's stores have been acknowledged, says it is there.  The last split (dispatched after the others, so waiting for
  // them cannot deadlock; bounded all the same) waits for the flags, adds the tiles to its own in LDS and clears the flags.
  constexpr int WAVES = WG_WAVES;
  const size_t wg0 = ((size_t)mt * gridDim.y + rb) * S;              // index of split 0's workgroup of this (row block, tile)
  uint32_t* ready = (uint32_t*)part;                                 // one word per workgroup, zero between launches
  float* tiles = t.tiles;                                            // [workgroups][128][128] floats in the scratch half of the workspace
  if (S > 1) {
    typedef unsigned long long u64;
    if (s_idx != S - 1) {
      u64* dst = (u64*)(tiles + (wg0 + s_idx) * (size_t)(GEMM_ROWS * 128));
      for (int idx = threadIdx.x; idx < rows * 64; idx += GEMM_THREADS) {
        const f2 v = *(const f2*)(s_fin + (idx >> 6) * GEMM_FIN_LD + 2 * (idx & 63));
        __hip_atomic_store(dst + idx, __builtin_bit_cast(u64, v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      // The tile went out as device-scope (write-through) stores, so nothing of it sits dirty in this XCD's L2: the stores
      // only have to be complete before the flag is set.  That is a wait for their acknowledgements, not the cache-wide
      // writeback a device-scope release fence asks for (which, from every wave of every contributor, cost 14 us of a
      // 42 us launch with four splits and 50 us with eight).
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_s_waitcnt(0x0F70);                            // vmcnt(0)
      __syncthreads();
      if (threadIdx.x == 0) __hip_atomic_store(ready + wg0 + s_idx, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return;
    }
    if (w == 0) {
      bool failed = false;
      int tries = 0;
      for (;;) {
        const uint32_t f = lane < S - 1 ? __hip_atomic_load(ready + wg0 + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 1u;
        if (!__any(f == 0u)) break;
        if (++tries >= t.spin_limit) { failed = true; break; }
        __builtin_amdgcn_s_sleep(8);
      }
      // the tiles are read with device-scope loads below, which are served from memory, not from this XCD's caches: no
      // invalidate is needed, only the order flag-before-tile, which the barrier below gives
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
      if (lane == 0) {
        s_failed = failed ? 1u : 0u;
        if (failed) report_give_up(t.status);
      }
    }
    __syncthreads();
    if (s_failed == 0u) {
      // own tile += the other splits' tiles: a thread's pieces (8 bytes each) of every contributor are requested together,
      // so the sum costs a few memory round trips, not one per contributor
      const u64* src = (const u64*)(tiles + wg0 * (size_t)(GEMM_ROWS * 128));
      for (int base = threadIdx.x; base < rows * 64; base += 4 * GEMM_THREADS) {
        u64 got[7][4];
#pragma unroll
        for (int k = 0; k < 7; ++k)
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int idx = base + u * GEMM_THREADS;
            got[k][u] = k < S - 1 && idx < rows * 64
                            ? __hip_atomic_load(src + (size_t)k * (GEMM_ROWS * 64) + idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0ull;
          }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int idx = base + u * GEMM_THREADS;
          if (idx < rows * 64) {
            f2* own = (f2*)(s_fin + (idx >> 6) * GEMM_FIN_LD + 2 * (idx & 63));
            f2 sum = *own;
#pragma unroll
            for (int k = 0; k < 7; ++k) { const f2 g = __builtin_bit_cast(f2, got[k][u]); sum.x += g.x; sum.y += g.y; }
            *own = sum;
          }
        }
      }
      if (threadIdx.x < S - 1) __hip_atomic_store(ready + wg0 + threadIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
  }

  // ---- output side, one activation row per wave and turn; lane holds output rows lane and lane + 64 of the row block
  const bool failed = load_status(t.status) != 0u || (S > 1 && s_failed != 0u);   // also: an earlier launch on this workspace gave up
  const int r0 = rb * 128 + lane, r1 = r0 + 64;
  const float rs0 = f16_bits_to_float(((const HTR_GLOBAL uint16_t*)t.scales)[r0]) * t.cbscale * INV_SQRT128;
  const float rs1 = f16_bits_to_float(((const HTR_GLOBAL uint16_t*)t.scales)[r1]) * t.cbscale * INV_SQRT128;
  const float sg0 = ((((const HTR_GLOBAL uint8_t*)t.sv)[r0 >> 3] >> (lane & 7)) & 1u) ? -1.f : 1.f;
  const float sg1 = ((((const HTR_GLOBAL uint8_t*)t.sv)[r1 >> 3] >> (lane & 7)) & 1u) ? -1.f : 1.f;
  float b0v = 0.f, b1v = 0.f;
  if (t.bias != nullptr) { b0v = load_elem_g(t.bias, y_dtype, r0); b1v = load_elem_g(t.bias, y_dtype, r1); }
  for (int j = w; j < rows; j += WAVES) {
    const float* own = s_fin + j * GEMM_FIN_LD;
    float v0s = own[lane] * rs0, v1s = own[lane + 64] * rs1;
    fwht128_wave(v0s, v1s, lane);
    v0s = __builtin_fmaf(v0s, sg0, b0v);
    v1s = __builtin_fmaf(v1s, sg1, b1v);
    if (failed) { v0s = __builtin_nanf(""); v1s = v0s; }
    store_elem_g(t.y, y_dtype, (size_t)(j0 + j) * m + r0, v0s);
    store_elem_g(t.y, y_dtype, (size_t)(j0 + j) * m + r1, v1s);
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

// ------------------------------------------------------------------------------------------------ workspace set-up
// Zeroes the first `bytes` (a multiple of 16) of a workspace and writes the header's mirror address.  A kernel, not a
// memset, so that it can be recorded into a HIP graph.
__global__ __launch_bounds__(256) void k_workspace_init(u4* __restrict__ ws, size_t bytes, unsigned long long mirror) {
  const size_t n16 = bytes / 16;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256)
    ws[i] = i == 0 ? u4{0u, 0u, (uint32_t)mirror, (uint32_t)(mirror >> 32)} : u4{0u, 0u, 0u, 0u};
}

// ------------------------------------------------------------------------------------------------ host side
thread_local int g_last_hip_error = 0;
std::atomic<int> g_spin_limit{1 << 20};     // polls (about a microsecond each) before a finishing workgroup gives up

struct Plan { int chunk, wgs, segfin, nbl, mb, prerot; size_t lds; };

// Workspace: two halves, split at workspace_bytes / 2 (rounded down to 256).  First half: [256-byte header: status
// word][one partial slot per workgroup]; it must be all-zero between calls.  Second half: scratch for the pre-rotated
// activations, left as it is.  The split depends only on the size the caller passes, not on the problem, so no call can
// leave scratch data where a later call of another shape expects zeroed slots (as long as the caller passes the same
// size with the same buffer).
constexpr size_t WS_HEADER = 256;
inline size_t align256(size_t v) { return (v + 255) / 256 * 256; }
inline size_t ws_need(size_t slot_bytes, size_t scratch_bytes) {
  const size_t a = align256(WS_HEADER + slot_bytes), b = align256(scratch_bytes);
  return 2 * (a > b ? a : b);
}
inline size_t ws_half(size_t workspace_bytes) { return workspace_bytes / 2 / 256 * 256; }
// bytes of the pre-rotated activations, their block sums and the row scales
inline size_t prerot_bytes(int n, int M) { return align256((size_t)M * n * 2) + align256((size_t)M * (n / 128) * 16) + align256((size_t)M * 4); }

// ---- facts of the device the plans are made for: compute units and LDS bytes per compute unit, read once per device
// (the current one) from the runtime; an unpartitioned MI355X (256 CUs, 160 KB) where no device can be asked (plans
// computed on a machine without a GPU).  htr_plan_device_override replaces them for every device (tests, tuning).
struct DeviceFacts { int cus; size_t lds; };
constexpr int MAX_DEVICES = 64;
constexpr DeviceFacts MI355X_FACTS = {256, 160 * 1024};
std::atomic<int> g_override_cus{0};
std::atomic<long> g_override_lds{0};
inline DeviceFacts device_facts() {
  static DeviceFacts table[MAX_DEVICES];
  static std::atomic<uint64_t> known{0};
  const int ov = g_override_cus.load(std::memory_order_acquire);
  if (ov > 0) return DeviceFacts{ov, (size_t)g_override_lds.load(std::memory_order_acquire)};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return MI355X_FACTS; }
  if (dev < 0 || dev >= MAX_DEVICES) return MI355X_FACTS;
  const uint64_t bit = (uint64_t)1 << dev;
  if (known.load(std::memory_order_acquire) & bit) return table[dev];
  int cus = 0, lds = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1 ||
      hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, dev) != hipSuccess || lds < 64 * 1024) {
    (void)hipGetLastError();
    return MI355X_FACTS;
  }
  table[dev] = DeviceFacts{cus, (size_t)lds};        // two threads racing here store the same values
  known.fetch_or(bit, std::memory_order_release);
  return table[dev];
}
inline int num_cu() { return device_facts().cus; }
constexpr int MAX_ROW_BLOCKS = 16384;
constexpr int MAX_CHUNK = 4096;
// the kernel divides step indices by n / 128 with a 40-bit reciprocal: exact while indices stay below 2^24
inline bool shape_ok(int m, int n) {
  return m > 0 && n > 0 && m % 128 == 0 && n % 128 == 0 && m / 128 <= MAX_ROW_BLOCKS && n / 128 < 65536 &&
         (long)(m / 128) * (n / 128) < (1L << 24) - 2 * MAX_CHUNK;
}

inline bool plan_for_chunk(int m, int n, int M, int chunk, Plan& pl) {
  const int nblk = n / 128, rbs = m / 128;
  const long vtotal = (long)rbs * nblk;
  if (chunk < 1 || chunk > vtotal || chunk > MAX_CHUNK) return false;
  pl.chunk = chunk;
  pl.wgs = (int)((vtotal + chunk - 1) / chunk);
  pl.segfin = (chunk + nblk - 1) / nblk;            // row blocks that can end inside one chunk
  pl.nbl = chunk < nblk ? chunk : nblk;
  pl.lds = lds_bytes(M, pl.nbl, pl.segfin);
  if (pl.lds > (size_t)LDS_BUDGET) return false;
  // a workgroup rotates its own column blocks while that is at most ROT_PAIRS (row, block) pairs (MAX_ROT_PAIRS with up
  // to eight rows: the kernel variant with several passes); beyond that the activations are rotated once, ahead of
  // the launch
  pl.prerot = M * pl.nbl > (M <= 8 ? MAX_ROT_PAIRS : ROT_PAIRS) ? 1 : 0;
  return true;
}

// Picks the chunk length (virtual steps per workgroup) with a cost model in microseconds fitted to chunk-length sweeps
// on MI355X (K4, 1..8 rows, nine shapes from 1024x4096 to 28672x4096, twenty chunk lengths each; the choice is within
// 1 % of the best measured chunk on average, 10 % at worst): a fixed latency chain (launch, x fetch, rotation, partial
// exchange, output rotation) that grows with the contributors a finisher reads, eight per round trip; a cost per
// step that depends on how many workgroups share a CU (one: the workgroup's own decode rate, 0.4 .. 0.5 us; several:
// throughput bound, proportional to the load of the fullest CU, plus a set-up per workgroup); a penalty for chunks
// that do not tile the rows of column blocks; the extra launch of a pre-rotation; and the growth of all per-step work
// with the number of activation rows.
inline bool search_plan(int m, int n, int M, int nsplit, int cus, Plan& pl) {
  const int nblk = n / 128, rbs = m / 128;
  const long vtotal = (long)rbs * nblk;
  pl.mb = M <= 8 ? 1 : (M <= 16 ? 2 : 4);
  if (nsplit > 0) {                                                 // explicit plan (tuning): chunk length in the low
    const int chunk = nsplit & 0xFFFFF;                             // 20 bits, bit 30 = force pre-rotation
    bool ok = chunk > 0 ? plan_for_chunk(m, n, M, chunk, pl) : false;
    if (ok && (nsplit & (1 << 30))) pl.prerot = 1;
    return ok;
  }
  if (vtotal >= (long)64 * cus && nblk <= 64 && plan_for_chunk(m, n, M, nblk, pl)) return true;
  const double rows = M <= 8 ? 1.0 + 0.06 * (M - 1) : (M <= 16 ? 2.2 : 6.5);
  double best = 1e30;
  bool found = false;
  const int max_chunk = (int)(vtotal < MAX_CHUNK ? vtotal : MAX_CHUNK);
  for (int chunk = 1; chunk <= max_chunk; ++chunk) {
    Plan c;
    c.mb = pl.mb;
    if (!plan_for_chunk(m, n, M, chunk, c)) continue;
    const double fill = (double)c.wgs / cus;
    const bool aligned = (nblk % chunk == 0) || (chunk % nblk == 0);
    const int contributors = chunk >= nblk ? 1 : (nblk + chunk - 1) / chunk;
    const double steps = chunk * (aligned ? 1.0 : 1.06 + 0.04 * (M - 1));
    // one workgroup per CU or fewer: the chip works through `chunk` steps once; more: the fullest CU works through
    // its workgroups one after the other, each with its own set-up and partial hand-over
    // (a grid slightly above one workgroup per CU leaves a few CUs with two: it costs nearly as much as two everywhere)
    const double fill2 = fill < 1.5 ? 1.5 : fill;
    const double body = fill <= 1.0 ? rows * (0.4 + 0.05 * fill) * steps
                                    : fill2 * (rows * 0.55 * steps + 0.5 + 0.1 * M);
    // hand-over: the contributors' slots are read eight per round trip to memory (0.45 us each)
    const double handover = 0.45 * ((contributors - 1 + 7) / 8);
    const int passes = (M * c.nbl + ROT_PAIRS - 1) / ROT_PAIRS;      // rotation passes inside the kernel, 0.3 us each after the first
    const double t = 4.5 + handover + (c.prerot ? 3.0 + 0.1 * M : 0.3 * (passes - 1)) + body;
    if (t < best) { best = t; pl = c; found = true; }
  }
  return found;
}

// The search above walks every chunk length (up to 4096 of them): tens of microseconds on the host, more than the launch
// it plans.  Plans depend only on (m, n, M, nsplit) and the device's CU count, so the last 64 distinct ones are kept.
inline bool make_plan(int m, int n, int M, int nsplit, Plan& pl) {
  const int cus = num_cu();
  struct Entry { int m, n, M, nsplit, cus; bool ok; Plan pl; };
  static Entry cache[64];
  static int filled = 0, next = 0;
  static std::atomic_flag busy = ATOMIC_FLAG_INIT;
  while (busy.test_and_set(std::memory_order_acquire)) {}
  for (int i = 0; i < filled; ++i) {
    const Entry& e = cache[i];
    if (e.m == m && e.n == n && e.M == M && e.nsplit == nsplit && e.cus == cus) {
      const bool ok = e.ok;
      pl = e.pl;
      busy.clear(std::memory_order_release);
      return ok;
    }
  }
  busy.clear(std::memory_order_release);
  Plan found = {};
  const bool ok = search_plan(m, n, M, nsplit, cus, found);
  while (busy.test_and_set(std::memory_order_acquire)) {}
  Entry& e = cache[next];
  e.m = m; e.n = n; e.M = M; e.nsplit = nsplit; e.cus = cus; e.ok = ok; e.pl = found;
  next = (next + 1) % 64;
  if (filled < 64) ++filled;
  busy.clear(std::memory_order_release);
  pl = found;
  return ok;
}

// The dispatcher places workgroups wherever resources allow, not evenly: with 512 equal workgroups some CUs receive
// three and others one, and the kernel ends with the most loaded CU.  Requesting 1/k of a CU's LDS (160 KB on MI355X) per
// workgroup (k = workgroups per CU when spread evenly) makes exactly k fit, so the spread is even.
inline size_t balanced_lds_request(size_t needed, int grid) {
  const DeviceFacts df = device_facts();
  const int k = (grid + df.cus - 1) / df.cus;
  if (k > 4) return needed;
  const size_t share = (df.lds / k) / 1024 * 1024 - 1024;
  return share > needed ? share : needed;
}

// One launch with the runtime's own return value (hipGetLastError after a launch macro would also report an earlier,
// unrelated failure of the thread as this launch's).
template <typename T> struct same_type { typedef T type; };
template <typename... KArgs>
hipError_t launch_kernel(void (*kern)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t st, typename same_type<KArgs>::type... args) {
  void* argv[] = {(void*)&args...};
  return hipLaunchKernel((const void*)kern, grid, block, argv, lds, st);
}
// Kernels that may ask for more than the default 48 KB of dynamic LDS get the limit raised to the whole 160 KB once per
// (kernel, device), not per launch with the launch's own value: the attribute is state of the function, and two host
// threads that set different values around their launches would race.
constexpr int MAX_DYNAMIC_LDS = 160 * 1024;
template <auto Kern> hipError_t allow_full_lds() {
  static std::atomic<uint64_t> done{0};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const uint64_t bit = (uint64_t)1 << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
  e = hipFuncSetAttribute((const void*)Kern, hipFuncAttributeMaxDynamicSharedMemorySize, MAX_DYNAMIC_LDS);
  if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
  return e;
}
#define HTR_CHECK_HIP(EXPR) do { hipError_t e_ = (EXPR); if (e_ != hipSuccess) { g_last_hip_error = (int)e_; return HTR_ERR_LAUNCH; } } while (0)

struct LinearLaunch {
  const uint32_t* qw; const void* x; const uint8_t* su; float* part;
  int m, n, M, chunk, flags, problems;
  unsigned long long nblk_magic;
  LinearTail tail;
};

template <int K, int MB, bool DEEP, bool PREROT, int RP = 1, bool PACE = false>
int launch_linear_v(const LinearLaunch& a, int grid, size_t lds, hipStream_t st) {
  constexpr int P = K <= 4 ? 4 : (K <= 6 ? 3 : 2);          // wave-steps of weights in flight
  constexpr int D = DEEP && P >= 4 ? 4 : 2;                 // steps decoded ahead of the activation exchange
  lds = balanced_lds_request(lds, grid * a.problems);
  HTR_CHECK_HIP((allow_full_lds<k_linear<K, MB, P, D, PREROT, RP, 0, PACE>>()));
  HTR_CHECK_HIP(launch_kernel(k_linear<K, MB, P, D, PREROT, RP, 0, PACE>, dim3(grid, a.problems), dim3(WG_THREADS), lds, st, a.qw, a.x, a.su,
                              a.part, a.m, a.n, a.M, a.chunk, a.flags, a.nblk_magic, a.tail));
  return HTR_OK;
}
// Where the two waves of a SIMD are kept in step by alternating priorities (k_linear's PACE): chunks of twelve steps and
// more, one launch (not a group), and either up to four activation rows or at most two chunks per row block.
// Measured on MI355X, K4, us without -> with: 28672x4096 1 row 19.1 -> 17.7, 4 rows 22.0 -> 20.5, 8 rows 23.3 -> 23.5;
// 14336x4096 1 / 4 / 8 rows 12.3 -> 11.8, 13.7 -> 12.9, 15.8 -> 14.4; 4096x14336 (eight chunks per row block) 1 / 4 / 6 /
// 8 rows 11.9 -> 11.2, 12.9 -> 12.7, 14.0 -> 14.1, 14.9 -> 16.0; 6144x4096 8 rows (chunks of 8) 10.0 -> 13.8.
inline bool paced(const LinearLaunch& a) {
  static const bool on = getenv("HTR_PACE") == nullptr || atoi(getenv("HTR_PACE")) != 0;
  const int nblk = a.n / 128;
  return on && a.problems == 1 && a.chunk >= 12 && (a.M <= 4 || (nblk + a.chunk - 1) / a.chunk <= 2);
}
// Short chunks are decoded completely ahead of the activation exchange (more registers, so only for one activation
// block and chunks whose prologue latency is a large part of the kernel); long chunks prefer occupancy.
template <int K, bool PREROT> int launch_linear_kr(const LinearLaunch& a, int mb, int grid, size_t lds, hipStream_t st) {
  const bool deep = a.chunk <= 8;
  if constexpr (!PREROT) {                 // more pairs than one pass rotates: the variant with several passes (up to 8 rows)
    const int nblk = a.n / 128;
    if (mb == 1 && a.M * (a.chunk < nblk ? a.chunk : nblk) > ROT_PAIRS)
      return paced(a) ? launch_linear_v<K, 1, false, false, MAX_ROT_PASSES, true>(a, grid, lds, st)
                      : launch_linear_v<K, 1, false, false, MAX_ROT_PASSES>(a, grid, lds, st);
    if (mb == 1 && !deep && paced(a)) return launch_linear_v<K, 1, false, false, 1, true>(a, grid, lds, st);
  }
  switch (mb) {
    case 1: return deep ? launch_linear_v<K, 1, true, PREROT>(a, grid, lds, st) : launch_linear_v<K, 1, false, PREROT>(a, grid, lds, st);
    case 2: return launch_linear_v<K, 2, false, PREROT>(a, grid, lds, st);
    default: return launch_linear_v<K, 4, false, PREROT>(a, grid, lds, st);
  }
}
template <int K> int launch_linear_k(const LinearLaunch& a, bool prerot, int mb, int grid, size_t lds, hipStream_t st) {
  return prerot ? launch_linear_kr<K, true>(a, mb, grid, lds, st) : launch_linear_kr<K, false>(a, mb, grid, lds, st);
}

// ---- batched kernel: split S of the column blocks per row block
struct BatchPlan { int S, cb, wgs, mb, rot, last_finishes; size_t lds; };
// rows x column blocks per split up to which a workgroup of the batched kernel rotates its own activations (256 pairs,
// eight passes per wave) instead of a rotation launch: 16 x 16 or 32 x 8
inline bool batch_rot_fits(int M, int cb) { return (M <= 16 && cb <= 16) || (M <= 32 && cb <= 8); }
constexpr int BATCH_MIN_M = 9;      // rows from which the library policy takes the batched kernel on every shape
inline int batch_groups(int M) { return M <= 16 ? 1 : (M <= 32 ? 2 : (M <= 64 ? 4 : 8)); }   // groups of 16 activation rows
inline size_t batch_lds_bytes(int M) {
  const int rows = 16 * batch_groups(M);
  const size_t blocks = (size_t)2 * rows * BATCH_ROWH * 2, small = (size_t)5 * rows * 4, fin = (size_t)2 * M * BATCH_FIN_STRIDE * 4;
  return M > 64 ? (blocks + small > fin ? blocks + small : fin) : blocks + small + fin;
}
inline bool make_batch_plan(int m, int n, int M, int want_S, BatchPlan& bp) {
  const int nblk = n / 128, rbs = m / 128;
  if ((long)M * n * 2 >= (1L << 31)) return false;          // the kernels address the rotated activations with 32-bit byte offsets
  bp.mb = batch_groups(M);
  bp.lds = batch_lds_bytes(M);
  bp.rot = 0;
  // Measured on MI355X (K4, 6..128 rows, 1024..28672 output rows): one workgroup per CU is the best fill; every further
  // split adds partial traffic that grows with the rows (14336x4096, 32 rows: 2 splits 19.9 us, 4 splits 24.5; 128
  // rows: 39 against 48).  So: the largest split that keeps the grid within the CU count, among the splits that leave
  // no column range empty, and at most 8 of them (the output side requests the slots of up to eight other splits in
  // one go; 1024x4096 and 2048x4096 at 8..32 rows: 8 splits 11..12 us, 16 splits 11..16, 32 splits 14..22).
  const int cus = num_cu();
  const int by_cus = cus / rbs > 1 ? cus / rbs : 1;
  const int limit = want_S > 0 ? want_S : (by_cus < 8 ? by_cus : 8);
  bool found = false;
  for (int S = 1; S <= nblk && S <= limit; ++S) {
    const int cb = (nblk + S - 1) / S;
    if ((nblk + cb - 1) / cb != S) continue;                       // some split would be empty
    if (want_S > 0 && S != want_S) continue;
    bp.S = S; bp.cb = cb; bp.wgs = rbs * S; found = true;
  }
  // Splits that finish rows for each other wait for each other, which is only safe while every workgroup of the grid is
  // resident at once: one workgroup per CU at most.  A larger grid (an explicit split, a device with fewer CUs than the
  // policy assumed) falls back to the last split finishing everything: it waits only for workgroups dispatched before it.
  bp.last_finishes = found && bp.wgs > cus ? 1 : 0;
  // Few rows over few column blocks per split, one workgroup per CU: every workgroup rotates its own slice.
  // HTR_BATCH_ROT=0 switches it off.
  static const bool rot_on = getenv("HTR_BATCH_ROT") == nullptr || atoi(getenv("HTR_BATCH_ROT")) != 0;
  if (found && rot_on && batch_rot_fits(M, bp.cb) && bp.wgs <= cus) {
    const int rows = 16 * bp.mb;
    bp.rot = 1;
    bp.lds = (size_t)bp.cb * rows * BATCH_ROWH * 2 + (size_t)bp.cb * 2 * rows * 4 + rows * 4 + (size_t)2 * M * BATCH_FIN_STRIDE * 4;
  }
  return found;
}

// ---- GEMM kernel (more than 128 rows): tiles of GEMM_ROWS activation rows in the grid's z, split S of the column blocks
// while the grid stays within one workgroup per compute unit (256 registers per lane leave room for one)
struct GemmPlan { int S, cb, mtiles, wgs, jb; };
constexpr int GEMM_MIN_M = HTR_MAX_ROWS_PER_TILE + 1;       // rows from which the library policy takes the GEMM kernel
inline bool gemm_plan_for(int m, int n, int M, int want_S, int jb, GemmPlan& gp) {
  const int nblk = n / 128, rbs = m / 128, rows = 32 * jb;
  if ((long)M * n * 2 >= (1L << 31)) return false;          // the kernel addresses the rotated activations with 32-bit byte offsets
  gp.jb = jb;
  gp.mtiles = (M + rows - 1) / rows;
  if (gp.mtiles > 65535) return false;
  const long base = (long)rbs * gp.mtiles;
  const int cus = num_cu();
  const int by_cus = cus / base > 1 ? (int)(cus / base) : 1;
  const int limit = want_S > 0 ? want_S : (by_cus < 4 ? by_cus : 4);
  bool found = false;
  for (int S = 1; S <= nblk && S <= limit && S <= 8; ++S) {
    const int cb = (nblk + S - 1) / S;
    if ((nblk + cb - 1) / cb != S) continue;                       // some split would be empty
    if (want_S > 0 && S != want_S) continue;
    gp.S = S; gp.cb = cb; gp.wgs = (int)(base * S); found = true;
  }
  return found;
}
// Tile height by a cost model in microseconds fitted to MI355X (K4): rounds of workgroups over the CUs x (steps per
// workgroup x 0.94 us with 96-row tiles, 1.16 us with 128-row tiles, + 10 us of fixed cost, + 4 + 1.5 (S - 1) us for the
// exchange between S column splits).  128-row tiles win where they save a round (14336x4096 at 256 rows: two tiles
// fill the chip once, 49 us, where three tiles of 96 rows take 73) or allow more splits of long rows (4096x14336 at 256
// rows: 55 against 64); 96-row tiles win otherwise (14336x4096 at 192 rows: 40 against 47; at 384 rows: 79 against 94).
// want_jb: 0 = this policy, 3 or 4 = that tile height.  By policy at most four splits (eight cost more than they save).
inline double gemm_plan_cost(const GemmPlan& gp) {
  const int cus = num_cu();
  const int rounds = (gp.wgs + cus - 1) / cus;
  return rounds * (gp.cb * (gp.jb == 3 ? 0.94 : 1.16) + 10.0 + (gp.S > 1 ? 4.0 + 1.5 * (gp.S - 1) : 0.0));
}
inline bool make_gemm_plan(int m, int n, int M, int want_S, int want_jb, GemmPlan& gp) {
  if (want_jb == 3 || want_jb == 4) return gemm_plan_for(m, n, M, want_S, want_jb, gp);
  GemmPlan a, b;
  const bool oka = gemm_plan_for(m, n, M, want_S, 3, a), okb = gemm_plan_for(m, n, M, want_S, 4, b);
  if (!oka && !okb) return false;
  gp = oka && (!okb || gemm_plan_cost(a) <= gemm_plan_cost(b)) ? a : b;
  return true;
}
// workspace of the GEMM kernel: one flag word per workgroup in the zeroed half; rotated activations and the exchange tiles
// (only with column splits) in the scratch half
inline size_t gemm_scratch_bytes(int n, int M, const GemmPlan& gp) {
  return prerot_bytes(n, M) + (gp.S > 1 ? (size_t)gp.wgs * (32 * gp.jb) * 128 * sizeof(float) : 0);
}
// nsplit bits 20 and 21 with the GEMM kernel: tiles of 96 or of 128 activation rows (neither: the policy above)
inline int gemm_want_jb(int nsplit) { return nsplit > 0 ? ((nsplit >> 20) & 1 ? 3 : ((nsplit >> 21) & 1 ? 4 : 0)) : 0; }
// nsplit bit 28: the GEMM kernel with the split in the low bits (0 = its own policy); otherwise from GEMM_MIN_M rows
inline bool wants_gemm(int M, int nsplit) { return nsplit > 0 ? (nsplit & (1 << 28)) != 0 : M >= GEMM_MIN_M; }

struct BatchArgs { const uint32_t* qw; float* part; const void* x; const uint8_t* su; int m, n, M, flags; };
template <int K, int MB, bool ROT> int launch_batch_v(const BatchArgs& a, const LinearTail& t, const BatchPlan& bp, hipStream_t st) {
  const size_t lds = balanced_lds_request(bp.lds, bp.wgs);
  HTR_CHECK_HIP((allow_full_lds<k_linear_batch<K, MB, 4, ROT>>()));
  HTR_CHECK_HIP(launch_kernel(k_linear_batch<K, MB, 4, ROT>, dim3(bp.S, a.m / 128), dim3(WG_THREADS), lds, st, a.qw, a.part, a.x, a.su,
                              a.m, a.n, a.M, bp.S, a.flags, t));
  return HTR_OK;
}
template <int K> int launch_batch_k(const BatchArgs& a, bool rot, const LinearTail& t, const BatchPlan& bp, hipStream_t st) {
  if (rot) return bp.mb == 1 ? launch_batch_v<K, 1, true>(a, t, bp, st) : launch_batch_v<K, 2, true>(a, t, bp, st);
  switch (bp.mb) {
    case 1: return launch_batch_v<K, 1, false>(a, t, bp, st);
    case 2: return launch_batch_v<K, 2, false>(a, t, bp, st);
    case 4: return launch_batch_v<K, 4, false>(a, t, bp, st);
    default: return launch_batch_v<K, 8, false>(a, t, bp, st);
  }
}
// nsplit bit 29: batched kernel with the split in the low bits (0 = policy); otherwise the policy decides by M
// Tall matrices (192 row blocks and more) fill the chip without column splits, so the batched kernel needs no exchange
// there and wins from 6 rows (65536x4096, 8 rows: 41 against 50 us; 152064x4096: 91 against 95).
// A matrix whose splits are four column blocks or fewer on a full grid (4096x4096: 8 splits of 4 blocks) is also ahead
// with the batched kernel at 7 and 8 rows, when its workgroups rotate their own slices (8 rows: 9.2 against 10.4 us).
inline bool wants_batch(int M, int nsplit, int m, int n) {
  if (wants_gemm(M, nsplit)) return false;
  if (nsplit > 0) return (nsplit & (1 << 29)) != 0;
  if (M >= BATCH_MIN_M || (M >= 6 && m / 128 >= 192)) return true;
  if (M >= 7) {
    BatchPlan bp;
    return make_batch_plan(m, n, M, 0, bp) && bp.rot && bp.cb <= 4 && bp.wgs >= num_cu();
  }
  return false;
}

// Rotation of all rows of x ahead of a linear launch: on the matrix unit for 16-bit rows on 16-byte boundaries, else the
// butterfly kernel (float32, odd alignments)
inline hipError_t launch_rotation(const void* x, const uint8_t* su, int n, int M, int x_dtype, const LinearTail& t, hipStream_t st) {
  static const bool mfma_on = getenv("HTR_ROTATE_MFMA") == nullptr || atoi(getenv("HTR_ROTATE_MFMA")) != 0;
  if (mfma_on && x_dtype != HTR_F32 && ((uintptr_t)x & 15) == 0)
    return launch_kernel(k_rotate_mfma, dim3((n / 128 + 4 * WG_WAVES - 1) / (4 * WG_WAVES), M), dim3(WG_THREADS), 0, st, x, su, n,
                         x_dtype == HTR_BF16 ? 1 : 0, (_Float16*)t.xt_g, (float*)t.xs_g, (float*)t.sc_g);
  return launch_kernel(k_rotate, dim3((n / 128 + WG_WAVES - 1) / WG_WAVES, M), dim3(WG_THREADS), 0, st, x, su, n, x_dtype,
                       (_Float16*)t.xt_g, (float*)t.xs_g, (float*)t.sc_g, (const htr_group_entry*)nullptr, 0ull);
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
    case HTR_ERR_BATCH: return "M must be in 1..2048 for one launch (1..128 for an explicit chunked or batched plan, 1..32 for a grouped problem)";
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
  if (K < 2 || K > 8 || !shape_ok(m, n) || M < 1 || M > HTR_MAX_BATCH) return 0;
  if (wants_gemm(M, nsplit)) {
    GemmPlan gp;
    if (!make_gemm_plan(m, n, M, nsplit > 0 ? nsplit & 0xFFFFF : 0, gemm_want_jb(nsplit), gp)) return 0;
    return ws_need((size_t)gp.wgs * sizeof(uint32_t), gemm_scratch_bytes(n, M, gp));
  }
  if (M > HTR_MAX_ROWS_PER_TILE) return 0;       // the other kernels take up to 128 rows
  if (wants_batch(M, nsplit, m, n)) {
    BatchPlan bp;
    if (!make_batch_plan(m, n, M, nsplit > 0 ? nsplit & 0xFFFFF : 0, bp)) return 0;
    return ws_need((size_t)bp.wgs * M * 128 * sizeof(float), prerot_bytes(n, M));
  }
  if (M > HTR_MAX_GROUP_ROWS) return 0;          // the chunked kernel takes up to 32 rows
  Plan pl;
  if (!make_plan(m, n, M, nsplit, pl)) return 0;
  return ws_need((size_t)pl.wgs * M * 128 * sizeof(float), prerot_bytes(n, M));
}

int htr_linear_plan(int m, int n, int K, int M, int nsplit, int* out6) {
  if (!out6) return HTR_ERR_NULL;
  if (K < 2 || K > 8) return HTR_ERR_K;
  if (!shape_ok(m, n)) return HTR_ERR_SHAPE;
  if (M < 1 || M > HTR_MAX_BATCH) return HTR_ERR_BATCH;
  if (wants_gemm(M, nsplit)) {
    GemmPlan gp;
    if (!make_gemm_plan(m, n, M, nsplit > 0 ? nsplit & 0xFFFFF : 0, gemm_want_jb(nsplit), gp)) return HTR_ERR_SPLIT;
    out6[0] = gp.cb; out6[1] = gp.wgs; out6[2] = gp.mtiles; out6[3] = gp.S; out6[4] = 1; out6[5] = (int)gemm_lds_bytes(gp.jb);
    return HTR_OK;
  }
  if (M > HTR_MAX_ROWS_PER_TILE) return HTR_ERR_BATCH;
  if (wants_batch(M, nsplit, m, n)) {
    BatchPlan bp;
    if (!make_batch_plan(m, n, M, nsplit > 0 ? nsplit & 0xFFFFF : 0, bp)) return HTR_ERR_SPLIT;
    out6[0] = bp.cb; out6[1] = bp.wgs; out6[2] = bp.last_finishes ? 0 : 1; out6[3] = bp.S; out6[4] = bp.rot ? 0 : 1; out6[5] = (int)bp.lds;
    return HTR_OK;
  }
  if (M > HTR_MAX_GROUP_ROWS) return HTR_ERR_BATCH;
  Plan pl;
  if (!make_plan(m, n, M, nsplit, pl)) return HTR_ERR_SPLIT;
  out6[0] = pl.chunk; out6[1] = pl.wgs; out6[2] = pl.segfin; out6[3] = pl.nbl; out6[4] = pl.prerot; out6[5] = (int)pl.lds;
  return HTR_OK;
}

void htr_set_spin_limit(int polls) { g_spin_limit.store(polls < 1 ? 1 : polls, std::memory_order_relaxed); }

int htr_plan_device_override(int compute_units, long lds_bytes_per_cu) {
  if (compute_units == 0) { g_override_cus.store(0, std::memory_order_release); return HTR_OK; }
  if (compute_units < 1 || compute_units > 4096 || lds_bytes_per_cu < 64 * 1024 || lds_bytes_per_cu > (1 << 20)) return HTR_ERR_SHAPE;
  g_override_lds.store(lds_bytes_per_cu, std::memory_order_release);
  g_override_cus.store(compute_units, std::memory_order_release);
  return HTR_OK;
}

int htr_workspace_init(void* workspace, size_t workspace_bytes, void* host_status_word, void* stream) {
  if (!workspace) return HTR_ERR_NULL;
  if (workspace_bytes < 2 * WS_HEADER || ((uintptr_t)workspace & 255) || ((uintptr_t)host_status_word & 3)) return HTR_ERR_WORKSPACE;
  const size_t half = ws_half(workspace_bytes);
  const size_t n16 = half / 16;
  const unsigned blocks = (unsigned)(n16 / 256 < 1 ? 1 : (n16 / 256 > 2048 ? 2048 : n16 / 256));
  HTR_CHECK_HIP(launch_kernel(k_workspace_init, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (u4*)workspace, half,
                              (unsigned long long)(uintptr_t)host_status_word));
  return HTR_OK;
}

unsigned long long htr_stream_capture_id(void* stream) {
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  unsigned long long id = 0;
  if (hipStreamGetCaptureInfo((hipStream_t)stream, &status, &id) != hipSuccess) { (void)hipGetLastError(); return 0; }
  return status == hipStreamCaptureStatusActive ? (id != 0 ? id : ~0ull) : 0;
}

int htr_linear(const void* qweight, const void* scales, const void* su, const void* sv, const void* x, const void* bias,
               void* y, int m, int n, int K, int M, int x_dtype, int y_dtype, int nsplit, void* workspace,
               size_t workspace_bytes, void* stream) {
  if (!qweight || !scales || !su || !sv || !x || !y) return HTR_ERR_NULL;
  if (K < 2 || K > 8) return HTR_ERR_K;
  if (!shape_ok(m, n)) return HTR_ERR_SHAPE;
  if (M < 1 || M > HTR_MAX_BATCH) return HTR_ERR_BATCH;
  if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return HTR_ERR_DTYPE;
  if (((uintptr_t)qweight & 15) || ((uintptr_t)scales & 1) || ((uintptr_t)x & (x_dtype == HTR_F32 ? 3 : 1)) ||
      ((uintptr_t)y & (y_dtype == HTR_F32 ? 3 : 1)) || (bias && ((uintptr_t)bias & (y_dtype == HTR_F32 ? 3 : 1))))
    return HTR_ERR_ALIGN;
  if (wants_gemm(M, nsplit)) {
    GemmPlan gp;
    if (!make_gemm_plan(m, n, M, nsplit > 0 ? nsplit & 0xFFFFF : 0, gemm_want_jb(nsplit), gp)) return HTR_ERR_SPLIT;
    const size_t need = htr_workspace_bytes(m, n, K, M, nsplit);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return HTR_ERR_WORKSPACE;
    unsigned char* wsp = (unsigned char*)workspace + ws_half(workspace_bytes);
    LinearTail t;
    t.scales = (const uint16_t*)scales; t.sv = (const uint8_t*)sv; t.bias = bias; t.y = y;
    t.xt_g = (const _Float16*)wsp;
    t.xs_g = (const float*)(wsp + align256((size_t)M * n * 2));
    t.sc_g = (const float*)(wsp + align256((size_t)M * n * 2) + align256((size_t)M * (n / 128) * 16));
    t.tiles = (float*)(wsp + prerot_bytes(n, M));
    t.status = (uint32_t*)workspace;
    t.cbscale = htr_cbscale();
    t.spin_limit = g_spin_limit.load(std::memory_order_relaxed);
    t.chunk_magic = 0;
    t.group = nullptr; t.group_prerot_stride = 0; t.group_part_stride = 0;
    hipStream_t st = (hipStream_t)stream;
    HTR_CHECK_HIP(launch_rotation(x, (const uint8_t*)su, n, M, x_dtype, t, st));
    const uint32_t* qwp = (const uint32_t*)qweight;
    float* flags = (float*)((unsigned char*)workspace + WS_HEADER);
    const int flg = x_dtype | (y_dtype << 2);
#define HTR_LAUNCH_GEMM(KK_, PP_)                                                                                          \
    {                                                                                                                      \
      if (gp.jb == 3) {                                                                                                    \
        HTR_CHECK_HIP((allow_full_lds<k_linear_gemm<KK_, PP_, 3>>()));                                                     \
        HTR_CHECK_HIP(launch_kernel(k_linear_gemm<KK_, PP_, 3>, dim3(gp.S, m / 128, gp.mtiles), dim3(GEMM_THREADS),        \
                                    gemm_lds_bytes(3), st, qwp, flags, m, n, M, gp.S, flg, t));                            \
      } else {                                                                                                             \
        HTR_CHECK_HIP((allow_full_lds<k_linear_gemm<KK_, 2, 4>>()));                                                       \
        HTR_CHECK_HIP(launch_kernel(k_linear_gemm<KK_, 2, 4>, dim3(gp.S, m / 128, gp.mtiles), dim3(GEMM_THREADS),          \
                                    gemm_lds_bytes(4), st, qwp, flags, m, n, M, gp.S, flg, t));                            \
      }                                                                                                                    \
    }
    switch (K) {
      case 2: HTR_LAUNCH_GEMM(2, 4); break;
      case 3: HTR_LAUNCH_GEMM(3, 4); break;
      case 4: HTR_LAUNCH_GEMM(4, 4); break;
      case 5: HTR_LAUNCH_GEMM(5, 2); break;
      case 6: HTR_LAUNCH_GEMM(6, 2); break;
      case 7: HTR_LAUNCH_GEMM(7, 2); break;
      default: HTR_LAUNCH_GEMM(8, 2); break;
    }
#undef HTR_LAUNCH_GEMM
    return HTR_OK;
  }
  if (M > HTR_MAX_ROWS_PER_TILE) return HTR_ERR_BATCH;        // explicit plans of the other kernels take up to 128 rows
  if (wants_batch(M, nsplit, m, n)) {
    BatchPlan bp;
    if (!make_batch_plan(m, n, M, nsplit > 0 ? nsplit & 0xFFFFF : 0, bp)) return HTR_ERR_SPLIT;
    const size_t need = htr_workspace_bytes(m, n, K, M, nsplit);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return HTR_ERR_WORKSPACE;
    unsigned char* wsp = (unsigned char*)workspace + ws_half(workspace_bytes);
    LinearTail t;
    t.scales = (const uint16_t*)scales; t.sv = (const uint8_t*)sv; t.bias = bias; t.y = y;
    t.xt_g = (const _Float16*)wsp;
    t.xs_g = (const float*)(wsp + align256((size_t)M * n * 2));
    t.sc_g = (const float*)(wsp + align256((size_t)M * n * 2) + align256((size_t)M * (n / 128) * 16));
    t.status = (uint32_t*)workspace;
    t.cbscale = htr_cbscale();
    t.spin_limit = g_spin_limit.load(std::memory_order_relaxed);
    t.chunk_magic = 0;
    t.group = nullptr; t.group_prerot_stride = 0; t.group_part_stride = 0; t.tiles = nullptr;
    hipStream_t st = (hipStream_t)stream;
    // the workgroups rotate their own activations where the plan allows it (16-bit rows on 16-byte boundaries)
    const bool rot = bp.rot && x_dtype != HTR_F32 && ((uintptr_t)x & 15) == 0;
    if (!rot) HTR_CHECK_HIP(launch_rotation(x, (const uint8_t*)su, n, M, x_dtype, t, st));
    BatchArgs ba;
    ba.qw = (const uint32_t*)qweight; ba.part = (float*)((unsigned char*)workspace + WS_HEADER); ba.x = x; ba.su = (const uint8_t*)su;
    ba.m = m; ba.n = n; ba.M = M; ba.flags = x_dtype | (y_dtype << 2) | (bp.last_finishes ? FLAG_LAST_FINISHES : 0);
    if (bp.rot && !rot) bp.lds = batch_lds_bytes(M);            // the staged kernel's layout
    HTR_FOR_K(K, return launch_batch_k<KK>(ba, rot, t, bp, st));
    return HTR_OK;
  }
  if (M > HTR_MAX_GROUP_ROWS) return HTR_ERR_BATCH;          // an explicit chunked plan: that kernel takes up to 32 rows
  Plan pl;
  if (!make_plan(m, n, M, nsplit, pl)) return HTR_ERR_SPLIT;
  // the in-kernel rotation reads 16-bit elements in pairs: float32 activations, and rows that do not start on a
  // 4-byte boundary, take the pre-rotation
  const bool prerot = pl.prerot || x_dtype == HTR_F32 || ((uintptr_t)x & 3);
  const size_t need = htr_workspace_bytes(m, n, K, M, nsplit);
  if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return HTR_ERR_WORKSPACE;

  unsigned char* wsp = (unsigned char*)workspace + ws_half(workspace_bytes);      // scratch half
  LinearLaunch a;
  a.qw = (const uint32_t*)qweight; a.x = x; a.su = (const uint8_t*)su;
  a.part = (float*)((unsigned char*)workspace + WS_HEADER);
  a.m = m; a.n = n; a.M = M; a.chunk = pl.chunk; a.flags = x_dtype | (y_dtype << 2); a.problems = 1;
  // Eight lanes of whole row blocks, one per XCD: possible when the chunks tile the rows of column blocks and the row
  // blocks divide by eight.  Measured on MI355X (K4, batch 1): -0.2 us on 4096x4096, -0.3 us on 4096x14336 (eight chunks
  // per row block), no change with two chunks per row block, +0.1 us with a single row block per lane (1024x4096),
  // hence the lower bound of two row blocks per lane.  HTR_LANES=0 switches it off.
  {
    static const bool lanes_on = getenv("HTR_LANES") == nullptr || atoi(getenv("HTR_LANES")) != 0;
    const int nblk = n / 128, rbs = m / 128;
    if (lanes_on && pl.chunk < nblk && nblk % pl.chunk == 0 && rbs % 8 == 0 && rbs >= 16 && pl.wgs % 8 == 0) a.flags |= FLAG_LANES | ((pl.wgs / 8) << FLAG_LANE_LEN_SHIFT);
  }
  a.nblk_magic = (((unsigned long long)1 << 40) + (unsigned)(n / 128) - 1) / (unsigned)(n / 128);
  LinearTail& t = a.tail;
  t.scales = (const uint16_t*)scales; t.sv = (const uint8_t*)sv; t.bias = bias; t.y = y;
  t.xt_g = nullptr; t.xs_g = nullptr; t.sc_g = nullptr;
  t.status = (uint32_t*)workspace;
  t.cbscale = htr_cbscale();
  t.spin_limit = g_spin_limit.load(std::memory_order_relaxed);
  t.group = nullptr; t.group_prerot_stride = 0; t.group_part_stride = 0; t.tiles = nullptr;
  t.chunk_magic = (((unsigned long long)1 << 40) + (unsigned)pl.chunk - 1) / (unsigned)pl.chunk;
  hipStream_t st = (hipStream_t)stream;
  if (prerot) {
    t.xt_g = (const _Float16*)wsp;
    t.xs_g = (const float*)(wsp + align256((size_t)M * n * 2));
    t.sc_g = (const float*)(wsp + align256((size_t)M * n * 2) + align256((size_t)M * (n / 128) * 16));
    HTR_CHECK_HIP(launch_rotation(x, (const uint8_t*)su, n, M, x_dtype, t, st));
  }
  HTR_FOR_K(K, return launch_linear_k<KK>(a, prerot, pl.mb, pl.wgs, pl.lds, st));
  return HTR_OK;
}

// ---- htr_linear for callers that can neither allocate nor bring a workspace: the workspace is an array in the
// library's own device image.  Host code only ever holds the address hipGetSymbolAddress returns for it on the current
// device (every device has its own copy of the array at its own address; the symbol's name itself is no device address).
static __device__ __align__(256) unsigned char scratch[HTR_STATIC_SCRATCH_BYTES];

namespace {
void* g_scratch_ptr[MAX_DEVICES];                 // per device: address of `scratch` there, once looked up
std::atomic<uint64_t> g_scratch_known{0};         // bit d: g_scratch_ptr[d] is valid
}

int htr_linear_static(const void* qweight, const void* scales, const void* su, const void* sv, const void* x, const void* bias,
                      void* y, int m, int n, int K, int M, int x_dtype, int y_dtype, int reset, void* stream) {
  if (K < 2 || K > 8) return HTR_ERR_K;
  if (!shape_ok(m, n)) return HTR_ERR_SHAPE;
  if (M < 1 || M > HTR_MAX_BATCH) return HTR_ERR_BATCH;
  const size_t need = htr_workspace_bytes(m, n, K, M, 0);
  if (need == 0 || need > (size_t)HTR_STATIC_SCRATCH_BYTES) return HTR_ERR_WORKSPACE;      // beyond the built-in workspace
  int dev = 0;
  HTR_CHECK_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= MAX_DEVICES) { g_last_hip_error = (int)hipErrorInvalidDevice; return HTR_ERR_LAUNCH; }
  const uint64_t bit = (uint64_t)1 << dev;
  if (!(g_scratch_known.load(std::memory_order_acquire) & bit)) {
    void* p = nullptr;
    HTR_CHECK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    g_scratch_ptr[dev] = p;                       // two threads racing here store the same address
    g_scratch_known.fetch_or(bit, std::memory_order_release);
  }
  void* ws = g_scratch_ptr[dev];
  if (reset) {
    const int rc = htr_workspace_init(ws, HTR_STATIC_SCRATCH_BYTES, nullptr, stream);
    if (rc != HTR_OK) return rc;
  }
  return htr_linear(qweight, scales, su, sv, x, bias, y, m, n, K, M, x_dtype, y_dtype, 0, ws, HTR_STATIC_SCRATCH_BYTES, stream);
}

// plan of a grouped launch: every problem has the same shape, so one plan serves all; the activations are always
// rotated ahead (one launch for all problems) and the chunk is chosen for the whole grid
static bool make_group_plan(int count, int m, int n, int max_M, Plan& pl) {
  const int nblk = n / 128, rbs = m / 128;
  const long vtotal = (long)rbs * nblk;
  pl.mb = max_M <= 8 ? 1 : (max_M <= 16 ? 2 : 4);
  // aim at a few workgroups per CU over all problems; chunks are whole rows of column blocks or divide one, so that
  // no chunk straddles a row block; of those the one nearest the target (in ratio) that fits LDS
  static const int per_cu = getenv("HTR_GROUP_WGS_PER_CU") ? atoi(getenv("HTR_GROUP_WGS_PER_CU")) : 4;
  const double target = (double)vtotal * count / ((double)(per_cu > 0 ? per_cu : 4) * num_cu());
  double best = 1e30;
  bool found = false;
  for (long chunk = 1; chunk <= vtotal && chunk <= MAX_CHUNK; ++chunk) {
    if (chunk < nblk ? nblk % chunk != 0 : chunk % nblk != 0) continue;
    Plan c;
    c.mb = pl.mb;
    if (!plan_for_chunk(m, n, max_M, (int)chunk, c)) continue;
    const double ratio = chunk > target ? chunk / target : target / chunk;
    if (ratio < best) { best = ratio; pl = c; found = true; }
  }
  pl.prerot = 1;
  return found;
}

size_t htr_grouped_workspace_bytes(int count, int m, int n, int K, int max_M) {
  if (K < 2 || K > 8 || !shape_ok(m, n) || max_M < 1 || max_M > HTR_MAX_GROUP_ROWS || count < 1 || count > HTR_MAX_GROUP) return 0;
  Plan pl;
  if (!make_group_plan(count, m, n, max_M, pl)) return 0;
  return ws_need((size_t)count * pl.wgs * max_M * 128 * sizeof(float), (size_t)count * prerot_bytes(n, max_M));
}

int htr_linear_grouped(const htr_group_entry* entries, int count, int m, int n, int K, int max_M, int x_dtype, int y_dtype,
                       void* workspace, size_t workspace_bytes, void* stream) {
  if (!entries) return HTR_ERR_NULL;
  if (count < 1 || count > HTR_MAX_GROUP) return HTR_ERR_COUNT;
  if (K < 2 || K > 8) return HTR_ERR_K;
  if (!shape_ok(m, n)) return HTR_ERR_SHAPE;
  if (max_M < 1 || max_M > HTR_MAX_GROUP_ROWS) return HTR_ERR_BATCH;
  if (!dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return HTR_ERR_DTYPE;
  if ((uintptr_t)entries & 7) return HTR_ERR_ALIGN;
  Plan pl;
  if (!make_group_plan(count, m, n, max_M, pl)) return HTR_ERR_SPLIT;
  const size_t need = htr_grouped_workspace_bytes(count, m, n, K, max_M);
  if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return HTR_ERR_WORKSPACE;

  unsigned char* wsp = (unsigned char*)workspace + ws_half(workspace_bytes);      // scratch half
  const size_t pre = prerot_bytes(n, max_M);
  LinearLaunch a;
  a.qw = nullptr; a.x = nullptr; a.su = nullptr;
  a.part = (float*)((unsigned char*)workspace + WS_HEADER);
  a.m = m; a.n = n; a.M = max_M; a.chunk = pl.chunk; a.flags = x_dtype | (y_dtype << 2); a.problems = count;
  a.nblk_magic = (((unsigned long long)1 << 40) + (unsigned)(n / 128) - 1) / (unsigned)(n / 128);
  LinearTail& t = a.tail;
  t.scales = nullptr; t.sv = nullptr; t.bias = nullptr; t.y = nullptr;
  t.xt_g = (const _Float16*)wsp;
  t.xs_g = (const float*)(wsp + align256((size_t)max_M * n * 2));
  t.sc_g = (const float*)(wsp + align256((size_t)max_M * n * 2) + align256((size_t)max_M * (n / 128) * 16));
  t.status = (uint32_t*)workspace;
  t.cbscale = htr_cbscale();
  t.spin_limit = g_spin_limit.load(std::memory_order_relaxed);
  t.chunk_magic = (((unsigned long long)1 << 40) + (unsigned)pl.chunk - 1) / (unsigned)pl.chunk;
  t.tiles = nullptr;
  t.group = entries; t.group_prerot_stride = pre; t.group_part_stride = (unsigned long long)pl.wgs * max_M * 128;
  hipStream_t st = (hipStream_t)stream;
  HTR_CHECK_HIP(launch_kernel(k_rotate, dim3((n / 128 + WG_WAVES - 1) / WG_WAVES, max_M, count), dim3(WG_THREADS), 0, st, (const void*)nullptr,
                              (const uint8_t*)nullptr, n, x_dtype, (_Float16*)t.xt_g, (float*)t.xs_g, (float*)t.sc_g, entries,
                              (unsigned long long)pre));
  HTR_FOR_K(K, return launch_linear_k<KK>(a, true, pl.mb, pl.wgs, pl.lds, st));
  return HTR_OK;
}

// ---- timing anchors (measurement only; see the kernels).  kind 1: htr_linear's launch for one bf16 / f16 row with the
// decode compiled out; kind 2: only the weight stream of that launch.  Same plan, grid and LDS request as htr_linear.
int htr_anchor_linear(int kind, const void* qweight, const void* scales, const void* su, const void* sv, const void* x, void* y,
                      int m, int n, int K, int x_dtype, int y_dtype, void* workspace, size_t workspace_bytes, void* stream) {
  if (!qweight || !scales || !su || !sv || !x || !y) return HTR_ERR_NULL;
  if (K != 4 || (kind != 1 && kind != 2)) return HTR_ERR_K;
  if (!shape_ok(m, n)) return HTR_ERR_SHAPE;
  if (x_dtype == HTR_F32 || !dtype_ok(x_dtype) || !dtype_ok(y_dtype)) return HTR_ERR_DTYPE;
  if (((uintptr_t)qweight & 15) || ((uintptr_t)x & 3)) return HTR_ERR_ALIGN;
  Plan pl;
  if (!make_plan(m, n, 1, 0, pl) || pl.prerot) return HTR_ERR_SPLIT;
  const size_t need = htr_workspace_bytes(m, n, K, 1, 0);
  if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 255)) return HTR_ERR_WORKSPACE;
  LinearLaunch a;
  a.qw = (const uint32_t*)qweight; a.x = x; a.su = (const uint8_t*)su;
  a.part = (float*)((unsigned char*)workspace + WS_HEADER);
  a.m = m; a.n = n; a.M = 1; a.chunk = pl.chunk; a.flags = x_dtype | (y_dtype << 2); a.problems = 1;
  const int nblk = n / 128, rbs = m / 128;
  if (pl.chunk < nblk && nblk % pl.chunk == 0 && rbs % 8 == 0 && rbs >= 16 && pl.wgs % 8 == 0) a.flags |= FLAG_LANES | ((pl.wgs / 8) << FLAG_LANE_LEN_SHIFT);
  a.nblk_magic = (((unsigned long long)1 << 40) + (unsigned)nblk - 1) / (unsigned)nblk;
  LinearTail& t = a.tail;
  t.scales = (const uint16_t*)scales; t.sv = (const uint8_t*)sv; t.bias = nullptr; t.y = y;
  t.xt_g = nullptr; t.xs_g = nullptr; t.sc_g = nullptr;
  t.status = (uint32_t*)workspace;
  t.cbscale = htr_cbscale();
  t.spin_limit = g_spin_limit.load(std::memory_order_relaxed);
  t.group = nullptr; t.group_prerot_stride = 0; t.group_part_stride = 0; t.tiles = nullptr;
  t.chunk_magic = (((unsigned long long)1 << 40) + (unsigned)pl.chunk - 1) / (unsigned)pl.chunk;
  hipStream_t st = (hipStream_t)stream;
  const size_t lds = balanced_lds_request(pl.lds, pl.wgs);
  if (kind == 2) {
    HTR_CHECK_HIP(launch_kernel(k_anchor_read<4, 4>, dim3(pl.wgs), dim3(WG_THREADS), lds, st, a.qw, m, n, a.chunk, a.flags, a.nblk_magic,
                                (uint32_t*)((unsigned char*)workspace + ws_half(workspace_bytes))));
    return HTR_OK;
  }
  if (pl.chunk <= 8) {
    HTR_CHECK_HIP((allow_full_lds<k_linear<4, 1, 4, 4, false, 1, 1>>()));
    HTR_CHECK_HIP(launch_kernel(k_linear<4, 1, 4, 4, false, 1, 1>, dim3(pl.wgs), dim3(WG_THREADS), lds, st, a.qw, a.x, a.su, a.part,
                                a.m, a.n, a.M, a.chunk, a.flags, a.nblk_magic, a.tail));
  } else {
    HTR_CHECK_HIP((allow_full_lds<k_linear<4, 1, 4, 2, false, 1, 1>>()));
    HTR_CHECK_HIP(launch_kernel(k_linear<4, 1, 4, 2, false, 1, 1>, dim3(pl.wgs), dim3(WG_THREADS), lds, st, a.qw, a.x, a.su, a.part,
                                a.m, a.n, a.M, a.chunk, a.flags, a.nblk_magic, a.tail));
  }
  return HTR_OK;
}

// The decode of one wave-step (2048 weights) on register data: `workgroups` workgroups of 8 waves, one per compute unit
// (two waves per SIMD, as in the batch-1 launches), `iters` wave-steps each; out_u64[2 * wave] = shader-clock cycles,
// out_u64[2 * wave + 1] = ticks of the 100 MHz reference clock over the loop.
int htr_anchor_decode(int K, int with_mfma, int iters, int workgroups, void* out_u64, void* stream) {
  if (!out_u64) return HTR_ERR_NULL;
  if (K < 2 || K > 5) return HTR_ERR_K;
  if (iters < 1 || workgroups < 1 || workgroups > 65536) return HTR_ERR_SHAPE;
  hipStream_t st = (hipStream_t)stream;
  const size_t lds = balanced_lds_request(1024, workgroups <= num_cu() ? num_cu() : workgroups);
#define HTR_LAUNCH_ANCHOR(KK_, MF_)                                                                                          \
  {                                                                                                                          \
    HTR_CHECK_HIP((allow_full_lds<k_anchor_decode<KK_, MF_>>()));                                                            \
    HTR_CHECK_HIP(launch_kernel(k_anchor_decode<KK_, MF_>, dim3(workgroups), dim3(WG_THREADS), lds, st, iters,               \
                                (unsigned long long*)out_u64, (float*)nullptr));                                             \
  }
  switch (K) {
    case 2: if (with_mfma) HTR_LAUNCH_ANCHOR(2, true) else HTR_LAUNCH_ANCHOR(2, false) break;
    case 3: if (with_mfma) HTR_LAUNCH_ANCHOR(3, true) else HTR_LAUNCH_ANCHOR(3, false) break;
    case 4: if (with_mfma) HTR_LAUNCH_ANCHOR(4, true) else HTR_LAUNCH_ANCHOR(4, false) break;
    default: if (with_mfma) HTR_LAUNCH_ANCHOR(5, true) else HTR_LAUNCH_ANCHOR(5, false) break;
  }
#undef HTR_LAUNCH_ANCHOR
  return HTR_OK;
}

size_t htr_viterbi_workspace_bytes(int64_t tiles, int T, int K) {
  if (tiles <= 0 || T < 1 || T > 256 || K < 2 || K > 8) return 0;
  return align256((size_t)tiles * (size_t)(T > 1 ? T - 1 : 1) * (65536u >> K));
}

int htr_viterbi(const void* x, const void* w, int64_t tiles, int T, int K, int tailbite, void* states_u16, void* workspace,
                size_t workspace_bytes, void* stream) {
  if (!x || !w || !states_u16) return HTR_ERR_NULL;
  if (K < 2 || K > 8) return HTR_ERR_K;
  if (tiles <= 0 || tiles > 0x7FFFFFFF || T < 1 || T > 256) return HTR_ERR_SHAPE;
  if (((uintptr_t)x & 3) || ((uintptr_t)w & 3) || ((uintptr_t)states_u16 & 1)) return HTR_ERR_ALIGN;
  const size_t need = htr_viterbi_workspace_bytes(tiles, T, K);
  if (!workspace || workspace_bytes < need) return HTR_ERR_WORKSPACE;
  hipStream_t st = (hipStream_t)stream;
  const double rms = __builtin_sqrt(MEAN_SQ);
#define HTR_LAUNCH_VIT(KK_)                                                                                              \
  {                                                                                                                      \
    const size_t lds = ((size_t)2 * VitCfg<KK_>::SJ + 2048 + 1024 + 512 + 64) * sizeof(float);                           \
    HTR_CHECK_HIP((allow_full_lds<k_viterbi<KK_>>()));                                                                   \
    HTR_CHECK_HIP(launch_kernel(k_viterbi<KK_>, dim3((unsigned)tiles), dim3(VitCfg<KK_>::THREADS), lds, st, (const float*)x, \
                                (const float*)w, T, tailbite ? 1 : 0, (uint8_t*)workspace, (uint16_t*)states_u16, rms)); \
  }
  switch (K) {
    case 2: HTR_LAUNCH_VIT(2); break;
    case 3: HTR_LAUNCH_VIT(3); break;
    case 4: HTR_LAUNCH_VIT(4); break;
    case 5: HTR_LAUNCH_VIT(5); break;
    case 6: HTR_LAUNCH_VIT(6); break;
    case 7: HTR_LAUNCH_VIT(7); break;
    default: HTR_LAUNCH_VIT(8); break;
  }
#undef HTR_LAUNCH_VIT
  return HTR_OK;
}

int htr_decode_raw(const void* qweight, void* out_i16, int64_t ntiles, int K, void* stream) {
  if (!qweight || !out_i16) return HTR_ERR_NULL;
  if (K < 2 || K > 8) return HTR_ERR_K;
  if (ntiles <= 0) return HTR_ERR_SHAPE;
  if (((uintptr_t)qweight & 15) || ((uintptr_t)out_i16 & 15)) return HTR_ERR_ALIGN;
  const int64_t blocks = (ntiles * 8 + 255) / 256;
  hipStream_t st = (hipStream_t)stream;
  HTR_FOR_K(K, HTR_CHECK_HIP(launch_kernel(k_decode_raw<KK>, dim3((unsigned)blocks), dim3(256), 0, st, (const uint32_t*)qweight,
                                           (int16_t*)out_i16, ntiles)));
  return HTR_OK;
}

int htr_dequant_w(const void* qweight, const void* scales, const void* su, const void* sv, void* out_bf16, int m, int n,
                  int K, void* stream) {
  if (!qweight || !scales || !su || !sv || !out_bf16) return HTR_ERR_NULL;
  if (K < 2 || K > 8) return HTR_ERR_K;
  if (m <= 0 || n <= 0 || m % 128 || n % 128 || m / 128 > 65535) return HTR_ERR_SHAPE;
  if (((uintptr_t)qweight & 15) || ((uintptr_t)out_bf16 & 3) || ((uintptr_t)scales & 1) || ((uintptr_t)sv & 3)) return HTR_ERR_ALIGN;
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid(n / 128, m / 128);
  const size_t lds = (size_t)128 * DQW_LD * sizeof(float);
  const float cb = htr_cbscale();
#define HTR_LAUNCH_DQW(KK_)                                                                                              \
  {                                                                                                                      \
    HTR_CHECK_HIP((allow_full_lds<k_dequant_w<KK_>>()));                                                                 \
    HTR_CHECK_HIP(launch_kernel(k_dequant_w<KK_>, grid, dim3(512), lds, st, (const uint32_t*)qweight, (const uint16_t*)scales, \
                                (const uint8_t*)su, (const uint8_t*)sv, (uint16_t*)out_bf16, n / 16, cb));               \
  }
  HTR_FOR_K(K, HTR_LAUNCH_DQW(KK));
#undef HTR_LAUNCH_DQW
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
  HTR_FOR_K(K, HTR_CHECK_HIP(launch_kernel(k_dequant_q<KK>, dim3((unsigned)blocks), dim3(256), 0, st, (const uint32_t*)qweight,
                                           (const uint16_t*)scales, (float*)out_f32, mt, nt, rms)));
  return HTR_OK;
}

}  // extern "C"
