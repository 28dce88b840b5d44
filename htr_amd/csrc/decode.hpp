// Part of htr_gfx950.hip, included inside its anonymous namespace: constants, small helpers, stream loads and the trellis decode core.

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

