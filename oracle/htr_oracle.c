/*
 * CPU oracle for the HTR-W1 packed-linear path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a checker: it restates, in plain C, the decode algorithm that the
 * reference defines in docs/FORMAT.md and htr/wire.py, so that the gfx950 kernels can be
 * compared against it.  Nothing in the shipped package links, loads or calls it; only the
 * test-suite, the smoke check and the cpu_baseline leg of the benchmark do.
 *
 * Every function names the reference lines it follows.  All of them are pinned by
 * known-answer tests that do not come from this file (generator constants from the closed
 * form, the reference's own string bit-oracle construction, the sign byte 170, Hadamard
 * orthogonality, brute-force placement checks); none is "parity unpinned".
 *
 * Build: see oracle/Makefile (gcc -O2 -fopenmp -shared -fPIC).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define HTR_L 16
#define HTR_S 65536
#define GEN_A 0xDF6ADFu
#define GEN_B 0x34983u

/* ---- generator: htr/wire.py:10-13, docs/FORMAT.md:11 --------------------------------- */
int htr_o_gen_value(uint32_t s) {
  uint64_t wide = (uint64_t)s * (uint64_t)GEN_A + (uint64_t)GEN_B; /* int64 product ... */
  uint32_t x = (uint32_t)(wide & 0xFFFFFFFFull);                  /* ... & 0xFFFFFFFF     */
  return (int)((x & 0xFF) + ((x >> 8) & 0xFF) + ((x >> 16) & 0xFF) + ((x >> 24) & 0xFF)) - 510;
}

/* ---- codebook normalisation: htr/wire.py:19-30, docs/FORMAT.md:10,12 ----------------- */
/* mean of v^2 over all 65536 states.  The integer sum is < 2^53, so the float64 mean is
 * the same in every summation order.                                                    */
double htr_o_mean_sq(void) {
  uint64_t acc = 0;
  for (uint32_t s = 0; s < HTR_S; ++s) {
    int64_t v = htr_o_gen_value(s);
    acc += (uint64_t)(v * v);
  }
  return (double)acc / (double)HTR_S;
}
double htr_o_rms(void) { return sqrt(htr_o_mean_sq()); }
double htr_o_cbscale(void) { return 1.0 / htr_o_rms(); }      /* htr/wire.py:28-30 */
void htr_o_codebook_f32(float* cb /* [65536] */) {             /* htr/wire.py:19-25 */
  const double rms = htr_o_rms();
  for (uint32_t s = 0; s < HTR_S; ++s) cb[s] = (float)((double)htr_o_gen_value(s) / rms);
}

/* ---- stream bit access: docs/FORMAT.md:20, htr/wire.py:46-51 -------------------------- */
/* stream bit p lives in word p>>5 at bit 31-(p&31) (MSB first).                          */
static inline uint32_t stream_bit(const int32_t* words, int p) {
  return (((uint32_t)words[p >> 5]) >> (31 - (p & 31))) & 1u;
}

/* ---- literal state extraction: htr/wire.py:54-63, docs/FORMAT.md:19 ------------------- */
/* s_t = the 16 stream bits at positions ((t+1)K - 16 + j) mod 256K, j = 0..15, MSB first */
void htr_o_unpack_states_literal(const int32_t* words, int64_t B, int K, uint16_t* states) {
  const int NB = 256 * K;
  for (int64_t b = 0; b < B; ++b) {
    const int32_t* w = words + b * 8 * K;
    for (int t = 0; t < 256; ++t) {
      uint32_t s = 0;
      for (int j = 0; j < 16; ++j) {
        int p = ((t + 1) * K - 16 + j) % NB;
        if (p < 0) p += NB;
        s = (s << 1) | stream_bit(w, p);
      }
      states[b * 256 + t] = (uint16_t)s;
    }
  }
}

/* ---- recurrence form: docs/FORMAT.md:16-17 -------------------------------------------- */
/* s_t = ((s_{t-1} << K) & 0xFFFF) | b_t with tail-biting start s_{-1} = s_255.  s_255 is
 * the last 16 bits of the stream (K*256 >= 16 always), so the walk can start there.      */
static void unpack_tile_recurrence(const int32_t* w, int K, uint16_t* st) {
  const int NB = 256 * K;
  uint32_t s = 0;
  for (int j = 0; j < 16; ++j) s = (s << 1) | stream_bit(w, NB - 16 + j);
  int p = 0;
  for (int t = 0; t < 256; ++t) {
    uint32_t b = 0;
    for (int k = 0; k < K; ++k) b = (b << 1) | stream_bit(w, p++);
    s = ((s << K) & 0xFFFFu) | b;
    st[t] = (uint16_t)s;
  }
}
void htr_o_unpack_states(const int32_t* words, int64_t B, int K, uint16_t* states) {
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < B; ++b) unpack_tile_recurrence(words + b * 8 * K, K, states + b * 256);
}

/* ---- pack: htr/wire.py:33-43 ---------------------------------------------------------- */
void htr_o_pack_states(const uint16_t* states, int64_t B, int K, int32_t* words) {
  for (int64_t b = 0; b < B; ++b) {
    uint32_t* w = (uint32_t*)(words + b * 8 * K);
    memset(w, 0, (size_t)(8 * K) * 4);
    int p = 0;
    for (int t = 0; t < 256; ++t) {
      uint32_t nb = states[b * 256 + t] & ((1u << K) - 1u);
      for (int k = K - 1; k >= 0; --k, ++p)
        if ((nb >> k) & 1u) w[p >> 5] |= 1u << (31 - (p & 31));
    }
  }
}

/* ---- signs: htr/wire.py:66-74, docs/FORMAT.md:28-29 ----------------------------------- */
void htr_o_unpack_signs(const uint8_t* u8, int64_t N, float* out) {
  for (int64_t j = 0; j < N; ++j) out[j] = ((u8[j >> 3] >> (j & 7)) & 1) ? -1.0f : 1.0f;
}
void htr_o_pack_signs(const float* s, int64_t N, uint8_t* u8) {
  memset(u8, 0, (size_t)(N / 8));
  for (int64_t j = 0; j < N; ++j)
    if (s[j] < 0) u8[j >> 3] |= (uint8_t)(1u << (j & 7));
}

/* ---- H128: htr/wire.py:80-87 (Sylvester, float64 / sqrt(n), cast to float32) ---------- */
void htr_o_hadamard(int n, float* H /* [n,n] */) {
  /* Sylvester doubling [[h,h],[h,-h]] has the closed form sign = parity(popcount(i & j)) */
  const double inv = 1.0 / sqrt((double)n);
  for (int i = 0; i < n; ++i)
    for (int j = 0; j < n; ++j)
      H[i * n + j] = (float)((__builtin_popcount((unsigned)(i & j)) & 1) ? -inv : inv);
}

/* in-place unnormalised fast Walsh-Hadamard on 128 doubles (same matrix as above x sqrt) */
static void fwht128_f64(double* v) {
  for (int h = 1; h < 128; h <<= 1)
    for (int i = 0; i < 128; i += h << 1)
      for (int j = i; j < i + h; ++j) {
        double a = v[j], b = v[j + h];
        v[j] = a + b;
        v[j + h] = a - b;
      }
}

/* ---- IEEE binary16 / bfloat16 -> float32 ---------------------------------------------- */
float htr_o_half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 0x1F, m = h & 0x3FF, bits;
  if (e == 0) {
    if (m == 0) bits = sign;
    else {
      int sh = 0;
      while (!(m & 0x400)) { m <<= 1; ++sh; }
      bits = sign | ((uint32_t)(113 - sh) << 23) | ((m & 0x3FF) << 13);
    }
  } else if (e == 31) bits = sign | 0x7F800000u | (m << 13);
  else bits = sign | ((e + 112) << 23) | (m << 13);
  float f;
  memcpy(&f, &bits, 4);
  return f;
}
static inline float bf16_to_float(uint16_t b) {
  uint32_t bits = (uint32_t)b << 16;
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* ---- integer decode, tile order: the value the GPU debug entry returns ---------------- */
/* out[tile, t] = v(s_t); follows htr/wire.py:99 (states) then :10-13 (values)            */
void htr_o_decode_raw(const int32_t* qw, int64_t ntiles, int K, int16_t* out) {
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < ntiles; ++b) {
    uint16_t st[256];
    unpack_tile_recurrence(qw + b * 8 * K, K, st);
    for (int t = 0; t < 256; ++t) out[b * 256 + t] = (int16_t)htr_o_gen_value(st[t]);
  }
}

/* ---- rotated-domain Q: htr/wire.py:95-102, docs/FORMAT.md:9,16 ------------------------ */
/* Q[16ti+r, 16tj+c] = cb[s_{ti,tj,16r+c}] * float32(scales[16ti+r])  (one f32 multiply)  */
void htr_o_dequant_q(const int32_t* qw, const uint16_t* scales_f16, int mt, int nt, int K, float* Q) {
  float* cb = (float*)malloc(sizeof(float) * HTR_S);
  htr_o_codebook_f32(cb);
  const int64_t n = (int64_t)nt * 16;
#pragma omp parallel for schedule(static)
  for (int ti = 0; ti < mt; ++ti) {
    uint16_t st[256];
    for (int tj = 0; tj < nt; ++tj) {
      unpack_tile_recurrence(qw + ((int64_t)ti * nt + tj) * 8 * K, K, st);
      for (int r = 0; r < 16; ++r) {
        const float sc = htr_o_half_to_float(scales_f16[ti * 16 + r]);
        float* row = Q + ((int64_t)ti * 16 + r) * n + (int64_t)tj * 16;
        for (int c = 0; c < 16; ++c) row[c] = cb[st[16 * r + c]] * sc;
      }
    }
  }
  free(cb);
}

/* integer v placed as a matrix [m, n] (same placement as Q) */
void htr_o_decode_v_matrix(const int32_t* qw, int mt, int nt, int K, int16_t* V) {
  const int64_t n = (int64_t)nt * 16;
#pragma omp parallel for schedule(static)
  for (int ti = 0; ti < mt; ++ti) {
    uint16_t st[256];
    for (int tj = 0; tj < nt; ++tj) {
      unpack_tile_recurrence(qw + ((int64_t)ti * nt + tj) * 8 * K, K, st);
      for (int r = 0; r < 16; ++r)
        for (int c = 0; c < 16; ++c)
          V[((int64_t)ti * 16 + r) * n + (int64_t)tj * 16 + c] = (int16_t)htr_o_gen_value(st[16 * r + c]);
    }
  }
}

/* ---- original-basis W: htr/wire.py:105-113, docs/FORMAT.md:7 -------------------------- */
/* W = Sv . Ho . Q . Hi . Su evaluated in float64 from the float32 Q (the reference does   */
/* the two block-Hadamard products as float32 matmuls whose summation order belongs to    */
/* the BLAS in use; float64 is the order-free statement of the same product).             */
void htr_o_dequant_w_f64(const int32_t* qw, const uint16_t* scales_f16, const uint8_t* su8, const uint8_t* sv8,
                         int mt, int nt, int K, double* W) {
  const int64_t m = (int64_t)mt * 16, n = (int64_t)nt * 16;
  float* Q = (float*)malloc(sizeof(float) * (size_t)(m * n));
  htr_o_dequant_q(qw, scales_f16, mt, nt, K, Q);
  const double inv = 1.0 / sqrt(128.0);
  /* rows: W <- Q . Hi (htr/wire.py:112) */
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < m; ++i) {
    double v[128];
    for (int64_t jb = 0; jb < n; jb += 128) {
      for (int j = 0; j < 128; ++j) v[j] = (double)Q[i * n + jb + j];
      fwht128_f64(v);
      for (int j = 0; j < 128; ++j) W[i * n + jb + j] = v[j] * inv;
    }
  }
  /* columns: W <- Ho . W (htr/wire.py:111), then signs (htr/wire.py:113) */
#pragma omp parallel for schedule(static)
  for (int64_t j = 0; j < n; ++j) {
    double v[128];
    const double suj = ((su8[j >> 3] >> (j & 7)) & 1) ? -1.0 : 1.0;
    for (int64_t ib = 0; ib < m; ib += 128) {
      for (int i = 0; i < 128; ++i) v[i] = W[(ib + i) * n + j];
      fwht128_f64(v);
      for (int i = 0; i < 128; ++i) {
        const int64_t r = ib + i;
        const double svr = ((sv8[r >> 3] >> (r & 7)) & 1) ? -1.0 : 1.0;
        W[r * n + j] = v[i] * inv * svr * suj;
      }
    }
  }
  free(Q);
}

/* ---- decode-then-matmul, factorised: docs/FORMAT.md:8 --------------------------------- */
/* y = sv . Ho( Q . Hi(su . x) ) (+ bias), float64 throughout from float32 Q and x.        */
/* x is given as bf16 bit patterns [M, n]; y as float64 [M, m].                            */
void htr_o_linear_f64(const int32_t* qw, const uint16_t* scales_f16, const uint8_t* su8, const uint8_t* sv8,
                      int mt, int nt, int K, const float* x, int M, const double* bias, double* y) {
  const int64_t m = (int64_t)mt * 16, n = (int64_t)nt * 16;
  const double inv = 1.0 / sqrt(128.0);
  double* xt = (double*)malloc(sizeof(double) * (size_t)(M * n));
  for (int r = 0; r < M; ++r)
    for (int64_t jb = 0; jb < n; jb += 128) {
      double v[128];
      for (int j = 0; j < 128; ++j) {
        const int64_t c = jb + j;
        v[j] = (((su8[c >> 3] >> (c & 7)) & 1) ? -1.0 : 1.0) * (double)x[r * n + c];
      }
      fwht128_f64(v);
      for (int j = 0; j < 128; ++j) xt[r * n + jb + j] = v[j] * inv;
    }
  float* cb = (float*)malloc(sizeof(float) * HTR_S);
  htr_o_codebook_f32(cb);
  double* yt = (double*)calloc((size_t)(M * m), sizeof(double));
#pragma omp parallel for schedule(static)
  for (int ti = 0; ti < mt; ++ti) {
    uint16_t st[256];
    for (int tj = 0; tj < nt; ++tj) {
      unpack_tile_recurrence(qw + ((int64_t)ti * nt + tj) * 8 * K, K, st);
      for (int r16 = 0; r16 < 16; ++r16) {
        const float sc = htr_o_half_to_float(scales_f16[ti * 16 + r16]);
        float q[16];
        for (int c = 0; c < 16; ++c) q[c] = cb[st[16 * r16 + c]] * sc; /* Q as the reference's float32 */
        for (int r = 0; r < M; ++r) {
          double acc = 0.0;
          const double* xr = xt + r * n + (int64_t)tj * 16;
          for (int c = 0; c < 16; ++c) acc += (double)q[c] * xr[c];
          yt[r * m + ti * 16 + r16] += acc;
        }
      }
    }
  }
  for (int r = 0; r < M; ++r)
    for (int64_t ib = 0; ib < m; ib += 128) {
      double v[128];
      for (int i = 0; i < 128; ++i) v[i] = yt[r * m + ib + i];
      fwht128_f64(v);
      for (int i = 0; i < 128; ++i) {
        const int64_t o = ib + i;
        double val = v[i] * inv * (((sv8[o >> 3] >> (o & 7)) & 1) ? -1.0 : 1.0);
        if (bias) val += bias[o];
        y[r * m + o] = val;
      }
    }
  free(yt);
  free(cb);
  free(xt);
}

/* ---- the CPU baseline shape: decode the full float32 W, then x @ W^T in float32 ------- */
/* "reference-shaped": htr/wire.py:105-113 followed by a plain matmul.  W is produced in  */
/* float32 with float32 butterflies (fast WHT instead of the dense 128x128 matmul).       */
static void fwht128_f32(float* v) {
  for (int h = 1; h < 128; h <<= 1)
    for (int i = 0; i < 128; i += h << 1)
      for (int j = i; j < i + h; ++j) {
        float a = v[j], b = v[j + h];
        v[j] = a + b;
        v[j + h] = a - b;
      }
}
void htr_o_dequant_w_f32(const int32_t* qw, const uint16_t* scales_f16, const uint8_t* su8, const uint8_t* sv8,
                         int mt, int nt, int K, float* W) {
  const int64_t m = (int64_t)mt * 16, n = (int64_t)nt * 16;
  const float inv = 0.08838834764831845f; /* 1/sqrt(128) */
  htr_o_dequant_q(qw, scales_f16, mt, nt, K, W);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < m; ++i)
    for (int64_t jb = 0; jb < n; jb += 128) {
      float* v = W + i * n + jb;
      fwht128_f32(v);
      for (int j = 0; j < 128; ++j) v[j] *= inv;
    }
#pragma omp parallel for schedule(static)
  for (int64_t ib = 0; ib < m; ib += 128) {
    float* col = (float*)malloc(sizeof(float) * 128);
    for (int64_t j = 0; j < n; ++j) {
      const float suj = ((su8[j >> 3] >> (j & 7)) & 1) ? -1.0f : 1.0f;
      for (int i = 0; i < 128; ++i) col[i] = W[(ib + i) * n + j];
      fwht128_f32(col);
      for (int i = 0; i < 128; ++i) {
        const int64_t r = ib + i;
        const float svr = ((sv8[r >> 3] >> (r & 7)) & 1) ? -1.0f : 1.0f;
        W[r * n + j] = col[i] * inv * svr * suj;
      }
    }
    free(col);
  }
}
void htr_o_matmul_xwT_f32(const float* x, const float* W, int M, int64_t m, int64_t n, float* y) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < m; ++i)
    for (int r = 0; r < M; ++r) {
      float acc = 0.f;
      const float* wr = W + i * n;
      const float* xr = x + (int64_t)r * n;
      for (int64_t j = 0; j < n; ++j) acc += wr[j] * xr[j];
      y[(int64_t)r * m + i] = acc;
    }
}

void htr_o_bf16_to_f32(const uint16_t* in, int64_t N, float* out) {
  for (int64_t i = 0; i < N; ++i) out[i] = bf16_to_float(in[i]);
}

int htr_o_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
void htr_o_set_num_threads(int t) {
#ifdef _OPENMP
  omp_set_num_threads(t);
#else
  (void)t;
#endif
}

/* ------------------------------------------------------------------------------------------------ encoder search
 * Batched bitshift-trellis Viterbi, restated from htr/reference.py:6-50 of the reference: minimises
 * sum_t w[t] * (x[t] - cb[s_t])^2 over state sequences with s_t = ((s_{t-1} << K) & mask) | bits, L-bit states
 * (L = 16 in the codec; smaller L exists so that tests can compare with an exhaustive search).  Two passes when
 * tailbite: the first fixes j0 = argmin(final cost) & (Sj - 1); the second admits at t = 0 only the states whose
 * upper part is j0 and at the end only the states whose lower part is j0, which makes the stream circular.
 * Arithmetic is float32 in the reference's order: d = (x - cb)^2, cost = m + w * d; every min / argmin takes the
 * FIRST index among equal values (htr/reference.py:29, 37, 41).  states: [B, T] uint32.  Returns 0, or -1 on
 * allocation failure. */
static int viterbi_pass(const float* x, const float* w, const float* cb, int L, int K, int T, int use_j0, uint32_t j0,
                        float* cost, float* m, uint8_t* bps) {
  const uint32_t S = 1u << L, nb = 1u << K, Sj = S >> K;
  for (uint32_t s = 0; s < S; ++s) {                                   /* htr/reference.py:22-27 */
    const float diff = x[0] - cb[s];
    const float d0 = w[0] * (diff * diff);
    cost[s] = (use_j0 && (s >> K) != j0) ? INFINITY : d0;
  }
  for (int t = 1; t < T; ++t) {                                        /* htr/reference.py:29-33 */
    for (uint32_t low = 0; low < Sj; ++low) {
      float best = cost[low];
      uint32_t bi = 0;
      for (uint32_t j = 1; j < nb; ++j) {
        const float c = cost[j * Sj + low];
        if (c < best) { best = c; bi = j; }
      }
      m[low] = best;
      bps[(size_t)(t - 1) * Sj + low] = (uint8_t)bi;
    }
    for (uint32_t low = 0; low < Sj; ++low)
      for (uint32_t b = 0; b < nb; ++b) {
        const uint32_t s = low * nb + b;
        const float diff = x[t] - cb[s];
        const float d = diff * diff;
        cost[s] = m[low] + w[t] * d;
      }
  }
  return 0;
}

int htr_o_viterbi(const float* x, const float* w, const float* cb, int L, int K, int T, int64_t B, int tailbite,
                  uint32_t* states) {
  const uint32_t S = 1u << L, Sj = S >> K;
  int fail = 0;
#pragma omp parallel for schedule(dynamic)
  for (int64_t b = 0; b < B; ++b) {
    float* cost = (float*)malloc(sizeof(float) * S);
    float* m = (float*)malloc(sizeof(float) * Sj);
    uint8_t* bps = (uint8_t*)malloc((size_t)(T > 1 ? T - 1 : 1) * Sj);
    if (!cost || !m || !bps) { fail = 1; free(cost); free(m); free(bps); continue; }
    const float* xb = x + b * T;
    const float* wb = w + b * T;
    viterbi_pass(xb, wb, cb, L, K, T, 0, 0, cost, m, bps);
    if (tailbite) {                                                    /* htr/reference.py:35-40 */
      uint32_t a = 0;
      for (uint32_t s = 1; s < S; ++s) if (cost[s] < cost[a]) a = s;
      const uint32_t j0 = a & (Sj - 1);
      viterbi_pass(xb, wb, cb, L, K, T, 1, j0, cost, m, bps);
      for (uint32_t s = 0; s < S; ++s) if ((s & (Sj - 1)) != j0) cost[s] = INFINITY;
    }
    uint32_t s = 0;                                                    /* htr/reference.py:41-49 */
    for (uint32_t q = 1; q < S; ++q) if (cost[q] < cost[s]) s = q;
    uint32_t* st = states + b * T;
    st[T - 1] = s;
    for (int t = T - 1; t > 0; --t) {
      const uint32_t low = s >> K;
      const uint32_t top = bps[(size_t)(t - 1) * Sj + low];
      s = top * Sj + low;
      st[t - 1] = s;
    }
    free(cost); free(m); free(bps);
  }
  return fail ? -1 : 0;
}
