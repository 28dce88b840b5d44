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
#include "decode.hpp"
#include "linear.hpp"
#include "linear_batch.hpp"
#include "linear_gemm.hpp"
#include "dequant.hpp"
#include "viterbi.hpp"
#include "anchors.hpp"
#include "plan.hpp"
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
