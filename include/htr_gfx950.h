/*
 * C ABI of libhtr_gfx950.so: the MI355X (gfx950) execution path for HTR-W1 packed linears.
 *
 * Plain pointers and sizes only.  All pointers except `problems` arrays are DEVICE pointers
 * on the current HIP device; `stream` is a hipStream_t passed as void* (NULL = default
 * stream).  Every call is asynchronous on `stream`, allocates nothing and never
 * synchronises.  Return value: 0 on success, otherwise an htr_status code whose text
 * htr_strerror() returns.
 *
 * Tensors use the HTR-W1 wire layout of the reference (docs/FORMAT.md:25-32):
 *   qweight int32 [m/16, n/16, 8K]  (uint32 bit patterns), K = 2..8
 *   scales  float16 [m]
 *   su      uint8 [n/8],  sv uint8 [m/8]   bit j%8 (LSB first) of byte j/8 set -> sign -1
 * m and n are multiples of 128.
 *
 * Each entry point names the reference interface it stands in for (paths relative to the
 * reference tree).
 */
#ifndef HTR_GFX950_H
#define HTR_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  HTR_OK = 0,
  HTR_ERR_NULL = 1,       /* a required pointer is NULL */
  HTR_ERR_K = 2,          /* K outside 2..8 */
  HTR_ERR_SHAPE = 3,      /* m or n not a positive multiple of 128 */
  HTR_ERR_BATCH = 4,      /* M outside 1..HTR_MAX_BATCH */
  HTR_ERR_DTYPE = 5,      /* dtype code not one of HTR_BF16/HTR_F16/HTR_F32 */
  HTR_ERR_WORKSPACE = 6,  /* workspace too small or misaligned */
  HTR_ERR_ALIGN = 7,      /* a tensor pointer is not aligned as required */
  HTR_ERR_LAUNCH = 8,     /* the HIP runtime refused the launch (see htr_last_hip_error) */
  HTR_ERR_SPLIT = 9,      /* explicit split count not usable for this shape */
  HTR_ERR_COUNT = 10      /* grouped call: count outside 1..HTR_MAX_GROUP */
} htr_status;

/* element type codes; same numbering as the reference's out-dtype map (htr/ops.py:79,94) */
enum { HTR_BF16 = 0, HTR_F16 = 1, HTR_F32 = 2 };

#define HTR_MAX_BATCH 2048      /* activation rows one htr_linear launch accepts */
#define HTR_MAX_ROWS_PER_TILE 128   /* up to here one workgroup holds all rows; beyond, the GEMM kernel works in tiles of 96 or 128 rows */
#define HTR_MAX_GROUP_ROWS 32   /* rows per problem of htr_linear_grouped (and of an explicit chunked plan, see nsplit) */
#define HTR_MAX_GROUP 4096 /* problems one htr_linear_grouped launch accepts */

const char* htr_strerror(int status);
/* hipError_t value of the last failed launch on this thread (0 if none) */
int htr_last_hip_error(void);
int htr_abi_version(void);

/* CBSCALE = 1/sqrt(mean_s v(s)^2) as the float32 the kernels multiply by.
 * Reference: wire.cbscale(), htr/wire.py:28-30 (used as ops.CB, htr/ops.py:7). */
float htr_cbscale(void);

/*
 * Bytes of zero-initialised device workspace htr_linear needs for this problem (a status
 * word, room for pre-rotated activations, one partial slot per workgroup).  The caller
 * allocates it once, zeroes it once, and may reuse it for any later call whose requirement
 * is not larger, as long as calls that share a workspace are ordered on one stream: kernels
 * leave the partial slots zero on exit.  The first 32-bit word stays zero unless a kernel
 * gave up waiting for a partial (see htr_set_spin_limit and htr_workspace_init for what follows).
 * Thread safety: calls from several host threads are safe as long as launches that share a
 * workspace are ordered on one stream.
 * The library splits the buffer at workspace_bytes / 2: the first half holds the status word and the
 * partial slots (the part that must be zero), the second half is scratch.  Pass the same
 * workspace_bytes whenever you pass the same buffer, so that the split stays where it was;
 * htr_linear and htr_linear_grouped may then share one buffer.
 * Reference: the per-device int32[65536] counter tensor (htr/ops.py:24-28) plus the
 * `part` tensors the extension allocates per call (htr/csrc/htr_kernels.cu:1145).
 * nsplit: as in htr_linear.
 */
size_t htr_workspace_bytes(int m, int n, int K, int M, int nsplit);

/*
 * Prepares (or clears) a workspace on `stream` with a fill kernel (no memset, so the call may be recorded into a HIP
 * graph): zeroes the half that must be zero, status word included, and stores `host_status_word` in bytes 8..15 of the
 * 256-byte header.  host_status_word is NULL or the address of a 4-byte word in pinned, device-visible host memory
 * (hipHostMalloc) that the caller has set to 0: a kernel that gives up waiting also stores 1 there, so the host can
 * notice the failure by reading its own memory, without a copy or a synchronisation.
 * Failure protocol: a launch that gives up marks its unfinished rows NaN and sets bit 0 of the status word (word 0 of
 * the workspace); the partials it did not collect stay in the slots.  From then on every launch on that workspace marks
 * ALL its outputs NaN, until the caller, after the stream has drained, calls htr_workspace_init again.
 * A caller that zeroes a fresh workspace itself (memset) and never registers a host word needs no call to this.
 * Reference: the zeroed per-device counter tensor of htr/ops.py:24-28 (which has no failure path: its kernels wait
 * without bound).
 */
int htr_workspace_init(void* workspace, size_t workspace_bytes, void* host_status_word, void* stream);

/*
 * 0 if `stream` is not being captured into a HIP graph, otherwise a non-zero id that is unique to the capture in
 * progress (hipStreamGetCaptureInfo).  Lets a host layer give every capture a workspace of its own, which must then
 * live as long as the graph.  Reference: none (torch.cuda.is_current_stream_capturing is the nearest).
 */
unsigned long long htr_stream_capture_id(void* stream);

/*
 * The launch plan htr_linear would use: out6 = {steps (128x128 weight blocks of one row block, walked row-major)
 * per workgroup, workgroups, row blocks that can end inside one workgroup's chunk, distinct column blocks per
 * workgroup, 1 if the activations are rotated by a launch of their own, dynamic LDS bytes}.  No reference counterpart
 * as a function; it exposes what nsplit_for / fused_nsplit decide there (htr/ops.py:31-45).
 * With 9 rows and more (6 and more for m >= 24576, 7 and more where a full grid has splits of at most four column blocks;
 * library policy) the batched kernel runs instead: out6 = {column blocks per split, workgroups (= row blocks x splits),
 * 1 if the splits of a row block finish rows for each other (only while the grid is at most one workgroup per compute
 * unit; 0: the last split finishes every row), splits per row block, 1 if the activations are rotated by a launch of their
 * own (0: the workgroups rotate their own slices: up to 16 rows over at most 16 column blocks per split, or up to 32 rows
 * over at most 8), dynamic LDS bytes}.  Entries 4 and 5 assume bf16 / f16 activations on a 16-byte boundary; float32 or
 * otherwise aligned activations always take the rotation launch and the staged kernel's LDS layout.
 * With more than HTR_MAX_ROWS_PER_TILE rows the fused decode -> matrix-unit (GEMM) kernel runs: the activations are
 * always rotated by a launch of their own, a workgroup owns one 128-row block of the weight, one tile of 96 or of 128
 * activation rows (the planner takes the height that saves a round of workgroups or allows more splits) and one of S
 * column splits, and the last split of a (row block, tile) adds up the others' partial tiles, which travel through
 * the workspace.  out6 = {column blocks per split, workgroups (= S x row blocks x row tiles), row tiles, S, 1, dynamic
 * LDS bytes}.  The reference has no such kernel: it dequantizes the weight and calls a library GEMM from
 * these row counts on (htr/ops.py:89-93), which stays the better choice from a few hundred rows.
 * Plans are made for the current device's compute-unit count and LDS size (an unpartitioned MI355X where no device can
 * be asked); see htr_plan_device_override.
 * nsplit: 0 = library policy; otherwise the steps per workgroup of the chunked kernel (1 .. HTR_MAX_GROUP_ROWS rows;
 * bit 30 set: force the separate rotation launch), or, with bit 29 set, the batched kernel with that many column
 * splits in the low bits (0 = its own policy; up to HTR_MAX_ROWS_PER_TILE rows), or, with bit 28 set, the GEMM kernel
 * with that many column splits in the low bits (0 = its own policy; at most 8; any row count up to HTR_MAX_BATCH) and
 * tiles of 96 (bit 20) or 128 (bit 21) activation rows (neither: its own policy).
 */
int htr_linear_plan(int m, int n, int K, int M, int nsplit, int* out6);

/*
 * Makes every later plan assume a device of `compute_units` compute units with `lds_bytes_per_cu` bytes of LDS each,
 * instead of what the runtime reports for the current device; compute_units = 0 returns to the device's own figures.
 * For tests of the planner and for tuning; the kernels themselves are correct for any plan the library hands out.
 * Reference: the environment override of the workgroup target, HTR_FUSED_WGS (htr/ops.py:44).
 */
int htr_plan_device_override(int compute_units, long lds_bytes_per_cu);

/*
 * y[M, m] = x[M, n] @ W^T (+ bias) for an HTR-W1 weight, one fused launch: input sign flip +
 * H128, trellis decode, row scale, fp32-accumulated product, output H128 + sign, bias, cast.
 * Reference: the decode branch of _linear_impl (htr/ops.py:75-76, :94-98), i.e.
 * prologue + gemv_epi / gemv_fused (htr/csrc/htr_kernels.cu:972-987, :1134-1173, :1034-1064).
 *   x      [M, n] row-major, x_dtype (bf16 / f16 / f32), 1 <= M <= HTR_MAX_BATCH
 *   bias   [m] in y_dtype, or NULL
 *   y      [M, m] row-major, y_dtype
 *   nsplit 0 = library policy; otherwise an explicit plan as in htr_linear_plan (tuning)
 *   x must be 4-byte aligned for the in-kernel rotation; other 2-byte aligned bf16/f16 rows take the rotation launch
 */
int htr_linear(const void* qweight, const void* scales, const void* su, const void* sv,
               const void* x, const void* bias, void* y,
               int m, int n, int K, int M, int x_dtype, int y_dtype, int nsplit,
               void* workspace, size_t workspace_bytes, void* stream);

/*
 * htr_linear on a workspace that is part of the library: for callers that cannot allocate device memory at the point
 * of the call and have no workspace to pass (code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation).  It has no counterpart in the reference.  The call allocates nothing, frees nothing and calls no
 * allocating routine; inputs and outputs are the caller's, as in htr_linear, and the launch policy is the library's
 * (nsplit = 0).  The workspace is an array of HTR_STATIC_SCRATCH_BYTES in the library's device image; every GPU the
 * library runs on holds its own copy until the process ends.
 * Limit: problems with htr_workspace_bytes(m, n, K, M, 0) > HTR_STATIC_SCRATCH_BYTES return HTR_ERR_WORKSPACE (all
 * decode shapes of up to 8 rows fit, 32 rows on 14336 x 4096 too; 64 rows there do not).
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different streams or graphs
 * running concurrently) race on it; order them on one stream.  The array starts zeroed and every launch leaves it as
 * it must be for the next one; after a launch that gave up waiting (NaN outputs, see htr_workspace_init) pass
 * reset != 0 once, with the stream drained: the call then clears the array with a fill kernel on `stream` first.
 * The first call on a device looks the array's address up there (hipGetSymbolAddress); make that call outside of
 * a graph capture.
 */
#define HTR_STATIC_SCRATCH_BYTES (8u << 20)
int htr_linear_static(const void* qweight, const void* scales, const void* su, const void* sv,
                      const void* x, const void* bias, void* y,
                      int m, int n, int K, int M, int x_dtype, int y_dtype, int reset, void* stream);

/*
 * One entry of a grouped launch: the HTR-W1 tensors, activations and output of one problem.  The table lives in
 * DEVICE memory (so that a routing kernel can fill it), is 8-byte aligned and is read by the kernels only.
 */
typedef struct {
  const void* qweight;
  const void* scales;
  const void* su;
  const void* sv;
  const void* x;      /* [M, n] row-major, 4-byte aligned */
  const void* bias;   /* [m] in the output type, or NULL */
  void* y;            /* [M, m] row-major */
  int32_t M;          /* activation rows of this problem, 0 .. max_M (0 = skip) */
  int32_t reserved;
} htr_group_entry;

/*
 * `count` packed linears of ONE shape (m, n, K) in two launches (activation rotation for all problems, then the fused
 * decode-product-epilogue for all problems): routed experts, whose per-expert launches would each pay the full launch
 * latency for a few microseconds of work.  No counterpart in the reference, which has no runtime kernel for routed
 * experts and composes them from per-expert linears (docs/ADAPTERS.md:19); the per-problem result is that of
 * htr_linear on the same tensors.  max_M bounds the rows of any problem (1 .. HTR_MAX_GROUP_ROWS).
 * Workspace: htr_grouped_workspace_bytes() bytes, zeroed once, same rules as for htr_linear.
 */
size_t htr_grouped_workspace_bytes(int count, int m, int n, int K, int max_M);
int htr_linear_grouped(const htr_group_entry* entries_device, int count, int m, int n, int K, int max_M,
                       int x_dtype, int y_dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Polls (about a microsecond each) a finishing workgroup waits for the partials of earlier workgroups before it gives
 * up, stores NaN for its rows and sets bit 0 of the first workspace word.  Default 2^20.  No counterpart in the
 * reference; exists so that the bounded wait can be exercised.
 */
void htr_set_spin_limit(int polls);

/*
 * Encoder search: tail-biting bitshift-trellis Viterbi over the 65536 codec states, one 256-weight tile per row.
 *   x, w      float32 [tiles, T] targets and per-element weights (T <= 256; the codec uses 256)
 *   states    uint16 [tiles, T]: s_t with s_t >> K == s_{t-1} & (2^(16-K) - 1), circular when tailbite != 0
 *   workspace htr_viterbi_workspace_bytes() bytes of device scratch (backpointers; no zero requirement)
 * K = 2..8.  Same result as the reference's portable search, htr.reference.viterbi(x, w, codebook_f32(), K)
 * (htr/reference.py:6-50), which its CUDA versions htr/vit_v1.py:46-110 and htr/vit_v2.py:100-162 also reproduce;
 * the state values are the procedural codebook, so no codebook tensor is passed.
 */
size_t htr_viterbi_workspace_bytes(int64_t tiles, int T, int K);
int htr_viterbi(const void* x, const void* w, int64_t tiles, int T, int K, int tailbite, void* states_u16,
                void* workspace, size_t workspace_bytes, void* stream);

/*
 * Integer decode, tile order: out[tile, t] = v(s_t) as int16, tile = ti*(n/16)+tj, t = 16r+c.
 * Reference: decode_raw (htr/csrc/htr_kernels.cu:943-951, kernel :154-172).
 */
int htr_decode_raw(const void* qweight, void* out_i16, int64_t ntiles, int K, void* stream);

/*
 * Rotated-domain Q[m, n] float32 = cb[s] * float32(scale_row), bit-exact with the
 * reference's CPU decoder.  Reference: wire.dequant_Q (htr/wire.py:95-102); the GPU
 * counterpart there is dequant_f16 (htr/csrc/htr_kernels.cu:932-941), which rounds to f16.
 */
int htr_dequant_q(const void* qweight, const void* scales, void* out_f32, int mt, int nt, int K, void* stream);

/*
 * Original-basis W[m, n] = Sv . Ho . Q . Hi . Su as bfloat16, row-major: the prefill path dequantizes once and hands W
 * to a library GEMM.  Reference: dequant_w (htr/csrc/htr_kernels.cu:1082-1095, kernels :657-903), used by
 * _linear_impl for M above the GEMV range (htr/ops.py:89-93); CPU definition wire.dequant (htr/wire.py:105-113).
 * out_bf16 and sv must be 4-byte aligned (bf16 pairs are stored, the sv bits of a row block are read as words).
 */
int htr_dequant_w(const void* qweight, const void* scales, const void* su, const void* sv, void* out_bf16,
                  int m, int n, int K, void* stream);

/*
 * Timing anchors: measurement only, the results they leave in y are meaningless.  No reference counterpart (the
 * reference reports its kernel's bandwidth without such anchors, docs/METHODOLOGY.md:87-90).
 * htr_anchor_linear: the launch htr_linear would make for ONE bf16 / f16 activation row of a K4 weight (same plan, grid
 * and LDS request), kind 1: with the trellis decode compiled out (stream, rotation, products, hand-over and output
 * side remain), kind 2: only the weight stream (the same descriptors, order and depth of loads, nothing else).
 * htr_anchor_decode: the decode of the inner loop on register data (K = 2..5), `workgroups` workgroups of 8 waves,
 * `iters` wave-steps (2048 weights each) per wave, with or without the four matrix instructions of a step;
 * out_u64[2 w] = shader-clock cycles and out_u64[2 w + 1] = ticks of the 100 MHz reference clock wave w spent in the loop.
 */
int htr_anchor_linear(int kind, const void* qweight, const void* scales, const void* su, const void* sv, const void* x,
                      void* y, int m, int n, int K, int x_dtype, int y_dtype, void* workspace, size_t workspace_bytes,
                      void* stream);
int htr_anchor_decode(int K, int with_mfma, int iters, int workgroups, void* out_u64, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* HTR_GFX950_H */
