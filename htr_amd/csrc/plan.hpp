// Part of htr_gfx950.hip, included inside its anonymous namespace: workspace layout, launch plans and launchers (host side).
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

