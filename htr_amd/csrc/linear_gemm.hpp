// Part of htr_gfx950.hip, included inside its anonymous namespace: k_linear_gemm: 129 to 2048 activation rows in one launch.
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

