// Part of htr_gfx950.hip, included inside its anonymous namespace: k_linear_batch: 9 to 128 activation rows.
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

