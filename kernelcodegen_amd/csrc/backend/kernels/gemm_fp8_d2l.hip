// ---- fp8 (e4m3) GEMM on v_mfma_f32_16x16x128_f8f6f4, operand tiles straight from global memory into LDS --------
// C[b] = scale_a * scale_b * A[b] * B[b]: A is [M][K]; B is [N][K] (both contiguous along k) or, with G8_BTR, row-major
// [K][N]; fp8 e4m3, one fp32 scale per tensor, fp32 accumulate, fp32 or bf16 out.  Full 256 x 256 x 128 tiles only (the emitter falls back to
// gemm_fp8.hip for every other case).  Parameters:
//   G8_NAME                      kernel symbol
//   G8_M G8_N G8_K G8_BATCH      problem: multiples of 256, 256 and 128
//   G8_GROUP_M                   tile rows per L2 strip
//   G8_OUT_BF16                  1: C is bf16, else fp32
//   G8_RELU                      1: fused max(0, .) epilogue
//   G8_SCALE_PTR                 0: (A, B, C, float, float); 1: (A, B, C, const float*, const float*);
//                                2: (A, B, const float*, const float*, C)   -- as in gemm_fp8.hip
//   G8_BTR                       1: B is row-major [K][N]; its tiles lie in LDS as in memory and the MFMA fragments come
//                                from transposing LDS reads (see the loads and fragB)
//   G8_PERSIST                   1: the grid is one workgroup per compute unit; workgroup w works through the output tiles
//                                w, w + gridDim.x, ... as one stream of k-tiles (see "Persistent workgroups")
//   G8_NT_STORE                  1: fp32 results are stored with the non-temporal hint
//   G8_STAGE_C                   1: results are turned round in LDS and stored as whole rows of the tile (see the epilogue)
//   G8_STAGGER                   n > 0: the first round's workgroups start up to 31 n x 512 cycles apart (see below)
//
// Why this shape.  The part is power bound on 8-bit products, and v_mfma_f32_16x16x128 reads and writes the fp32
// accumulators half as often per result as v_mfma_f32_32x32x64: a register-only loop on random e4m3 operands sustains
// 4.8 against 4.0 PFLOP/s, 3.9 against 3.5 with the fragment reads from LDS.  One instruction takes a whole 128-byte
// k-tile, so a tile is one k-step: eight wavefronts (4 x 2) of 64 x 128 results = 4 x 8 MFMA tiles, 32 MFMAs per tile.
//
// LDS.  Two buffers per operand of 256 rows x 128 bytes (A's two, then B's two), no padding; chunk c (16 bytes) of row r lies at position
// c ^ ((r / 2) % 8).  Lane l of a fragment holds row l % 16 and the chunks l / 16 and l / 16 + 4 of the row (the same
// regrouping of k for A and B, so the products pair up): the sixteen lanes that a ds_read_b128 serves in one pass
// (lanes 0-3, 12-15, 20-27 of a half-wave, then the rest) then read sixteen different groups of four banks.
//
// Feeding.  global_load_lds_dwordx4: one instruction of a wavefront moves 1 KiB, eight rows, lane i to byte 16 i of
// the block, so the swizzle is applied on the source side (the lane that fills position p of row r fetches chunk
// p ^ ((r / 2) % 8), inside the row's one 128-byte line).  No staging registers, no LDS stores.  The instruction is
// written out: through the builtin the compiler waits for all outstanding loads in front of LDS reads it cannot tell
// apart from the landing tile.
//
// Pipeline.  The MFMAs of a tile go column by column; the B fragment of a column is read two columns ahead (four B
// fragments in registers), the four A fragments of a tile have a second set.  One barrier per tile, in front of
// column 6: by then a wavefront has received all its fragments of the tile (so the tile's buffer is free) and has
// waited for its share of the next tile (so that tile is complete once everyone has arrived).  Behind the barrier,
// under the MFMAs of columns 6 and 7, the next tile's A fragments and first two B fragments are read, and the loads
// of the tile after next start into the freed buffer (four instructions behind each of these two columns; spread over
// four columns, two each, measured 1 to 4 % slower): they have until the next tile's column 6 to land.
#ifndef KCG_GEMM8D_HELPERS
#define KCG_GEMM8D_HELPERS
template <bool B> struct KcgBool8d { static constexpr bool v = B; };
#endif
#ifndef G8_SCALE_PTR
#define G8_SCALE_PTR 0
#define G8_SCALE_PTR_DEFAULTED
#endif
#if (G8_M % 256) || (G8_N % 256) || (G8_K % 128)
#error "gemm_fp8_d2l: whole 256 x 256 x 128 tiles only"
#endif
#if G8_OUT_BF16
#define G8_C_T unsigned short
#else
#define G8_C_T float
#endif
#define G8_KT (G8_K / 128)
#ifndef G8_BTR
#define G8_BTR 0
#define G8_BTR_DEFAULTED
#endif
#ifndef G8_PERSIST
#define G8_PERSIST 0
#define G8_PERSIST_DEFAULTED
#endif
#if G8_PERSIST && (G8_BATCH != 1 || ((G8_K / 128) % 2))
#error "gemm_fp8_d2l: persistent workgroups need one batch and an even number of k-tiles"
#endif
#ifndef G8_NT_STORE
#define G8_NT_STORE 0
#define G8_NT_STORE_DEFAULTED
#endif
#ifndef G8_STAGGER
#define G8_STAGGER 0
#define G8_STAGGER_DEFAULTED
#endif
#ifndef G8_STAGE_C
#define G8_STAGE_C 0
#define G8_STAGE_C_DEFAULTED
#endif
#if G8_STAGE_C && G8_PERSIST
#error "gemm_fp8_d2l: results do not go through LDS with persistent workgroups (whose LDS holds the next tile by then)"
#endif

extern "C" __global__ __launch_bounds__(512)
#if G8_SCALE_PTR == 2
void G8_NAME(const unsigned char* __restrict__ A, const unsigned char* __restrict__ B,
             const float* __restrict__ scale_a_p, const float* __restrict__ scale_b_p, G8_C_T* __restrict__ C) {
  const float scale_a = *scale_a_p, scale_b = *scale_b_p;
#elif G8_SCALE_PTR == 1
void G8_NAME(const unsigned char* __restrict__ A, const unsigned char* __restrict__ B, G8_C_T* __restrict__ C,
             const float* __restrict__ scale_a_p, const float* __restrict__ scale_b_p) {
  const float scale_a = *scale_a_p, scale_b = *scale_b_p;
#else
void G8_NAME(const unsigned char* __restrict__ A, const unsigned char* __restrict__ B, G8_C_T* __restrict__ C,
             float scale_a, float scale_b) {
#endif
  // bytes: a row, an operand tile.  LDS holds A's two tiles, then B's two: the other buffer of an operand is 32 KiB away,
  // which an LDS instruction's 16-bit offset field reaches (one address register per fragment for both buffers)
  constexpr int ROWB = 128, TILE = 256 * ROWB, BUF = TILE, B_AT = 2 * TILE;
  constexpr int TM = 4, TN = 8;
  __shared__ __attribute__((aligned(1024))) char kcg_smem[4 * TILE];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int wm = wave / 2, wn = wave % 2;
  const int l16 = lane & 15, lq = lane >> 4;

#if G8_STAGGER
  // Out of step on purpose.  All workgroups of a launch start together and take the same time for a tile, so all of
  // them write their results at the same moment and start their next tile's loads behind that burst.  The workgroups
  // of the first round (one per compute unit) start up to 31 * G8_STAGGER sleeps of 512 cycles apart, in 32 classes
  // per XCD; the rounds after them inherit the offsets.  Measured together with the non-temporal result stores on
  // 4096 x 11008 x 4096: 0.152 ms with both against 0.174 (stores only), 0.186 (stagger only) and 0.190 ms (neither).
  if (blockIdx.x < 256 && blockIdx.y == 0) {
    const int steps = (int)((blockIdx.x >> 3) & 31) * G8_STAGGER;
    for (int d = 0; d < steps; ++d) __builtin_amdgcn_s_sleep(8);
  }
#endif
  const int tiles_m = G8_M / 256, tiles_n = G8_N / 256;
  int tile_m, tile_n;
  kcg_tile_coords(blockIdx.x, tiles_m, tiles_n, G8_GROUP_M, tile_m, tile_n);
  // (the division in kcg_tile_coords runs on the vector unit: the tile origins go back into scalar registers here, the
  // load instructions below take their base addresses from there)
  int m0 = __builtin_amdgcn_readfirstlane(tile_m * 256), n0 = __builtin_amdgcn_readfirstlane(tile_n * 256);
  // Persistent workgroups.  The k-tiles of a workgroup's consecutive output tiles form one stream: the loads of the next
  // output tile's first k-tiles are issued behind the barriers of this one's last two, its first fragments are read
  // under this one's last MFMAs, and only then are the results stored: the stores drain while the next tile multiplies,
  // and the next tile's loads are ahead of them in the memory pipeline instead of behind them as with a new workgroup.
  int pid = blockIdx.x;
  bool has_next = G8_PERSIST && pid + (int)gridDim.x < tiles_m * tiles_n;
  int m0n = 0, n0n = 0;
  if (has_next) {
    kcg_tile_coords(pid + (int)gridDim.x, tiles_m, tiles_n, G8_GROUP_M, tile_m, tile_n);
    m0n = __builtin_amdgcn_readfirstlane(tile_m * 256); n0n = __builtin_amdgcn_readfirstlane(tile_n * 256);
  }
  const long batch = blockIdx.y;
  A += batch * (long)G8_M * G8_K;
  B += batch * (long)G8_K * G8_N;
  C += batch * (long)G8_M * G8_N;

  // ---- loads: instruction t (0..3) of this wavefront moves rows (4 wave + t) * 8 .. + 7 of an operand tile ----
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)kcg_smem;
  const unsigned lds_wave = __builtin_amdgcn_readfirstlane(lds_base + wave_u * 4096);
  const unsigned dma_lane = (unsigned)(lane >> 3) * (unsigned)G8_K + (unsigned)(((lane & 7) ^ (lane >> 4)) * 16);
  const unsigned char* rowsA = A + (long)(m0 + wave_u * 32) * G8_K;
  const unsigned char* rowsAn = A + (long)(m0n + wave_u * 32) * G8_K;
#if G8_BTR
  // Row-major weights, B[K][N]: a tile is 128 k rows of 256 bytes of consecutive n; an instruction moves four of them,
  // block 4 wave + t.  The 16-byte granule g of row k lies at granule g ^ f(k), f(k) = k % 8 + 8 ((k / 16) % 2): the
  // sixteen rows that the transposing reads of two lane groups take together (k0 .. k0 + 7 and k0 + 16 .. k0 + 23) then
  // fall on sixteen different groups of four banks.  For lane i of block 4 wave + t: f = i / 16 + 4 (t % 2) + 8 (wave % 2).
  const unsigned dma_lane_b = (unsigned)(lane >> 4) * (unsigned)G8_N + (unsigned)((((lane & 15) ^ (lane >> 4)) ^ (8 * (wave & 1))) * 16);
  const unsigned char* rowsB = B + (long)(wave_u * 16) * G8_N + n0;
  const unsigned char* rowsBn = B + (long)(wave_u * 16) * G8_N + n0n;
#else
  const unsigned char* rowsB = B + (long)(n0 + wave_u * 32) * G8_K;
  const unsigned char* rowsBn = B + (long)(n0n + wave_u * 32) * G8_K;
#endif
  // u: 0..3 = A, 4..7 = B; the parity of the eight-row (B[K][N]: four-row) group within the tile is that of t
  // (k-tile kt of this output tile, or, past its end, k-tile kt - G8_KT of the workgroup's next one)
  auto dma = [&](int u, int kt, int buf) __attribute__((always_inline)) {
    const int t = u & 3;
    const bool nxt = kt >= G8_KT;
    if (nxt) kt -= G8_KT;
    const unsigned char* rA = nxt ? rowsAn : rowsA;
    const unsigned char* rB = nxt ? rowsBn : rowsB;
#if G8_BTR
    const unsigned char* base = u < 4 ? rA + (long)t * 8 * G8_K + (long)kt * 128 : rB + ((long)kt * 128 + t * 4) * G8_N;
    const unsigned lane_off = (u < 4 ? dma_lane : dma_lane_b) ^ (unsigned)((t & 1) * 64);
#else
    const unsigned char* base = (u < 4 ? rA : rB) + (long)t * 8 * G8_K + (long)kt * 128;
    const unsigned lane_off = dma_lane ^ (unsigned)((t & 1) * 64);
#endif
    // the block's place in LDS: the wavefront's 4 KiB of the operand tile plus a constant; the sum is formed here each
    // time (the empty statement hides that lds_wave never changes): sixteen sums kept in scalar registers for the
    // whole kernel were what pushed the persistent form's registers into scratch memory
    unsigned w = lds_wave;
    asm volatile("" : "+s"(w));
    const unsigned dst = w + (unsigned)(buf * BUF + (u < 4 ? 0 : B_AT) + t * 1024);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(lane_off), "s"(base), "s"(dst) : "memory");
  };

  // ---- fragments ----
  const int sw = (l16 >> 1) & 7;
  const int pos0 = (lq ^ sw) * 16, pos1 = ((lq + 4) ^ sw) * 16;                 // the lane's two chunks of a row
  const char* fA = kcg_smem + (wm * 64 + l16) * ROWB;
  const char* fB = kcg_smem + B_AT + (wn * 128 + l16) * ROWB;
  auto frag = [&](const char* row) __attribute__((always_inline)) -> kcg_i32x8 {
    const kcg_i32x4 lo = *(const kcg_i32x4*)(row + pos0), hi = *(const kcg_i32x4*)(row + pos1);
    kcg_i32x8 r = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return r;
  };

  // B fragment of column tile j out of buffer `buf`
#if G8_BTR
  // four transposing reads (ds_read_b64_tr_b8: within each group of 16 lanes, lane r supplies the address of 8 bytes,
  // and lane i receives byte i % 8 ... of rows 2 j + i / 8: with the even lanes at sB[k + r / 2][n .. n + 7] and the odd
  // ones at [n + 8 .. n + 15], lane i receives the eight consecutive k of column n + i) for the lane group's k values
  // 16 q .. + 15 and 64 + 16 q .. + 15, in the order the A fragment has them
  typedef __attribute__((address_space(3))) char* kcg_lds_ptr8d;
  typedef int kcg_i32x2_trd __attribute__((ext_vector_type(2)));
  const int fswz = ((lane & 15) >> 1) | (((lane >> 4) & 1) << 3);
  const unsigned bT = lds_base + B_AT + (16 * lq + ((lane & 15) >> 1)) * 256 + (((8 * wn) ^ fswz) * 16) + 8 * (lane & 1);
  auto fragB = [&](int buf, int j) __attribute__((always_inline)) -> kcg_i32x8 {
    const kcg_lds_ptr8d p = (kcg_lds_ptr8d)(size_t)((bT + buf * BUF) ^ (unsigned)(j * 16));
    kcg_i32x8 r;
#pragma unroll
    for (int x = 0; x < 4; ++x) {
      const kcg_i32x2_trd v = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
          (__attribute__((address_space(3))) kcg_i32x2_trd*)(p + ((x & 1) * 8 + (x >> 1) * 64) * 256));
      r[2 * x] = v[0];
      r[2 * x + 1] = v[1];
    }
    return r;
  };
#else
  auto fragB = [&](int buf, int j) __attribute__((always_inline)) -> kcg_i32x8 { return frag(fB + buf * BUF + j * 16 * ROWB); };
#endif

  kcg_f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.0f;

  // ---- prologue: tile 0 into buffer 0, wait, tile 1 into buffer 1, first fragments ----
#pragma unroll
  for (int u = 0; u < 8; ++u) dma(u, 0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);                                           // vmcnt(0)
  __syncthreads();
  if (1 < G8_KT) {
#pragma unroll
    for (int u = 0; u < 8; ++u) dma(u, 1, 1);
  }
  kcg_i32x8 fa[2][TM], fb[4];
#pragma unroll
  for (int i = 0; i < TM; ++i) fa[0][i] = frag(fA + i * 16 * ROWB);
  fb[0] = fragB(0, 0);
  fb[1] = fragB(0, 1);

  // The results of the 16 x 16 tiles of column j: lane l, register v -> row 4 (l / 16) + v, column l % 16
  // (a lane's 16 bytes per row instead of 4, with the MFMA operands exchanged, and the rows' pieces in another order
  // were measured: the same time)
  const float scale = scale_a * scale_b;
  auto store_column = [&](int j, int mt, int nt) __attribute__((always_inline)) {
    char* Cw = (char*)(C + (long)(mt + (wave_u >> 1) * 64) * G8_N + nt + (wave_u & 1) * 128);
    unsigned lane_at = (unsigned)((4 * lq * G8_N + l16) * sizeof(G8_C_T));
    asm volatile("" : "+v"(lane_at));                      // one register, not 128 precomputed offsets
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        G8_C_T* at = (G8_C_T*)(Cw + (lane_at + (unsigned)(((i * 16 + v) * G8_N + j * 16) * sizeof(G8_C_T))));
        const float r = G8_RELU ? fmaxf(acc[i][j][v] * scale, 0.0f) : acc[i][j][v] * scale;
#if G8_OUT_BF16
        *at = (unsigned short)kcg_f32_to_bf16_bits(r);
#elif G8_NT_STORE
        __builtin_nontemporal_store(r, at);
#else
        *at = r;
#endif
      }
  };

  // Tile kt out of buffer par, A fragments in set par.  Column j's B fragment sits in slot j % 4 and is read two
  // columns ahead.  The barrier stands in front of column 6: the fragments of columns 6 and 7 are in registers by then.
  auto tile = [&](const int kt, auto par_c) {
    constexpr int par = decltype(par_c)::v ? 1 : 0;
    const bool more = kt + 1 < G8_KT || has_next;         // there is a next tile: read its first fragments
    const bool fetch = kt + 2 < G8_KT || has_next;        // and one after it: load it into this tile's buffer
    const char* nA = fA + (par ^ 1) * BUF;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      __builtin_amdgcn_sched_barrier(0);
      if (j + 2 < TN) fb[(j + 2) & 3] = fragB(par, j + 2);
      if (j == 6) {
        __builtin_amdgcn_s_waitcnt(0x0F70);               // vmcnt(0): this wavefront's share of tile kt+1 has landed
        __syncthreads();                                   // (its wait for LDS covers the last fragment reads of tile kt)
      }
      if (j >= 6 && more) {                                // the next tile's A fragments and its first two B fragments
        fa[par ^ 1][2 * (j - 6)] = frag(nA + (2 * (j - 6)) * 16 * ROWB);
        fa[par ^ 1][2 * (j - 6) + 1] = frag(nA + (2 * (j - 6) + 1) * 16 * ROWB);
        fb[j - 6] = fragB(par ^ 1, j - 6);
      }
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        __builtin_amdgcn_sched_barrier(0);
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fa[par][i], fb[j & 3], acc[i][j], 0, 0, 0, 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      // all eight loads of tile kt+2 go out in the two columns behind the barrier, four each: they then have six columns
      // of MFMA work to land before the next barrier asks for them
      if (j >= 6 && fetch) {
        const int u = 2 * (j - 6);
        dma(u, kt + 2, par); dma(u + 1, kt + 2, par); dma(4 + u, kt + 2, par); dma(5 + u, kt + 2, par);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  for (;;) {
    int kt = 0;
    for (; kt + 1 < G8_KT; kt += 2) {
      tile(kt, KcgBool8d<false>{});
      tile(kt + 1, KcgBool8d<true>{});
    }
    if (kt < G8_KT) tile(kt, KcgBool8d<false>{});

    // (storing a tile's results column by column under the first k-tile of the workgroup's next tile instead, through
    // buffer stores, was measured: 0.172 against 0.168 ms)
#if G8_STAGE_C
    // Whole rows.  Out of the accumulators a store instruction writes 16 values of each of four rows (64 bytes in fp32,
    // 32 in bf16), and the pieces of a 128-byte line leave at different times.  Here the tile goes through LDS: as fp32
    // in two halves of 128 rows (the wavefront's MFMA tile rows 0-1, then 2-3: every wavefront takes part in both), as
    // bf16 at once.  Row r of the staged part is 256 values, its chunk c of 16 values at chunk c ^ ((r / 4) % 4), so that
    // the four rows a wavefront writes at a time fall on different banks; then every lane stores 16 bytes of a row, a
    // wavefront one whole row (fp32) or two (bf16) at a time.
    {
      constexpr int ES = (int)sizeof(G8_C_T), PASSES = ES == 4 ? 2 : 1, RP = 256 / PASSES;   // rows per pass
      constexpr int LPR = 256 * ES / 16, RPI = 64 / LPR, EPL = 16 / ES;                       // lanes per row, rows per instruction, values per lane
      G8_C_T* stage = (G8_C_T*)kcg_smem;
      const int srow0 = (wave_u >> 1) * (64 / PASSES) + 4 * lq;     // + 16 ii + v: the lane's row within the staged part
      const int scol0 = (wave_u & 1) * 128 + l16;                   // + 16 j
#pragma unroll
      for (int pass = 0; pass < PASSES; ++pass) {
        __syncthreads();                                   // the k loop's last fragment reads / the first half's reads are done
#pragma unroll
        for (int ii = 0; ii < TM / PASSES; ++ii)
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
              const int i = pass * (TM / PASSES) + ii;
              const float r = G8_RELU ? fmaxf(acc[i][j][v] * scale, 0.0f) : acc[i][j][v] * scale;
              const int row = srow0 + 16 * ii + v, col = scol0 + 16 * j;      // (row / 4) % 4 == lq
#if G8_OUT_BF16
              stage[row * 256 + (col ^ (16 * lq))] = (unsigned short)kcg_f32_to_bf16_bits(r);
#else
              stage[row * 256 + (col ^ (16 * lq))] = r;
#endif
            }
        __syncthreads();
#pragma unroll
        for (int x = 0; x < RP / 8 / RPI; ++x) {
          const int row = wave_u * (RP / 8) + x * RPI + lane / LPR;           // row of the staged part
          const int col = (lane % LPR) * EPL;
          const kcg_f32x4 val = *(const kcg_f32x4*)(stage + row * 256 + (col ^ (16 * ((row >> 2) & 3))));
          const int trow = PASSES == 2 ? (row >> 5) * 64 + 32 * pass + (row & 31) : row;
          G8_C_T* at = C + (long)(m0 + trow) * G8_N + n0 + col;
#if G8_NT_STORE
          __builtin_nontemporal_store(val, (kcg_f32x4*)at);
#else
          *(kcg_f32x4*)at = val;
#endif
        }
      }
    }
#else
#pragma unroll
    for (int j = 0; j < TN; ++j) store_column(j, m0, n0);
#endif
    if (!has_next) break;
    // the next output tile becomes the current one; its first fragments are in registers, its first k-tiles on their way
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.0f;
    pid += (int)gridDim.x;
    m0 = m0n; n0 = n0n; rowsA = rowsAn; rowsB = rowsBn;
    has_next = pid + (int)gridDim.x < tiles_m * tiles_n;
    if (has_next) {
      kcg_tile_coords(pid + (int)gridDim.x, tiles_m, tiles_n, G8_GROUP_M, tile_m, tile_n);
      m0n = __builtin_amdgcn_readfirstlane(tile_m * 256); n0n = __builtin_amdgcn_readfirstlane(tile_n * 256);
      rowsAn = A + (long)(m0n + wave_u * 32) * G8_K;
#if G8_BTR
      rowsBn = B + (long)(wave_u * 16) * G8_N + n0n;
#else
      rowsBn = B + (long)(n0n + wave_u * 32) * G8_K;
#endif
    }
  }
}
#undef G8_C_T
#undef G8_KT
#ifdef G8_SCALE_PTR_DEFAULTED
#undef G8_SCALE_PTR
#undef G8_SCALE_PTR_DEFAULTED
#endif
#ifdef G8_BTR_DEFAULTED
#undef G8_BTR
#undef G8_BTR_DEFAULTED
#endif
#ifdef G8_PERSIST_DEFAULTED
#undef G8_PERSIST
#undef G8_PERSIST_DEFAULTED
#endif
#ifdef G8_NT_STORE_DEFAULTED
#undef G8_NT_STORE
#undef G8_NT_STORE_DEFAULTED
#endif
#ifdef G8_STAGGER_DEFAULTED
#undef G8_STAGGER
#undef G8_STAGGER_DEFAULTED
#endif
#ifdef G8_STAGE_C_DEFAULTED
#undef G8_STAGE_C
#undef G8_STAGE_C_DEFAULTED
#endif
