// ---- fp32 GEMM on v_mfma_f32_32x32x2_f32, operand tiles straight from global memory into LDS ----------------------
// C[b] = A[b] * B[b]: A [M][K], B [K][N], C [M][N], all row-major fp32; whole GL_BM x GL_BN x GL_BK tiles only (the emitter
// falls back to gemm_f32.hip for every other case).  Parameters:
//   GL_NAME                      kernel symbol
//   GL_M GL_N GL_K GL_BATCH      problem: multiples of GL_BM, GL_BN and GL_BK
//   GL_BM GL_BN GL_BK            workgroup tile: GL_BM a multiple of 64, GL_BN 64, 128 or 256, GL_BK 16 or 32
//   GL_WM GL_WN                  wavefronts along m and n; a wavefront's part of the tile is whole 32 x 32 MFMA tiles
//   GL_WK                        (1 or 2) groups of GL_WM x GL_WN wavefronts that share the tile's results and split the
//                                steps of every k-tile between them (group g takes the steps u with u % GL_WK == g); the
//                                groups' partial sums are added through LDS after the last k-tile.  Small tiles have one
//                                wavefront per SIMD otherwise, and nothing runs while it waits at the k-tile's barrier.
//   GL_GROUP_M                   tile rows per L2 strip
//   GL_RELU                      1: fused max(0, .) epilogue
//
// For 256 x 256 tiles: sixteen wavefronts (4 x 4) of 64 x 64 results = 2 x 2 MFMA tiles of 32 x 32.  What gemm_f32.hip
// spends between global memory and LDS - a float4 per operand and thread in registers, four scattered LDS stores to turn
// a k-contiguous row of A into the k-major tile - is not there: a k-tile is (GL_BM + GL_BN) GL_BK / 256 global_load_lds_dwordx4
// of 1 KiB, dealt round-robin to the wavefronts (one of each operand per wavefront for 256 x 256 tiles), and both tiles
// lie in LDS as they lie in memory.
//
// A in LDS: GL_BM rows of 64 bytes (16 k; 128 bytes with GL_BK 32), no padding; the 16-byte chunk c (four k) of row m
// lies at position c ^ ((m / 4) % 4) (GL_BK 32: c ^ ((m / 2) % 8)).  A lane of an MFMA holds row m = lane % 32 and,
// with one ds_read_b128, the four k of chunk 2 u + lane / 32 (u: the steps of eight k of the k-tile); the sixteen lanes
// that such a read serves in one pass (rows 0-3, 12-15, 20-27 of a 32-row block, then the rest) then fall on sixteen
// different groups of four banks.  The swizzle is applied on the source side of the load: lane i of a block writes 16
// bytes at 16 i, that is position i % 4 of row i / 4 (i % 8 of row i / 8), and fetches the chunk that belongs there.
// B in LDS: GL_BK rows (k) of GL_BN floats, as in memory (a 1 KiB block is 256 / GL_BN rows); a lane reads one float of row k
// at column n = lane % 32 of its block.
// An MFMA sums over the two k that its two half-waves hold; which two is free as long as both operands agree: MFMA e
// of step u takes k = 8 u + e from the lower half-wave and 8 u + 4 + e from the upper.
//
// Pipeline.  One barrier per k-tile, in front of the MFMAs of its last step: by then a wavefront has read all its
// fragments of the tile (so the buffer is free) and has waited for its own loads of the next tile (so that tile is
// complete once everyone has arrived).  Behind it the first step's fragments of the next tile are read; the loads of
// the tile after next start at the top of the next tile.  Fragments are read one step ahead into a second set.
#ifndef KCG_GEMM32D_HELPERS
#define KCG_GEMM32D_HELPERS
template <bool B> struct KcgBool32d { static constexpr bool v = B; };
#endif
#if (GL_M % GL_BM) || (GL_N % GL_BN) || (GL_K % GL_BK) || (GL_BK != 16 && GL_BK != 32)
#error "gemm_f32_d2l: whole tiles only"
#endif
#if (GL_BM % 64) || (GL_BN != 64 && GL_BN != 128 && GL_BN != 256) || (GL_BM % (32 * GL_WM)) || (GL_BN % (32 * GL_WN))
#error "gemm_f32_d2l: GL_BM is a multiple of 64, GL_BN 64, 128 or 256 (a 1 KiB block is whole rows of the B tile), 32 x 32 MFMA tiles per wavefront"
#endif
#ifndef GL_WK
#define GL_WK 1
#define GL_WK_DEFAULTED
#endif
#if (GL_WK != 1 && GL_WK != 2) || (GL_WK == 2 && GL_BK != 32) || (GL_WK == 2 && GL_BM * GL_BN * 4 > (GL_BM + GL_BN) * GL_BK * 8)
#error "gemm_f32_d2l: GL_WK is 1 or 2; 2 needs k-tiles of 32 (an even number of steps per group) and results that fit the LDS tiles"
#endif
// GL_NBUF (2, 3 or 4) LDS buffers per operand: the loads of k-tile kt + GL_NBUF - 1 start at the top of k-tile kt.  A small
// tile's k-tile is shorter than a load's way from the L2 (64 x 64 x 32: sixteen MFMAs, 0.43 us), and with two buffers every
// k-tile then lasts as long as a load.  More than two buffers need every wavefront to issue the same number of loads
// per k-tile (the wait for "all but the youngest tiles" counts instructions).
#ifndef GL_NBUF
#define GL_NBUF 2
#define GL_NBUF_DEFAULTED
#endif
#define GL_KT (GL_K / GL_BK)
#define GL_NG (GL_WM * GL_WN)
#define GL_NW (GL_NG * GL_WK)
#define GL_TM (GL_BM / GL_WM / 32)
#define GL_TN (GL_BN / GL_WN / 32)

extern "C" __global__ __launch_bounds__(64 * GL_NW)
void GL_NAME(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C) {
  constexpr int ROW_A = GL_BK * 4, CH = GL_BK / 4;        // bytes and 16-byte chunks of a row of the A tile
  constexpr int SW_SH = GL_BK == 16 ? 2 : 1;              // chunk c of row m lies at c ^ ((m >> SW_SH) % CH)
  constexpr int TILE_A = GL_BM * ROW_A, TILE_B = GL_BN * ROW_A;  // bytes of the operand tiles
  constexpr int B_AT = GL_NBUF * TILE_A;                  // A's buffers, then B's
  constexpr int ROW_B = GL_BN * 4;                        // bytes of a row (k) of the B tile
  constexpr int BLK_A = TILE_A / 1024, BLK = (TILE_A + TILE_B) / 1024;   // 1 KiB blocks of the A tile, of both tiles
  constexpr int STEPS = GL_BK / 8;                        // MFMA steps of eight k (four MFMAs per tile pair) per k-tile
  __shared__ __attribute__((aligned(1024))) char kcg_smem[GL_NBUF * (TILE_A + TILE_B)];
  static_assert(GL_NBUF == 2 || (GL_NBUF >= 3 && GL_NBUF <= 4 && BLK % (GL_WM * GL_WN * GL_WK) == 0),
                "gemm_f32_d2l: GL_NBUF is 2, or 3 or 4 with the k-tile's 1 KiB blocks a multiple of the wavefronts");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int wk = wave / GL_NG;                             // the wavefront's group: its share of every k-tile's steps
  const int wm = (wave % GL_NG) / GL_WN, wn = wave % GL_WN;
  const int l32 = lane & 31, lh = lane >> 5;

  const int tiles_m = GL_M / GL_BM, tiles_n = GL_N / GL_BN;
  int tile_m, tile_n;
  kcg_tile_coords(blockIdx.x, tiles_m, tiles_n, GL_GROUP_M, tile_m, tile_n);
  // (the division in kcg_tile_coords runs on the vector unit: the tile origins go back into scalar registers here, the
  // load instructions below take their base addresses from there)
  const int m0 = __builtin_amdgcn_readfirstlane(tile_m * GL_BM), n0 = __builtin_amdgcn_readfirstlane(tile_n * GL_BN);
  const long batch = blockIdx.y;
  A += batch * (long)GL_M * GL_K;
  B += batch * (long)GL_K * GL_N;
  C += batch * (long)GL_M * GL_N;

  // ---- loads: block b of a k-tile's BLK blocks of 1 KiB (A's sixteen-row groups, then B's groups of 256 / GL_BN rows)
  //      is moved by wavefront b % GL_NW ----
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)kcg_smem;
  // (GL_BK 32: a block is eight rows, and the rows of an odd block are swizzled with 4 more: byte offset ^ 64)
  const unsigned a_lane = (unsigned)(lane / CH) * (unsigned)(GL_K * 4) + (unsigned)(((lane % CH) ^ ((lane >> 4) & 3)) * 16);
  const unsigned b_lane = (unsigned)(lane / (GL_BN / 4)) * (unsigned)(GL_N * 4) + (unsigned)(lane % (GL_BN / 4)) * 16u;
  const char* tileA = (const char*)(A + (long)m0 * GL_K);
  const char* tileB = (const char*)(B + n0);
  auto dma = [&](int kt, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int x = 0; x < (BLK + GL_NW - 1) / GL_NW; ++x) {
      const int blk = wave_u + x * GL_NW;                  // wave-uniform
      if (BLK % GL_NW == 0 || blk < BLK) {
        const bool is_a = blk < BLK_A;
        const int bb = blk - BLK_A;                        // B: rows bb * (1024 / ROW_B) .. of the k-tile
        unsigned dst = lds_base + (is_a ? (unsigned)(buf * TILE_A + blk * 1024) : (unsigned)(B_AT + buf * TILE_B + bb * 1024));
        dst = __builtin_amdgcn_readfirstlane(dst);
        const char* src = is_a ? tileA + (long)blk * (1024 / ROW_A) * GL_K * 4 + (long)kt * ROW_A
                               : tileB + ((long)kt * GL_BK + (long)bb * (1024 / ROW_B)) * GL_N * 4;
        const unsigned lane_off = is_a ? (GL_BK == 32 ? a_lane ^ (unsigned)((blk & 1) * 64) : a_lane) : b_lane;
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(lane_off), "s"(src), "s"(dst) : "memory");
      }
    }
  };

  // ---- fragments of half u of the tile in buffer buf ----
  const int ma = wm * (GL_TM * 32) + l32;                  // the lane's row of A's first block; the next are 32 further each
  // (group wk reads step u + wk where the text below says u, u a multiple of GL_WK: the group's chunk 2 wk of A goes into
  // the swizzle term, which is exact because 2 u, 2 wk and lh occupy different bits, its eight rows of B into the base)
  const int sw = ((ma >> SW_SH) & (CH - 1)) ^ (2 * wk);    // the same for every block: 32 rows further changes nothing
  const char* fA = kcg_smem + ma * ROW_A;
  const char* fB = kcg_smem + B_AT + (8 * wk + lh * 4) * ROW_B + (wn * (GL_TN * 32) + l32) * 4;
  auto read_fragments = [&](int buf, int u, kcg_f32x4 (&a)[GL_TM], float (&b)[GL_TN][4]) __attribute__((always_inline)) {
    const int pos = ((2 * u + lh) ^ sw) * 16;
#pragma unroll
    for (int i = 0; i < GL_TM; ++i) a[i] = *(const kcg_f32x4*)(fA + buf * TILE_A + i * 32 * ROW_A + pos);
#pragma unroll
    for (int j = 0; j < GL_TN; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) b[j][e] = *(const float*)(fB + buf * TILE_B + (8 * u + e) * ROW_B + j * 128);
  };

  kcg_f32x16 acc[GL_TM][GL_TN];
#pragma unroll
  for (int i = 0; i < GL_TM; ++i)
#pragma unroll
    for (int j = 0; j < GL_TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // ---- prologue: tile 0 into buffer 0, wait, first fragments ----
  dma(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);                      // vmcnt(0)
  __syncthreads();
  kcg_f32x4 fa[2][GL_TM];
  float fb[2][GL_TN][4];
  read_fragments(0, 0, fa[0], fb[0]);

  auto half = [&](kcg_f32x4 (&a)[GL_TM], float (&b)[GL_TN][4]) __attribute__((always_inline)) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int i = 0; i < GL_TM; ++i)
#pragma unroll
        for (int j = 0; j < GL_TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][e], b[j][e], acc[i][j], 0, 0, 0);
  };
  auto tile = [&](const int kt, auto par_c) {
    constexpr int par = decltype(par_c)::v ? 1 : 0;
    const bool more = kt + 1 < GL_KT;
    if (more) dma(kt + 1, par ^ 1);                        // the other buffer is free since the last barrier
    __builtin_amdgcn_sched_barrier(0);
    // the group's own steps: wk, wk + GL_WK, ... (read_fragments adds the wk); OWN of them per k-tile, fragment set s & 1 for the s-th
    constexpr int OWN = STEPS / GL_WK;
#pragma unroll
    for (int s = 0; s < OWN; ++s) {
      if (s + 1 < OWN) {
        read_fragments(par, (s + 1) * GL_WK, fa[(s + 1) & 1], fb[(s + 1) & 1]);
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);                // vmcnt(0): this wavefront's blocks of tile kt+1 have landed
        __syncthreads();                                   // (its wait for LDS covers the last fragment reads of tile kt)
        if (more) read_fragments(par ^ 1, 0, fa[0], fb[0]);     // OWN is even: the step below uses set 1
      }
      half(fa[s & 1], fb[s & 1]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
#if GL_NBUF == 2
  {
    int kt = 0;
    for (; kt + 1 < GL_KT; kt += 2) {
      tile(kt, KcgBool32d<false>{});
      tile(kt + 1, KcgBool32d<true>{});
    }
    if (kt < GL_KT) tile(kt, KcgBool32d<false>{});
  }
#else
  {
    // k-tile kt lies in buffer kt % GL_NBUF; tiles 1 .. GL_NBUF - 2 are sent for here, tile kt + GL_NBUF - 1 at the top of
    // tile kt, into the buffer that tile kt - 1 was read from (free since that tile's barrier).  Loads land in the order
    // they were issued, so "tile kt + 1 has landed" is "at most the loads of the GL_NBUF - 2 tiles after it are out".
    constexpr int PER = BLK / GL_NW;                       // load instructions per wavefront and k-tile
    constexpr int OWN = STEPS / GL_WK;
#pragma unroll
    for (int t = 1; t < GL_NBUF - 1; ++t)
      if (t < GL_KT) dma(t, t);
    int buf = 0, nbuf = GL_NBUF - 1;                       // buffer of tile kt, of tile kt + GL_NBUF - 1
#pragma unroll 1
    for (int kt = 0; kt < GL_KT; ++kt) {
      const bool sent = kt + GL_NBUF - 1 < GL_KT;
      if (sent) dma(kt + GL_NBUF - 1, nbuf);
      const int next = buf + 1 == GL_NBUF ? 0 : buf + 1;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < OWN; ++s) {
        if (s + 1 < OWN) {
          read_fragments(buf, (s + 1) * GL_WK, fa[(s + 1) & 1], fb[(s + 1) & 1]);
        } else {
          if (sent) __builtin_amdgcn_s_waitcnt(0x0F70 | (((GL_NBUF - 2) * PER) & 15) | ((((GL_NBUF - 2) * PER) >> 4) << 14));
          else __builtin_amdgcn_s_waitcnt(0x0F70);         // the last tiles: nothing younger is out, wait for all
          __syncthreads();
          if (kt + 1 < GL_KT) read_fragments(next, 0, fa[0], fb[0]);
        }
        half(fa[s & 1], fb[s & 1]);
        __builtin_amdgcn_sched_barrier(0);
      }
      buf = next;
      nbuf = nbuf + 1 == GL_NBUF ? 0 : nbuf + 1;
    }
  }
#endif

#if GL_WK == 2
  // ---- the second group's partial sums through LDS (the tiles are no longer read: every wavefront is past the last
  //      k-tile's barrier and the fragment reads that followed it were skipped) ----
  {
    float* part = (float*)kcg_smem + (wave % GL_NG) * (GL_TM * GL_TN * 16 * 64) + lane;
    __syncthreads();                                       // the other group's last MFMAs have read their fragments
    if (wk == 1) {
#pragma unroll
      for (int i = 0; i < GL_TM; ++i)
#pragma unroll
        for (int j = 0; j < GL_TN; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) part[((i * GL_TN + j) * 16 + v) * 64] = acc[i][j][v];
    }
    __syncthreads();
    if (wk == 1) return;
#pragma unroll
    for (int i = 0; i < GL_TM; ++i)
#pragma unroll
      for (int j = 0; j < GL_TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] += part[((i * GL_TN + j) * 16 + v) * 64];
  }
#endif
  // ---- epilogue: lane l, register v -> row 8*(v/4) + 4*(l/32) + v%4, column l%32 ----
#pragma unroll
  for (int i = 0; i < GL_TM; ++i)
#pragma unroll
    for (int j = 0; j < GL_TN; ++j) {
      const int col = n0 + wn * (GL_TN * 32) + j * 32 + l32;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * (GL_TM * 32) + i * 32 + 8 * (v / 4) + 4 * lh + (v % 4);
        float o = acc[i][j][v];
#if GL_RELU
        o = fmaxf(0.0f, o);
#endif
        C[(long)row * GL_N + col] = o;
      }
    }
}
#undef GL_KT
#undef GL_NW
#undef GL_NG
#ifdef GL_WK_DEFAULTED
#undef GL_WK
#undef GL_WK_DEFAULTED
#endif
#ifdef GL_NBUF_DEFAULTED
#undef GL_NBUF
#undef GL_NBUF_DEFAULTED
#endif
#undef GL_TM
#undef GL_TN
