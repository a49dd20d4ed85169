// ---- fp32 GEMM on v_mfma_f32_32x32x2_f32, operand tiles straight from global memory into LDS ----------------------
// C[b] = A[b] * B[b]: A [M][K], B [K][N], C [M][N], all row-major fp32; whole GL_BM x GL_BN x GL_BK tiles only (the emitter
// falls back to gemm_f32.hip for every other case).  Parameters:
//   GL_NAME                      kernel symbol
//   GL_M GL_N GL_K GL_BATCH      problem: multiples of GL_BM, GL_BN and GL_BK
//   GL_BM GL_BN GL_BK            workgroup tile: GL_BM a multiple of 64, GL_BN 64, 128 or 256, GL_BK 16 or 32
//   GL_WM GL_WN                  wavefronts along m and n; a wavefront's part of the tile is whole 32 x 32 MFMA tiles
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
#define GL_KT (GL_K / GL_BK)
#define GL_NW (GL_WM * GL_WN)
#define GL_TM (GL_BM / GL_WM / 32)
#define GL_TN (GL_BN / GL_WN / 32)

extern "C" __global__ __launch_bounds__(64 * GL_NW)
void GL_NAME(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C) {
  constexpr int ROW_A = GL_BK * 4, CH = GL_BK / 4;        // bytes and 16-byte chunks of a row of the A tile
  constexpr int SW_SH = GL_BK == 16 ? 2 : 1;              // chunk c of row m lies at c ^ ((m >> SW_SH) % CH)
  constexpr int TILE_A = GL_BM * ROW_A, TILE_B = GL_BN * ROW_A;  // bytes of the operand tiles
  constexpr int B_AT = 2 * TILE_A;                        // A's two buffers, then B's two
  constexpr int ROW_B = GL_BN * 4;                        // bytes of a row (k) of the B tile
  constexpr int BLK_A = TILE_A / 1024, BLK = (TILE_A + TILE_B) / 1024;   // 1 KiB blocks of the A tile, of both tiles
  constexpr int STEPS = GL_BK / 8;                        // MFMA steps of eight k (four MFMAs per tile pair) per k-tile
  __shared__ __attribute__((aligned(1024))) char kcg_smem[2 * TILE_A + 2 * TILE_B];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int wm = wave / GL_WN, wn = wave % GL_WN;
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
  const int sw = (ma >> SW_SH) & (CH - 1);                 // the same for every block: 32 rows further changes nothing
  const char* fA = kcg_smem + ma * ROW_A;
  const char* fB = kcg_smem + B_AT + lh * 4 * ROW_B + (wn * (GL_TN * 32) + l32) * 4;
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
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      if (st + 1 < STEPS) {
        read_fragments(par, st + 1, fa[(st + 1) & 1], fb[(st + 1) & 1]);
      } else {
        __builtin_amdgcn_s_waitcnt(0x0F70);                // vmcnt(0): this wavefront's blocks of tile kt+1 have landed
        __syncthreads();                                   // (its wait for LDS covers the last fragment reads of tile kt)
        if (more) read_fragments(par ^ 1, 0, fa[0], fb[0]);
      }
      half(fa[st & 1], fb[st & 1]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  {
    int kt = 0;
    for (; kt + 1 < GL_KT; kt += 2) {
      tile(kt, KcgBool32d<false>{});
      tile(kt + 1, KcgBool32d<true>{});
    }
    if (kt < GL_KT) tile(kt, KcgBool32d<false>{});
  }

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
#undef GL_TM
#undef GL_TN
