// ---- fp32 GEMM on v_mfma_f32_32x32x2_f32, operand tiles straight from global memory into LDS ----------------------
// C[b] = A[b] * B[b]: A [M][K], B [K][N], C [M][N], all row-major fp32; whole GD_BM x GD_BN x GD_BK tiles only (the emitter
// falls back to gemm_f32.hip for every other case).  Parameters:
//   GD_NAME                      kernel symbol
//   GD_M GD_N GD_K GD_BATCH      problem: multiples of GD_BM, GD_BN and GD_BK
//   GD_BM GD_BN GD_BK            workgroup tile: GD_BM a multiple of 64, GD_BN 64, 128 or 256, GD_BK 16 or 32
//   GD_WM GD_WN                  wavefronts along m and n; a wavefront's part of the tile is whole 32 x 32 MFMA tiles
//   GD_GROUP_M                   tile rows per L2 strip
//   GD_RELU                      1: fused max(0, .) epilogue
//
// For 256 x 256 tiles: sixteen wavefronts (4 x 4) of 64 x 64 results = 2 x 2 MFMA tiles of 32 x 32.  What gemm_f32.hip
// spends between global memory and LDS - a float4 per operand and thread in registers, four scattered LDS stores to turn
// a k-contiguous row of A into the k-major tile - is not there: a k-tile is (GD_BM + GD_BN) GD_BK / 256 global_load_lds_dwordx4
// of 1 KiB, dealt round-robin to the wavefronts (one of each operand per wavefront for 256 x 256 tiles), and both tiles
// lie in LDS as they lie in memory.
//
// A in LDS: GD_BM rows of 64 bytes (16 k; 128 bytes with GD_BK 32), no padding; the 16-byte chunk c (four k) of row m
// lies at position c ^ ((m / 4) % 4) (GD_BK 32: c ^ ((m / 2) % 8)).  A lane of an MFMA holds row m = lane % 32 and,
// with one ds_read_b128, the four k of chunk 2 u + lane / 32 (u: the steps of eight k of the k-tile); the sixteen lanes
// that such a read serves in one pass (rows 0-3, 12-15, 20-27 of a 32-row block, then the rest) then fall on sixteen
// different groups of four banks.  The swizzle is applied on the source side of the load: lane i of a block writes 16
// bytes at 16 i, that is position i % 4 of row i / 4 (i % 8 of row i / 8), and fetches the chunk that belongs there.
// B in LDS: GD_BK rows (k) of GD_BN floats, as in memory (a 1 KiB block is 256 / GD_BN rows); a lane reads one float of row k
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
#if (GD_M % GD_BM) || (GD_N % GD_BN) || (GD_K % GD_BK) || (GD_BK != 16 && GD_BK != 32)
#error "gemm_f32_d2l: whole tiles only"
#endif
#if (GD_BM % 64) || (GD_BN != 64 && GD_BN != 128 && GD_BN != 256) || (GD_BM % (32 * GD_WM)) || (GD_BN % (32 * GD_WN))
#error "gemm_f32_d2l: GD_BM is a multiple of 64, GD_BN 64, 128 or 256 (a 1 KiB block is whole rows of the B tile), 32 x 32 MFMA tiles per wavefront"
#endif
#define GD_KT (GD_K / GD_BK)
#define GD_NW (GD_WM * GD_WN)
#define GD_TM (GD_BM / GD_WM / 32)
#define GD_TN (GD_BN / GD_WN / 32)

extern "C" __global__ __launch_bounds__(64 * GD_NW)
void GD_NAME(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C) {
  constexpr int ROW_A = GD_BK * 4, CH = GD_BK / 4;        // bytes and 16-byte chunks of a row of the A tile
  constexpr int SW_SH = GD_BK == 16 ? 2 : 1;              // chunk c of row m lies at c ^ ((m >> SW_SH) % CH)
  constexpr int TILE_A = GD_BM * ROW_A, TILE_B = GD_BN * ROW_A;  // bytes of the operand tiles
  constexpr int B_AT = 2 * TILE_A;                        // A's two buffers, then B's two
  constexpr int ROW_B = GD_BN * 4;                        // bytes of a row (k) of the B tile
  constexpr int BLK_A = TILE_A / 1024, BLK = (TILE_A + TILE_B) / 1024;   // 1 KiB blocks of the A tile, of both tiles
  constexpr int STEPS = GD_BK / 8;                        // MFMA steps of eight k (four MFMAs per tile pair) per k-tile
  __shared__ __attribute__((aligned(1024))) char kcg_smem[2 * TILE_A + 2 * TILE_B];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int wm = wave / GD_WN, wn = wave % GD_WN;
  const int l32 = lane & 31, lh = lane >> 5;

  const int tiles_m = GD_M / GD_BM, tiles_n = GD_N / GD_BN;
  int tile_m, tile_n;
  kcg_tile_coords(blockIdx.x, tiles_m, tiles_n, GD_GROUP_M, tile_m, tile_n);
  // (the division in kcg_tile_coords runs on the vector unit: the tile origins go back into scalar registers here, the
  // load instructions below take their base addresses from there)
  const int m0 = __builtin_amdgcn_readfirstlane(tile_m * GD_BM), n0 = __builtin_amdgcn_readfirstlane(tile_n * GD_BN);
  const long batch = blockIdx.y;
  A += batch * (long)GD_M * GD_K;
  B += batch * (long)GD_K * GD_N;
  C += batch * (long)GD_M * GD_N;

  // ---- loads: block b of a k-tile's BLK blocks of 1 KiB (A's sixteen-row groups, then B's groups of 256 / GD_BN rows)
  //      is moved by wavefront b % GD_NW ----
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)kcg_smem;
  // (GD_BK 32: a block is eight rows, and the rows of an odd block are swizzled with 4 more: byte offset ^ 64)
  const unsigned a_lane = (unsigned)(lane / CH) * (unsigned)(GD_K * 4) + (unsigned)(((lane % CH) ^ ((lane >> 4) & 3)) * 16);
  const unsigned b_lane = (unsigned)(lane / (GD_BN / 4)) * (unsigned)(GD_N * 4) + (unsigned)(lane % (GD_BN / 4)) * 16u;
  const char* tileA = (const char*)(A + (long)m0 * GD_K);
  const char* tileB = (const char*)(B + n0);
  auto dma = [&](int kt, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int x = 0; x < (BLK + GD_NW - 1) / GD_NW; ++x) {
      const int blk = wave_u + x * GD_NW;                  // wave-uniform
      if (BLK % GD_NW == 0 || blk < BLK) {
        const bool is_a = blk < BLK_A;
        const int bb = blk - BLK_A;                        // B: rows bb * (1024 / ROW_B) .. of the k-tile
        unsigned dst = lds_base + (is_a ? (unsigned)(buf * TILE_A + blk * 1024) : (unsigned)(B_AT + buf * TILE_B + bb * 1024));
        dst = __builtin_amdgcn_readfirstlane(dst);
        const char* src = is_a ? tileA + (long)blk * (1024 / ROW_A) * GD_K * 4 + (long)kt * ROW_A
                               : tileB + ((long)kt * GD_BK + (long)bb * (1024 / ROW_B)) * GD_N * 4;
        const unsigned lane_off = is_a ? (GD_BK == 32 ? a_lane ^ (unsigned)((blk & 1) * 64) : a_lane) : b_lane;
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(lane_off), "s"(src), "s"(dst) : "memory");
      }
    }
  };

  // ---- fragments of half u of the tile in buffer buf ----
  const int ma = wm * (GD_TM * 32) + l32;                  // the lane's row of A's first block; the next are 32 further each
  const int sw = (ma >> SW_SH) & (CH - 1);                 // the same for every block: 32 rows further changes nothing
  const char* fA = kcg_smem + ma * ROW_A;
  const char* fB = kcg_smem + B_AT + lh * 4 * ROW_B + (wn * (GD_TN * 32) + l32) * 4;
  auto read_fragments = [&](int buf, int u, kcg_f32x4 (&a)[GD_TM], float (&b)[GD_TN][4]) __attribute__((always_inline)) {
    const int pos = ((2 * u + lh) ^ sw) * 16;
#pragma unroll
    for (int i = 0; i < GD_TM; ++i) a[i] = *(const kcg_f32x4*)(fA + buf * TILE_A + i * 32 * ROW_A + pos);
#pragma unroll
    for (int j = 0; j < GD_TN; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) b[j][e] = *(const float*)(fB + buf * TILE_B + (8 * u + e) * ROW_B + j * 128);
  };

  kcg_f32x16 acc[GD_TM][GD_TN];
#pragma unroll
  for (int i = 0; i < GD_TM; ++i)
#pragma unroll
    for (int j = 0; j < GD_TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // ---- prologue: tile 0 into buffer 0, wait, first fragments ----
  dma(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);                      // vmcnt(0)
  __syncthreads();
  kcg_f32x4 fa[2][GD_TM];
  float fb[2][GD_TN][4];
  read_fragments(0, 0, fa[0], fb[0]);

  auto half = [&](kcg_f32x4 (&a)[GD_TM], float (&b)[GD_TN][4]) __attribute__((always_inline)) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int i = 0; i < GD_TM; ++i)
#pragma unroll
        for (int j = 0; j < GD_TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][e], b[j][e], acc[i][j], 0, 0, 0);
  };
  auto tile = [&](const int kt, auto par_c) {
    constexpr int par = decltype(par_c)::v ? 1 : 0;
    const bool more = kt + 1 < GD_KT;
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
    for (; kt + 1 < GD_KT; kt += 2) {
      tile(kt, KcgBool32d<false>{});
      tile(kt + 1, KcgBool32d<true>{});
    }
    if (kt < GD_KT) tile(kt, KcgBool32d<false>{});
  }

  // ---- epilogue: lane l, register v -> row 8*(v/4) + 4*(l/32) + v%4, column l%32 ----
#pragma unroll
  for (int i = 0; i < GD_TM; ++i)
#pragma unroll
    for (int j = 0; j < GD_TN; ++j) {
      const int col = n0 + wn * (GD_TN * 32) + j * 32 + l32;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * (GD_TM * 32) + i * 32 + 8 * (v / 4) + 4 * lh + (v % 4);
        float o = acc[i][j][v];
#if GD_RELU
        o = fmaxf(0.0f, o);
#endif
        C[(long)row * GD_N + col] = o;
      }
    }
}
#undef GD_KT
#undef GD_NW
#undef GD_TM
#undef GD_TN
