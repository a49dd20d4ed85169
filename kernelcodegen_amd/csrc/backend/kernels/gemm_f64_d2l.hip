// ---- fp64 GEMM on v_mfma_f64_16x16x4_f64, operand tiles straight from global memory into LDS ----------------------
// C[b] = A[b] * B[b]: A [M][K], B [K][N], C [M][N], all row-major fp64; whole GE_BM x GE_BN x 16 tiles only (the emitter
// falls back to gemm_f64.hip for every other case).  Parameters:
//   GE_NAME                      kernel symbol
//   GE_M GE_N GE_K GE_BATCH      problem: multiples of GE_BM, GE_BN and 16
//   GE_BM GE_BN                  workgroup tile: GE_BM a multiple of 64, GE_BN 128 or 256
//   GE_WM GE_WN                  wavefronts along m and n; a wavefront's part of the tile is whole 16 x 16 MFMA tiles
//   GE_GROUP_M                   tile rows per L2 strip
//   GE_RELU                      1: fused max(0, .) epilogue
//
// The fp32 GEMM's direct-load form (gemm_f32_d2l.hip) in fp64: a k-tile is (GE_BM + GE_BN) / 8 global_load_lds_dwordx4
// of 1 KiB, dealt round-robin to the wavefronts; no staging registers, no LDS stores, and no recombining of B's rows in
// registers: both tiles lie in LDS as they lie in memory.
//
// A in LDS: GE_BM rows of 128 bytes (16 k), no padding; the 16-byte chunk c (two k) of row m lies at position
// c ^ ((m / 2) % 8), applied on the source side of the load.  One v_mfma_f64_16x16x4_f64 takes A[m = lane % 16][k] with
// one k per group of sixteen lanes; which k is free as long as both operands agree: in step (u, e) - u the half of the
// k-tile, e = 0, 1 - lane group q = lane / 16 takes k = 8 u + 2 q + e, so that one ds_read_b128 of chunk 4 u + q serves
// two MFMAs.  The sixteen lanes such a read serves in one pass (0-3 and 12-15 of group 0, 4-11 of group 1, ...) fall on
// sixteen different groups of four banks.
// B in LDS: 16 rows (k) of GE_BN doubles, as in memory, except that in odd rows the halves of every 32 doubles are
// exchanged (byte offset ^ 128 within the row, again on the source side): a fragment read takes one double per lane at
// column n = lane % 16 of two rows k and k + 2 per 32 lanes, whose sixteen doubles otherwise fall on the same banks.
//
// Pipeline: as in gemm_f32_d2l.hip.  One barrier per k-tile, in front of the MFMAs of its last step (of four); behind it
// the first fragments of the next tile; the loads of the tile after next go out at the top of the next tile.  Fragments
// are read one MFMA step ahead (B) and one half ahead (A, whose read serves two steps).
#ifndef KCG_GEMM64D_HELPERS
#define KCG_GEMM64D_HELPERS
template <bool B> struct KcgBool64d { static constexpr bool v = B; };
typedef double kcg_f64x2d __attribute__((ext_vector_type(2)));
typedef double kcg_f64x4d __attribute__((ext_vector_type(4)));
#endif
#if (GE_M % GE_BM) || (GE_N % GE_BN) || (GE_K % 16)
#error "gemm_f64_d2l: whole tiles only"
#endif
#if (GE_BM % 64) || (GE_BN != 128 && GE_BN != 256) || (GE_BM % (16 * GE_WM)) || (GE_BN % (32 * GE_WN))
#error "gemm_f64_d2l: GE_BM is a multiple of 64, GE_BN 128 or 256, 16 x 16 MFMA tiles per wavefront, an even number of them along n"
#endif
#define GE_KT (GE_K / 16)
#define GE_NW (GE_WM * GE_WN)
#define GE_TM (GE_BM / GE_WM / 16)
#define GE_TN (GE_BN / GE_WN / 16)

extern "C" __global__ __launch_bounds__(64 * GE_NW)
void GE_NAME(const double* __restrict__ A, const double* __restrict__ B, double* __restrict__ C) {
  constexpr int ROW_A = 128, ROW_B = GE_BN * 8;           // bytes of a row of the A tile (16 k), of the B tile (one k)
  constexpr int TILE_A = GE_BM * ROW_A, TILE_B = 16 * ROW_B;
  constexpr int B_AT = 2 * TILE_A;                        // A's two buffers, then B's two
  constexpr int BLK_A = TILE_A / 1024, BLK = (TILE_A + TILE_B) / 1024;   // 1 KiB blocks of the A tile, of both tiles
  constexpr int BPR = ROW_B / 1024;                       // blocks per row of the B tile (1 or 2)
  __shared__ __attribute__((aligned(1024))) char kcg_smem[2 * TILE_A + 2 * TILE_B];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int wm = wave / GE_WN, wn = wave % GE_WN;
  const int l16 = lane & 15, lq = lane >> 4;

  const int tiles_m = GE_M / GE_BM, tiles_n = GE_N / GE_BN;
  int tile_m, tile_n;
  kcg_tile_coords(blockIdx.x, tiles_m, tiles_n, GE_GROUP_M, tile_m, tile_n);
  // (the division in kcg_tile_coords runs on the vector unit: the tile origins go back into scalar registers here, the
  // load instructions below take their base addresses from there)
  const int m0 = __builtin_amdgcn_readfirstlane(tile_m * GE_BM), n0 = __builtin_amdgcn_readfirstlane(tile_n * GE_BN);
  const long batch = blockIdx.y;
  A += batch * (long)GE_M * GE_K;
  B += batch * (long)GE_K * GE_N;
  C += batch * (long)GE_M * GE_N;

  // ---- loads: block b of a k-tile's BLK blocks of 1 KiB (A's eight-row groups, then B's rows or half rows) is moved by
  //      wavefront b % GE_NW ----
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)kcg_smem;
  // (A: a block is eight rows; the rows of an odd block are swizzled with 4 more: byte offset ^ 64)
  const unsigned a_lane = (unsigned)(lane >> 3) * (unsigned)(GE_K * 8) + (unsigned)(((lane & 7) ^ ((lane >> 4) & 3)) * 16);
  const unsigned b_lane = (unsigned)lane * 16u;
  const char* tileA = (const char*)(A + (long)m0 * GE_K);
  const char* tileB = (const char*)(B + n0);
  auto dma = [&](int kt, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int x = 0; x < (BLK + GE_NW - 1) / GE_NW; ++x) {
      const int blk = wave_u + x * GE_NW;                  // wave-uniform
      if (BLK % GE_NW == 0 || blk < BLK) {
        const bool is_a = blk < BLK_A;
        const int bb = blk - BLK_A;                        // B: row bb / BPR of the k-tile, part bb % BPR of it
        unsigned dst = lds_base + (is_a ? (unsigned)(buf * TILE_A + blk * 1024) : (unsigned)(B_AT + buf * TILE_B + bb * 1024));
        dst = __builtin_amdgcn_readfirstlane(dst);
        const char* src = is_a ? tileA + (long)blk * 8 * GE_K * 8 + (long)kt * ROW_A
                               : tileB + ((long)kt * 16 + (long)(bb / BPR)) * GE_N * 8 + (long)(bb % BPR) * 1024;
        const unsigned lane_off = is_a ? a_lane ^ (unsigned)((blk & 1) * 64) : b_lane ^ (unsigned)(((bb / BPR) & 1) * 128);
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(lane_off), "s"(src), "s"(dst) : "memory");
      }
    }
  };

  // ---- fragments: A for half u of the tile in buffer buf (two k per lane and 16-row block), B for MFMA step 2 u + e ----
  const int ma = wm * (GE_TM * 16) + l16;                  // the lane's row of A's first block; the next are 16 further each
  const int sw = (ma >> 1) & 7;                            // the same for every block: 16 rows further changes nothing
  const char* fA = kcg_smem + ma * ROW_A;
  const char* fB = kcg_smem + B_AT + lq * 2 * ROW_B + (wn * (GE_TN * 16) + l16) * 8;
  auto read_a = [&](int buf, int u, kcg_f64x2d (&a)[GE_TM]) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < GE_TM; ++i) a[i] = *(const kcg_f64x2d*)(fA + buf * TILE_A + i * 16 * ROW_A + (((4 * u + lq) ^ sw) * 16));
  };
  auto read_b = [&](int buf, int st, double (&b)[GE_TN]) __attribute__((always_inline)) {
    const int u = st >> 1, e = st & 1;   // row 8 u + 2 q + e: odd for e = 1, where the halves of 32 doubles are exchanged
#pragma unroll
    for (int j = 0; j < GE_TN; ++j) b[j] = *(const double*)(fB + buf * TILE_B + (8 * u + e) * ROW_B + ((j * 128) ^ (e * 128)));
  };

  kcg_f64x4d acc[GE_TM][GE_TN];
#pragma unroll
  for (int i = 0; i < GE_TM; ++i)
#pragma unroll
    for (int j = 0; j < GE_TN; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.0;

  // ---- prologue: tile 0 into buffer 0, wait, first fragments ----
  dma(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);                      // vmcnt(0)
  __syncthreads();
  kcg_f64x2d fa[2][GE_TM];
  double fb[2][GE_TN];
  read_a(0, 0, fa[0]);
  read_b(0, 0, fb[0]);

  // MFMA step st = 2 u + e of a tile: A from set u, element e; B from set st % 2.  Fragments are read one step ahead.
  auto step = [&](int st) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < GE_TM; ++i)
#pragma unroll
      for (int j = 0; j < GE_TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[st >> 1][i][st & 1], fb[st & 1][j], acc[i][j], 0, 0, 0);
  };
  auto tile = [&](const int kt, auto par_c) {
    constexpr int par = decltype(par_c)::v ? 1 : 0;
    const bool more = kt + 1 < GE_KT;
    if (more) dma(kt + 1, par ^ 1);                        // the other buffer is free since the last barrier
    __builtin_amdgcn_sched_barrier(0);
    read_b(par, 1, fb[1]);
    step(0);
    __builtin_amdgcn_sched_barrier(0);
    read_a(par, 1, fa[1]);
    read_b(par, 2, fb[0]);
    step(1);
    __builtin_amdgcn_sched_barrier(0);
    read_b(par, 3, fb[1]);
    step(2);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0F70);                    // vmcnt(0): this wavefront's blocks of tile kt+1 have landed
    __syncthreads();                                       // (its wait for LDS covers the last fragment reads of tile kt)
    if (more) {
      read_a(par ^ 1, 0, fa[0]);
      read_b(par ^ 1, 0, fb[0]);
    }
    step(3);
    __builtin_amdgcn_sched_barrier(0);
  };
  {
    int kt = 0;
    for (; kt + 1 < GE_KT; kt += 2) {
      tile(kt, KcgBool64d<false>{});
      tile(kt + 1, KcgBool64d<true>{});
    }
    if (kt < GE_KT) tile(kt, KcgBool64d<false>{});
  }

  // ---- epilogue: lane l, register v -> row l / 16 + 4 v, column l % 16 ----
#pragma unroll
  for (int i = 0; i < GE_TM; ++i)
#pragma unroll
    for (int j = 0; j < GE_TN; ++j) {
      const int col = n0 + wn * (GE_TN * 16) + j * 16 + l16;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int row = m0 + wm * (GE_TM * 16) + i * 16 + lq + 4 * v;
        double o = acc[i][j][v];
#if GE_RELU
        o = o > 0.0 ? o : 0.0;
#endif
        C[(long)row * GE_N + col] = o;
      }
    }
}
#undef GE_KT
#undef GE_NW
#undef GE_TM
#undef GE_TN
