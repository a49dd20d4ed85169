// ---- fp64 GEMM / batched GEMM on v_mfma_f64_16x16x4_f64 ---------------------
// C[b] = op(A[b]) * op(B[b]), fp64 in, fp64 MFMA, fp64 out.
// Parameters:
//   GD_NAME   kernel symbol
//   GD_M GD_N GD_K GD_BATCH      problem (row-major, dense, static)
//   GD_TA / GD_TB                1: operand stored column-major (A as [K][M], B as [N][K])
//   GD_BM GD_BN GD_BK            workgroup tile; GD_BK a multiple of 8
//   GD_WM GD_WN                  wavefronts along M and N; block = 64*GD_WM*GD_WN
//   GD_GROUP_M                   tile rows per L2 strip
//   GD_EDGE                      1: some tile is ragged, guard loads and stores
//   GD_RELU                      1: fused max(0, .) epilogue
//
// LDS holds both operand tiles k-major, sA[k][m] and sB[k][n], double buffered.  One v_mfma_f64_16x16x4_f64 takes,
// per lane, A[m = lane%16][k = lane/16] and B[k = lane/16][n = lane%16]: with k-major tiles the 16 lanes of a quarter
// wave read 16 consecutive doubles.  Rows are padded by 16 doubles, which puts the rows of neighbouring k (the other
// quarter of a half-wave's 8-byte read) on the other half of the banks.
// Lane l, accumulator register v of a 16x16 tile hold row l/16 + 4*v, column l%16 (probed on the device: the
// installation's headers do not say).
#define GD_NT (64 * GD_WM * GD_WN)
#define GD_WTM (GD_BM / GD_WM)
#define GD_WTN (GD_BN / GD_WN)
#define GD_TM (GD_WTM / 16)
#define GD_TN (GD_WTN / 16)
#define GD_LDA_S (GD_BM + 16)
#define GD_LDB_S (GD_BN + 16)
#define GD_KT ((GD_K + GD_BK - 1) / GD_BK)
#define GD_AV ((GD_BM * GD_BK / 2 + GD_NT - 1) / GD_NT)
#define GD_BV ((GD_BN * GD_BK / 2 + GD_NT - 1) / GD_NT)

#if (GD_BM % (16 * GD_WM)) || (GD_BN % (16 * GD_WN)) || (GD_BK % 8)
#error "tile shape does not divide into 16x16 MFMA tiles"
#endif

typedef double kcg_f64x2 __attribute__((ext_vector_type(2)));
typedef double kcg_f64x4 __attribute__((ext_vector_type(4)));

extern "C" __global__ __launch_bounds__(GD_NT)
void GD_NAME(const double* __restrict__ A, const double* __restrict__ B, double* __restrict__ C) {
  __shared__ __attribute__((aligned(16))) double sA[2][GD_BK][GD_LDA_S];
  __shared__ __attribute__((aligned(16))) double sB[2][GD_BK][GD_LDB_S];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / GD_WN;
  const int wn = wave % GD_WN;
  const int l16 = lane & 15;
  const int lq = lane >> 4;

  const int tiles_m = (GD_M + GD_BM - 1) / GD_BM;
  const int tiles_n = (GD_N + GD_BN - 1) / GD_BN;
  int tile_m, tile_n;
  kcg_tile_coords(blockIdx.x, tiles_m, tiles_n, GD_GROUP_M, tile_m, tile_n);
  const int m0 = tile_m * GD_BM;
  const int n0 = tile_n * GD_BN;
  const long batch = blockIdx.y;
  A += batch * (long)GD_M * GD_K;
  B += batch * (long)GD_K * GD_N;
  C += batch * (long)GD_M * GD_N;

  kcg_f64x2 ra[GD_AV], rb[GD_BV];

  // ---- global -> registers (one k-tile of A and of B), 16 bytes = two doubles per load ----
  auto load_tiles = [&](int k0) {
#pragma unroll
    for (int i = 0; i < GD_AV; ++i) {
      const int q = i * GD_NT + tid;
      kcg_f64x2 v = {0.0, 0.0};
      if (q < GD_BM * GD_BK / 2) {
#if GD_TA == 0
        const int r = q / (GD_BK / 2), kc = (q % (GD_BK / 2)) * 2;   // 2 along k
        const double* p = A + (long)(m0 + r) * GD_K + (k0 + kc);
#if GD_EDGE || (GD_K % 2)
        if (m0 + r < GD_M) {
#pragma unroll
          for (int j = 0; j < 2; ++j) if (k0 + kc + j < GD_K) v[j] = p[j];
        }
#else
        v = *(const kcg_f64x2*)p;
#endif
#else
        const int kk = q / (GD_BM / 2), mc = (q % (GD_BM / 2)) * 2;   // 2 along m
        const double* p = A + (long)(k0 + kk) * GD_M + (m0 + mc);
#if GD_EDGE || (GD_M % 2)
        if (k0 + kk < GD_K) {
#pragma unroll
          for (int j = 0; j < 2; ++j) if (m0 + mc + j < GD_M) v[j] = p[j];
        }
#else
        v = *(const kcg_f64x2*)p;
#endif
#endif
      }
      ra[i] = v;
    }
#pragma unroll
    for (int i = 0; i < GD_BV; ++i) {
      const int q = i * GD_NT + tid;
      kcg_f64x2 v = {0.0, 0.0};
      if (q < GD_BN * GD_BK / 2) {
#if GD_TB == 0
        const int kk = q / (GD_BN / 2), nc = (q % (GD_BN / 2)) * 2;   // 2 along n
        const double* p = B + (long)(k0 + kk) * GD_N + (n0 + nc);
#if GD_EDGE || (GD_N % 2)
        if (k0 + kk < GD_K) {
#pragma unroll
          for (int j = 0; j < 2; ++j) if (n0 + nc + j < GD_N) v[j] = p[j];
        }
#else
        v = *(const kcg_f64x2*)p;
#endif
#else
        const int r = q / (GD_BK / 2), kc = (q % (GD_BK / 2)) * 2;   // 2 along k
        const double* p = B + (long)(n0 + r) * GD_K + (k0 + kc);
#if GD_EDGE || (GD_K % 2)
        if (n0 + r < GD_N) {
#pragma unroll
          for (int j = 0; j < 2; ++j) if (k0 + kc + j < GD_K) v[j] = p[j];
        }
#else
        v = *(const kcg_f64x2*)p;
#endif
#endif
      }
      rb[i] = v;
    }
  };

  // ---- registers -> LDS ----
  auto store_tiles = [&](int buf) {
#pragma unroll
    for (int i = 0; i < GD_AV; ++i) {
      const int q = i * GD_NT + tid;
      if (q < GD_BM * GD_BK / 2) {
#if GD_TA == 0
        const int r = q / (GD_BK / 2), kc = (q % (GD_BK / 2)) * 2;
#pragma unroll
        for (int j = 0; j < 2; ++j) sA[buf][kc + j][r] = ra[i][j];
#else
        const int kk = q / (GD_BM / 2), mc = (q % (GD_BM / 2)) * 2;
        *(kcg_f64x2*)&sA[buf][kk][mc] = ra[i];
#endif
      }
    }
#pragma unroll
    for (int i = 0; i < GD_BV; ++i) {
      const int q = i * GD_NT + tid;
      if (q < GD_BN * GD_BK / 2) {
#if GD_TB == 0
        const int kk = q / (GD_BN / 2), nc = (q % (GD_BN / 2)) * 2;
        *(kcg_f64x2*)&sB[buf][kk][nc] = rb[i];
#else
        const int r = q / (GD_BK / 2), kc = (q % (GD_BK / 2)) * 2;
#pragma unroll
        for (int j = 0; j < 2; ++j) sB[buf][kc + j][r] = rb[i][j];
#endif
      }
    }
  };

  kcg_f64x4 acc[GD_TM][GD_TN];
#pragma unroll
  for (int i = 0; i < GD_TM; ++i)
#pragma unroll
    for (int j = 0; j < GD_TN; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.0;

  load_tiles(0);
  store_tiles(0);
  __syncthreads();

  // fragments of one k-step (four k values: lane quarter lq takes k = kk + lq) of the tile in LDS buffer `buf`
  double fa[2][GD_TM], fb[2][GD_TN];
  auto read_fragments = [&](int buf, int kk, double (&a)[GD_TM], double (&b)[GD_TN]) {
#pragma unroll
    for (int i = 0; i < GD_TM; ++i) a[i] = sA[buf][kk + lq][wm * GD_WTM + i * 16 + l16];
#pragma unroll
    for (int j = 0; j < GD_TN; ++j) b[j] = sB[buf][kk + lq][wn * GD_WTN + j * 16 + l16];
  };
  read_fragments(0, 0, fa[0], fb[0]);

  // One k-tile, as in the fp32 kernel: the global loads of the next tile are issued first; the fragments of step
  // s+1 are read while the MFMAs of step s run; the next tile goes into the other LDS buffer one step before the
  // last; the barrier stands before the last step's MFMAs, and the first fragments of the next tile are read behind
  // it.  GD_BK / 4 is even, so the fragment sets keep their roles.
  constexpr int NS = GD_BK / 4;
  for (int kt = 0; kt < GD_KT; ++kt) {
    const int buf = kt & 1;
    const bool more = kt + 1 < GD_KT;
    if (more) load_tiles((kt + 1) * GD_BK);
    __builtin_amdgcn_sched_barrier(0);      // keeps the global loads up here, a whole tile ahead of their LDS stores
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const int cur = s & 1;
      if (s + 1 < NS) {
        read_fragments(buf, 4 * (s + 1), fa[cur ^ 1], fb[cur ^ 1]);
      } else {
        __syncthreads();
        if (more) read_fragments(buf ^ 1, 0, fa[cur ^ 1], fb[cur ^ 1]);
      }
      if (s == NS - 2 && more) store_tiles(buf ^ 1);
#pragma unroll
      for (int i = 0; i < GD_TM; ++i)
#pragma unroll
        for (int j = 0; j < GD_TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[cur][i], fb[cur][j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- epilogue ----
#pragma unroll
  for (int i = 0; i < GD_TM; ++i)
#pragma unroll
    for (int j = 0; j < GD_TN; ++j) {
      const int col = n0 + wn * GD_WTN + j * 16 + l16;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int row = m0 + wm * GD_WTM + i * 16 + lq + 4 * v;
        double o = acc[i][j][v];
#if GD_RELU
        o = o > 0.0 ? o : 0.0;
#endif
#if GD_EDGE
        if (row < GD_M && col < GD_N)
#endif
          C[(long)row * GD_N + col] = o;
      }
    }
}
#undef GD_NT
#undef GD_WTM
#undef GD_WTN
#undef GD_TM
#undef GD_TN
#undef GD_LDA_S
#undef GD_LDB_S
#undef GD_KT
#undef GD_AV
#undef GD_BV
