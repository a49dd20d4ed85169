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
// LDS holds both operand tiles with k innermost, sA[m][k] and sB[n][k], rows of GD_BK + 2 doubles, double buffered.
// One v_mfma_f64_16x16x4_f64 takes, per lane, A[m = lane%16][k = lane/16] and B[k = lane/16][n = lane%16]; a fragment
// read is 8 bytes per lane, served 32 lanes at a time.  The 16 lanes of a quarter wave read at a pitch of 9 (BK 16) or 5
// (BK 8) sixteen-byte units, an odd number, which spreads them over all sixteen such units of the banks, and the
// neighbouring k (the other quarter of the half-wave) is the other half of each unit: no conflicts.  An operand that
// is contiguous along k in memory is stored as it lies; one that is contiguous along m / n is loaded two k rows at a
// time and recombined in registers (two doubles of one row become the two k of two rows).  (Both used to lie k-major,
// s[k][m]; a k-contiguous operand was scattered into that form by 8-byte stores that fell eight at a time on the same
// banks, SQ_LDS_BANK_CONFLICT 117 M of 369 M LDS cycles per launch of the 4096^3 product, and the k-major reads
// themselves measured slower than the present ones.)
// Lane l, accumulator register v of a 16x16 tile hold row l/16 + 4*v, column l%16 (probed on the device: the
// installation's headers do not say).
#define GD_NT (64 * GD_WM * GD_WN)
#define GD_WTM (GD_BM / GD_WM)
#define GD_WTN (GD_BN / GD_WN)
#define GD_TM (GD_WTM / 16)
#define GD_TN (GD_WTN / 16)
#define GD_LDK_S (GD_BK + 2)
#define GD_IDX(k, x) ((x) * GD_LDK_S + (k))
#define GD_KT ((GD_K + GD_BK - 1) / GD_BK)

#if (GD_BM % (16 * GD_WM)) || (GD_BN % (16 * GD_WN)) || (GD_BK % 8)
#error "tile shape does not divide into 16x16 MFMA tiles"
#endif

#ifndef KCG_GEMM64_HELPERS
#define KCG_GEMM64_HELPERS
template <int V> struct KcgIntD { static constexpr int v = V; };
#endif
typedef double kcg_f64x2 __attribute__((ext_vector_type(2)));
typedef double kcg_f64x4 __attribute__((ext_vector_type(4)));

extern "C" __global__ __launch_bounds__(GD_NT)
void GD_NAME(const double* __restrict__ A, const double* __restrict__ B, double* __restrict__ C) {
  __shared__ __attribute__((aligned(16))) double sA[2][GD_BM * GD_LDK_S];
  __shared__ __attribute__((aligned(16))) double sB[2][GD_BN * GD_LDK_S];

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

  // One k-tile of an operand on its way from global memory to LDS.  ROWS = extent of the tile along m (A) or n (B), ld =
  // the operand's leading dimension, x0 = the tile's first row / column, xlim = the operand's extent along it.
  //   KC (the operand is contiguous along k): a unit is two consecutive k of one row, 16 bytes, stored as they are.
  //   else (contiguous along m / n): a unit is two consecutive k of two consecutive rows: two 16-byte loads, one from
  //   each k row, recombined into the two k of each row and stored as two 16-byte pieces.
  auto load_operand = [&](auto kc_c, auto rows_c, const double* __restrict__ g, long ld, int x0, int xlim, int k0, auto& regs) {
    constexpr bool KC = decltype(kc_c)::v != 0;
    constexpr int ROWS = decltype(rows_c)::v;
    constexpr int UNITS = KC ? ROWS * GD_BK / 2 : ROWS * GD_BK / 4, PER = (UNITS + GD_NT - 1) / GD_NT;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = i * GD_NT + tid;
      kcg_f64x2 v0 = {0.0, 0.0}, v1 = {0.0, 0.0};
      if (UNITS % GD_NT == 0 || q < UNITS) {
        if (KC) {
          const int r = q / (GD_BK / 2), kc = (q % (GD_BK / 2)) * 2;
          const double* p = g + (long)(x0 + r) * ld + (k0 + kc);
          if (GD_EDGE || (GD_K % 2)) {
            if (x0 + r < xlim) {
#pragma unroll
              for (int j = 0; j < 2; ++j) if (k0 + kc + j < GD_K) v0[j] = p[j];
            }
          } else {
            v0 = *(const kcg_f64x2*)p;
          }
        } else {
          const int kp = q / (ROWS / 2), xc = (q % (ROWS / 2)) * 2;
          const double* p = g + (long)(k0 + 2 * kp) * ld + (x0 + xc);
          if (GD_EDGE || (GD_K % 2) || (ld % 2)) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              if (x0 + xc + j < xlim && k0 + 2 * kp < GD_K) v0[j] = p[j];
              if (x0 + xc + j < xlim && k0 + 2 * kp + 1 < GD_K) v1[j] = p[ld + j];
            }
          } else {
            v0 = *(const kcg_f64x2*)p;
            v1 = *(const kcg_f64x2*)(p + ld);
          }
        }
      }
      regs[i][0] = v0;
      if (!KC) regs[i][1] = v1;
    }
  };
  auto store_operand = [&](auto kc_c, auto rows_c, double* s, const auto& regs) {
    constexpr bool KC = decltype(kc_c)::v != 0;
    constexpr int ROWS = decltype(rows_c)::v;
    constexpr int UNITS = KC ? ROWS * GD_BK / 2 : ROWS * GD_BK / 4, PER = (UNITS + GD_NT - 1) / GD_NT;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = i * GD_NT + tid;
      if (UNITS % GD_NT == 0 || q < UNITS) {
        if (KC) {
          const int r = q / (GD_BK / 2), kc = (q % (GD_BK / 2)) * 2;
          *(kcg_f64x2*)&s[GD_IDX(kc, r)] = regs[i][0];
        } else {
          const int kp = q / (ROWS / 2), xc = (q % (ROWS / 2)) * 2;
          const kcg_f64x2 lo = {regs[i][0][0], regs[i][1][0]}, hi = {regs[i][0][1], regs[i][1][1]};
          *(kcg_f64x2*)&s[GD_IDX(2 * kp, xc)] = lo;
          *(kcg_f64x2*)&s[GD_IDX(2 * kp, xc + 1)] = hi;
        }
      }
    }
  };
  constexpr bool A_KC = GD_TA == 0, B_KC = GD_TB != 0;
  constexpr int A_PER = ((A_KC ? GD_BM * GD_BK / 2 : GD_BM * GD_BK / 4) + GD_NT - 1) / GD_NT;
  constexpr int B_PER = ((B_KC ? GD_BN * GD_BK / 2 : GD_BN * GD_BK / 4) + GD_NT - 1) / GD_NT;
  kcg_f64x2 ra[A_PER][A_KC ? 1 : 2], rb[B_PER][B_KC ? 1 : 2];
  auto load_tiles = [&](int k0) {
    load_operand(KcgIntD<A_KC>{}, KcgIntD<GD_BM>{}, A, GD_TA ? GD_M : GD_K, m0, GD_M, k0, ra);
    load_operand(KcgIntD<B_KC>{}, KcgIntD<GD_BN>{}, B, GD_TB ? GD_K : GD_N, n0, GD_N, k0, rb);
  };
  auto store_tiles = [&](int buf) {
    store_operand(KcgIntD<A_KC>{}, KcgIntD<GD_BM>{}, sA[buf], ra);
    store_operand(KcgIntD<B_KC>{}, KcgIntD<GD_BN>{}, sB[buf], rb);
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
    for (int i = 0; i < GD_TM; ++i) a[i] = sA[buf][GD_IDX(kk + lq, wm * GD_WTM + i * 16 + l16)];
#pragma unroll
    for (int j = 0; j < GD_TN; ++j) b[j] = sB[buf][GD_IDX(kk + lq, wn * GD_WTN + j * 16 + l16)];
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
#undef GD_LDK_S
#undef GD_IDX
#undef GD_KT
