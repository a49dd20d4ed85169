// ---- fp32 GEMM / batched GEMM on v_mfma_f32_32x32x2_f32 ---------------------
// C[b] = op(A[b]) * op(B[b]), fp32 in, full-precision fp32 MFMA, fp32 out.
// Parameters:
//   GM_NAME   kernel symbol
//   GM_M GM_N GM_K GM_BATCH      problem (row-major, dense, static)
//   GM_TA / GM_TB                1: operand stored column-major (A as [K][M], B as [N][K])
//   GM_BM GM_BN GM_BK            workgroup tile; GM_BK even
//   GM_WM GM_WN                  wavefronts along M and N; block = 64*GM_WM*GM_WN
//   GM_GROUP_M                   tile rows per L2 strip
//   GM_EDGE                      1: some tile is ragged, guard loads and stores
//   GM_RELU                      1: fused max(0, .) epilogue
//
// LDS holds both operand tiles k-major, sA[k][m] and sB[k][n], double buffered.
// One v_mfma_f32_32x32x2_f32 takes, per lane, A[m = lane%32][k = lane/32] and
// B[k = lane/32][n = lane%32]: with k-major tiles the 32 lanes of a half-wave
// read 32 consecutive floats, which is conflict free.  Row padding of 4 floats
// spreads the transposing stores of a k-contiguous operand over the banks.
// Lane l, accumulator register v of a 32x32 tile hold
//   row 8*(v/4) + 4*(l/32) + v%4, column l%32.
#define GM_NT (64 * GM_WM * GM_WN)
#define GM_WTM (GM_BM / GM_WM)
#define GM_WTN (GM_BN / GM_WN)
#define GM_TM (GM_WTM / 32)
#define GM_TN (GM_WTN / 32)
#ifndef GM_PAD
#define GM_PAD 4
#endif
#define GM_LDA_S (GM_BM + GM_PAD)
#define GM_LDB_S (GM_BN + GM_PAD)
#define GM_KT ((GM_K + GM_BK - 1) / GM_BK)
#define GM_AV ((GM_BM * GM_BK / 4 + GM_NT - 1) / GM_NT)
#define GM_BV ((GM_BN * GM_BK / 4 + GM_NT - 1) / GM_NT)

#if (GM_BM % (32 * GM_WM)) || (GM_BN % (32 * GM_WN)) || (GM_BK % 4)
#error "tile shape does not divide into 32x32 MFMA tiles"
#endif

extern "C" __global__ __launch_bounds__(GM_NT)
void GM_NAME(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C) {
  __shared__ __attribute__((aligned(16))) float sA[2][GM_BK][GM_LDA_S];
  __shared__ __attribute__((aligned(16))) float sB[2][GM_BK][GM_LDB_S];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / GM_WN;
  const int wn = wave % GM_WN;
  const int l32 = lane & 31;
  const int lh = lane >> 5;

  const int tiles_m = (GM_M + GM_BM - 1) / GM_BM;
  const int tiles_n = (GM_N + GM_BN - 1) / GM_BN;
  int tile_m, tile_n;
  kcg_tile_coords(blockIdx.x, tiles_m, tiles_n, GM_GROUP_M, tile_m, tile_n);
  const int m0 = tile_m * GM_BM;
  const int n0 = tile_n * GM_BN;
  const long batch = blockIdx.y;
  A += batch * (long)GM_M * GM_K;
  B += batch * (long)GM_K * GM_N;
  C += batch * (long)GM_M * GM_N;

  kcg_f32x4 ra[GM_AV], rb[GM_BV];

  // ---- global -> registers (one k-tile of A and of B) ----
  auto load_tiles = [&](int k0) {
#pragma unroll
    for (int i = 0; i < GM_AV; ++i) {
      const int q = i * GM_NT + tid;
      kcg_f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (q < GM_BM * GM_BK / 4) {
#if GM_TA == 0
        const int r = q / (GM_BK / 4), kc = (q % (GM_BK / 4)) * 4;   // 4 along k
        const float* p = A + (long)(m0 + r) * GM_K + (k0 + kc);
#if GM_EDGE || (GM_K % 4)
        if (m0 + r < GM_M) {
#pragma unroll
          for (int j = 0; j < 4; ++j) if (k0 + kc + j < GM_K) v[j] = p[j];
        }
#else
        v = *(const kcg_f32x4*)p;
#endif
#else
        const int kk = q / (GM_BM / 4), mc = (q % (GM_BM / 4)) * 4;   // 4 along m
        const float* p = A + (long)(k0 + kk) * GM_M + (m0 + mc);
#if GM_EDGE || (GM_M % 4)
        if (k0 + kk < GM_K) {
#pragma unroll
          for (int j = 0; j < 4; ++j) if (m0 + mc + j < GM_M) v[j] = p[j];
        }
#else
        v = *(const kcg_f32x4*)p;
#endif
#endif
      }
      ra[i] = v;
    }
#pragma unroll
    for (int i = 0; i < GM_BV; ++i) {
      const int q = i * GM_NT + tid;
      kcg_f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (q < GM_BN * GM_BK / 4) {
#if GM_TB == 0
        const int kk = q / (GM_BN / 4), nc = (q % (GM_BN / 4)) * 4;   // 4 along n
        const float* p = B + (long)(k0 + kk) * GM_N + (n0 + nc);
#if GM_EDGE || (GM_N % 4)
        if (k0 + kk < GM_K) {
#pragma unroll
          for (int j = 0; j < 4; ++j) if (n0 + nc + j < GM_N) v[j] = p[j];
        }
#else
        v = *(const kcg_f32x4*)p;
#endif
#else
        const int r = q / (GM_BK / 4), kc = (q % (GM_BK / 4)) * 4;   // 4 along k
        const float* p = B + (long)(n0 + r) * GM_K + (k0 + kc);
#if GM_EDGE || (GM_K % 4)
        if (n0 + r < GM_N) {
#pragma unroll
          for (int j = 0; j < 4; ++j) if (k0 + kc + j < GM_K) v[j] = p[j];
        }
#else
        v = *(const kcg_f32x4*)p;
#endif
#endif
      }
      rb[i] = v;
    }
  };

  // ---- registers -> LDS ----
  auto store_tiles = [&](int buf) {
#pragma unroll
    for (int i = 0; i < GM_AV; ++i) {
      const int q = i * GM_NT + tid;
      if (q < GM_BM * GM_BK / 4) {
#if GM_TA == 0
        const int r = q / (GM_BK / 4), kc = (q % (GM_BK / 4)) * 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) sA[buf][kc + j][r] = ra[i][j];
#else
        const int kk = q / (GM_BM / 4), mc = (q % (GM_BM / 4)) * 4;
        *(kcg_f32x4*)&sA[buf][kk][mc] = ra[i];
#endif
      }
    }
#pragma unroll
    for (int i = 0; i < GM_BV; ++i) {
      const int q = i * GM_NT + tid;
      if (q < GM_BN * GM_BK / 4) {
#if GM_TB == 0
        const int kk = q / (GM_BN / 4), nc = (q % (GM_BN / 4)) * 4;
        *(kcg_f32x4*)&sB[buf][kk][nc] = rb[i];
#else
        const int r = q / (GM_BK / 4), kc = (q % (GM_BK / 4)) * 4;
#pragma unroll
        for (int j = 0; j < 4; ++j) sB[buf][kc + j][r] = rb[i][j];
#endif
      }
    }
  };

  kcg_f32x16 acc[GM_TM][GM_TN];
#pragma unroll
  for (int i = 0; i < GM_TM; ++i)
#pragma unroll
    for (int j = 0; j < GM_TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  load_tiles(0);
  store_tiles(0);
  __syncthreads();

  // fragments of one k-step (two k values: lane half lh takes k = kk + lh) of the tile in LDS buffer `buf`
  float fa[2][GM_TM], fb[2][GM_TN];
  auto read_fragments = [&](int buf, int kk, float (&a)[GM_TM], float (&b)[GM_TN]) {
#pragma unroll
    for (int i = 0; i < GM_TM; ++i) a[i] = sA[buf][kk + lh][wm * GM_WTM + i * 32 + l32];
#pragma unroll
    for (int j = 0; j < GM_TN; ++j) b[j] = sB[buf][kk + lh][wn * GM_WTN + j * 32 + l32];
  };
  read_fragments(0, 0, fa[0], fb[0]);

  // One k-tile: the global loads of the next tile are issued first; the fragments of step s+1 are read while
  // the MFMAs of step s run; the next tile goes into the other LDS buffer one step before the last; the
  // barrier stands before the last step's MFMAs, whose fragments are in registers by then, and the first
  // fragments of the next tile are read behind it, so neither the stores nor the barrier nor the first
  // LDS reads of a tile leave the MFMA pipe idle.  GM_BK / 2 is even, so the fragment sets keep their roles.
  constexpr int NS = GM_BK / 2;
  for (int kt = 0; kt < GM_KT; ++kt) {
    const int buf = kt & 1;
    const bool more = kt + 1 < GM_KT;
    if (more) load_tiles((kt + 1) * GM_BK);
    // Without this fence the compiler sinks the global loads down to the LDS stores that use them, and every
    // k-tile ends with the whole workgroup waiting out the memory latency in front of the barrier.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const int cur = s & 1;
      if (s + 1 < NS) {
        read_fragments(buf, 2 * (s + 1), fa[cur ^ 1], fb[cur ^ 1]);
      } else {
        __syncthreads();
        if (more) read_fragments(buf ^ 1, 0, fa[cur ^ 1], fb[cur ^ 1]);
      }
      if (s == (NS >= 2 ? NS - 2 : 0) && more) store_tiles(buf ^ 1);
#pragma unroll
      for (int i = 0; i < GM_TM; ++i)
#pragma unroll
        for (int j = 0; j < GM_TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[cur][i], fb[cur][j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- epilogue ----
#pragma unroll
  for (int i = 0; i < GM_TM; ++i)
#pragma unroll
    for (int j = 0; j < GM_TN; ++j) {
      const int col = n0 + wn * GM_WTN + j * 32 + l32;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * GM_WTM + i * 32 + 8 * (v / 4) + 4 * lh + (v % 4);
        float o = acc[i][j][v];
#if GM_RELU
        o = fmaxf(0.0f, o);
#endif
#if GM_EDGE
        if (row < GM_M && col < GM_N)
#endif
          C[(long)row * GM_N + col] = o;
      }
    }
}
#undef GM_NT
#undef GM_WTM
#undef GM_WTN
#undef GM_TM
#undef GM_TN
#undef GM_PAD
#undef GM_LDA_S
#undef GM_LDB_S
#undef GM_KT
#undef GM_AV
#undef GM_BV
