// ---- bf16 GEMM / batched GEMM on v_mfma_f32_32x32x16_bf16 --------------------
// C[b] = op(A[b]) * op(B[b]); bf16 operands, fp32 accumulate, fp32 or bf16 out.
// Parameters:
//   GB_NAME   kernel symbol
//   GB_M GB_N GB_K GB_BATCH      problem (row-major, dense, static)
//   GB_TA / GB_TB                1: operand stored column-major (A as [K][M], B as [N][K])
//   GB_BM GB_BN GB_BK            workgroup tile, GB_BK a multiple of 16
//   GB_WM GB_WN                  wavefronts along M and N; block = 64*GB_WM*GB_WN
//   GB_GROUP_M                   tile rows per L2 strip
//   GB_EDGE                      1: ragged tiles, guard loads and stores
//   GB_OUT_BF16                  1: C is bf16, else fp32
//
// One v_mfma_f32_32x32x16_bf16 takes per lane eight consecutive-k values of
// row (A) / column (B) lane%32, k group lane/32.  Both LDS tiles are therefore
// kept "k-contiguous": sA[m][k], sB[n][k], one 16-byte chunk per ds_read_b128.
// Rows are padded by 16 bytes (row stride = 2*GB_BK + 16): 16 consecutive rows
// at one chunk column then start in 16 different groups of 4 banks, so the
// fragment reads, the 16-byte stores of a k-contiguous operand and the
// transposed stores of the other layout are all conflict free.
// An operand whose global layout is contiguous along m or n (A column-major,
// B row-major) is transposed on the way in: each lane loads an 8(k) x 8(m|n)
// block as eight 16-byte rows, transposes it in registers with byte permutes
// and stores eight 16-byte k-chunks.
#ifndef KCG_GEMM16_HELPERS
#define KCG_GEMM16_HELPERS
typedef unsigned short kcg_u16;

// 16-byte chunks, contiguous along k in global memory.  Tile rows x BK.
template <int ROWS, int BK, int NT, bool GUARD>
struct KcgKLoader {
  static constexpr int CPR = BK / 8;
  static constexpr int CHUNKS = ROWS * CPR;
  static constexpr int PER = (CHUNKS + NT - 1) / NT;
  kcg_u32x4 r[PER];
  __device__ __forceinline__ void load(const kcg_u16* __restrict__ g, long ld, int row0, int k0,
                                       int row_lim, int k_lim, int tid) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = i * NT + tid;
      kcg_u32x4 v = {0u, 0u, 0u, 0u};
      if (CHUNKS % NT == 0 || q < CHUNKS) {
        const int rr = q / CPR, c = q % CPR;
        const kcg_u16* p = g + (long)(row0 + rr) * ld + (k0 + c * 8);
        if (!GUARD) {
          v = *(const kcg_u32x4*)p;
        } else if (row0 + rr < row_lim) {
          kcg_u16 t[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) t[j] = (k0 + c * 8 + j < k_lim) ? p[j] : (kcg_u16)0;
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = (unsigned)t[2 * j] | ((unsigned)t[2 * j + 1] << 16);
        }
      }
      r[i] = v;
    }
  }
  __device__ __forceinline__ void store(char* s, int row_bytes, int tid) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = i * NT + tid;
      if (CHUNKS % NT == 0 || q < CHUNKS) {
        const int rr = q / CPR, c = q % CPR;
        *(kcg_u32x4*)(s + rr * row_bytes + c * 16) = r[i];
      }
    }
  }
};

// 8(k) x 8(m|n) blocks, contiguous along m|n in global memory, transposed in
// registers.  Tile is COLS (m|n) x BK.
template <int COLS, int BK, int NT, bool GUARD>
struct KcgTLoader {
  static constexpr int KB = BK / 8;
  static constexpr int BLOCKS = KB * (COLS / 8);
  static constexpr int PER = (BLOCKS + NT - 1) / NT;
  kcg_u32x4 r[PER][8];
  __device__ __forceinline__ void load(const kcg_u16* __restrict__ g, long ld, int col0, int k0,
                                       int col_lim, int k_lim, int tid) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = i * NT + tid;
      const int kb = q % KB, cb = q / KB;
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) {
        kcg_u32x4 v = {0u, 0u, 0u, 0u};
        if (BLOCKS % NT == 0 || q < BLOCKS) {
          const int k = k0 + kb * 8 + kk;
          const kcg_u16* p = g + (long)k * ld + (col0 + cb * 8);
          if (!GUARD) {
            v = *(const kcg_u32x4*)p;
          } else if (k < k_lim) {
            kcg_u16 t[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) t[j] = (col0 + cb * 8 + j < col_lim) ? p[j] : (kcg_u16)0;
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = (unsigned)t[2 * j] | ((unsigned)t[2 * j + 1] << 16);
          }
        }
        r[i][kk] = v;
      }
    }
  }
  __device__ __forceinline__ void store(char* s, int row_bytes, int tid) const {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int q = i * NT + tid;
      if (BLOCKS % NT == 0 || q < BLOCKS) {
        const int kb = q % KB, cb = q / KB;
#pragma unroll
        for (int c = 0; c < 8; ++c) {
          // column c of the block: halves c%2 of dword c/2 of each of the 8 k rows
          kcg_u32x4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const unsigned lo = r[i][2 * e][c / 2], hi = r[i][2 * e + 1][c / 2];
            o[e] = (c & 1) ? __builtin_amdgcn_perm(hi, lo, 0x07060302u)
                           : __builtin_amdgcn_perm(hi, lo, 0x05040100u);
          }
          *(kcg_u32x4*)(s + (cb * 8 + c) * row_bytes + kb * 16) = o;
        }
      }
    }
  }
};
#endif  // KCG_GEMM16_HELPERS

#define GB_NT (64 * GB_WM * GB_WN)
#define GB_WTM (GB_BM / GB_WM)
#define GB_WTN (GB_BN / GB_WN)
#define GB_TM (GB_WTM / 32)
#define GB_TN (GB_WTN / 32)
#define GB_ROWB (GB_BK * 2 + 16)
#define GB_KT ((GB_K + GB_BK - 1) / GB_BK)
#define GB_GUARD ((GB_EDGE != 0) | ((GB_K % 8) != 0) | ((GB_TA != 0) & ((GB_M % 8) != 0)) | ((GB_TB == 0) & ((GB_N % 8) != 0)))

#if (GB_BM % (32 * GB_WM)) || (GB_BN % (32 * GB_WN)) || (GB_BK % 16)
#error "tile shape does not divide into 32x32x16 MFMA tiles"
#endif

extern "C" __global__ __launch_bounds__(GB_NT)
void GB_NAME(const kcg_u16* __restrict__ A, const kcg_u16* __restrict__ B,
#if GB_OUT_BF16
             kcg_u16* __restrict__ C
#else
             float* __restrict__ C
#endif
) {
  __shared__ __attribute__((aligned(16))) char kcg_smem[2 * (GB_BM + GB_BN) * GB_ROWB];
  char* sA = kcg_smem;                                  // [2][GB_BM][GB_ROWB]
  char* sB = kcg_smem + 2 * GB_BM * GB_ROWB;            // [2][GB_BN][GB_ROWB]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / GB_WN;
  const int wn = wave % GB_WN;
  const int l32 = lane & 31;
  const int lh = lane >> 5;

  const int tiles_m = (GB_M + GB_BM - 1) / GB_BM;
  const int tiles_n = (GB_N + GB_BN - 1) / GB_BN;
  int tile_m, tile_n;
  kcg_tile_coords(blockIdx.x, tiles_m, tiles_n, GB_GROUP_M, tile_m, tile_n);
  const int m0 = tile_m * GB_BM;
  const int n0 = tile_n * GB_BN;
  const long batch = blockIdx.y;
  A += batch * (long)GB_M * GB_K;
  B += batch * (long)GB_K * GB_N;
  C += batch * (long)GB_M * GB_N;

#if GB_TA == 0
  KcgKLoader<GB_BM, GB_BK, GB_NT, GB_GUARD> la;
#define GB_LOAD_A(k0) la.load(A, GB_K, m0, (k0), GB_M, GB_K, tid)
#else
  KcgTLoader<GB_BM, GB_BK, GB_NT, GB_GUARD> la;
#define GB_LOAD_A(k0) la.load(A, GB_M, m0, (k0), GB_M, GB_K, tid)
#endif
#if GB_TB == 1
  KcgKLoader<GB_BN, GB_BK, GB_NT, GB_GUARD> lb;
#define GB_LOAD_B(k0) lb.load(B, GB_K, n0, (k0), GB_N, GB_K, tid)
#else
  KcgTLoader<GB_BN, GB_BK, GB_NT, GB_GUARD> lb;
#define GB_LOAD_B(k0) lb.load(B, GB_N, n0, (k0), GB_N, GB_K, tid)
#endif

  kcg_f32x16 acc[GB_TM][GB_TN];
#pragma unroll
  for (int i = 0; i < GB_TM; ++i)
#pragma unroll
    for (int j = 0; j < GB_TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  GB_LOAD_A(0);
  GB_LOAD_B(0);
  la.store(sA, GB_ROWB, tid);
  lb.store(sB, GB_ROWB, tid);
  __syncthreads();

  for (int kt = 0; kt < GB_KT; ++kt) {
    const int buf = kt & 1;
    const char* cA = sA + buf * (GB_BM * GB_ROWB) + (wm * GB_WTM + l32) * GB_ROWB + lh * 16;
    const char* cB = sB + buf * (GB_BN * GB_ROWB) + (wn * GB_WTN + l32) * GB_ROWB + lh * 16;
    if (kt + 1 < GB_KT) {
      GB_LOAD_A((kt + 1) * GB_BK);
      GB_LOAD_B((kt + 1) * GB_BK);
    }

#pragma unroll
    for (int ks = 0; ks < GB_BK / 16; ++ks) {
      kcg_bf16x8 fa[GB_TM], fb[GB_TN];
#pragma unroll
      for (int i = 0; i < GB_TM; ++i) fa[i] = *(const kcg_bf16x8*)(cA + i * 32 * GB_ROWB + ks * 32);
#pragma unroll
      for (int j = 0; j < GB_TN; ++j) fb[j] = *(const kcg_bf16x8*)(cB + j * 32 * GB_ROWB + ks * 32);
#pragma unroll
      for (int i = 0; i < GB_TM; ++i)
#pragma unroll
        for (int j = 0; j < GB_TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }

    if (kt + 1 < GB_KT) {
      la.store(sA + (buf ^ 1) * (GB_BM * GB_ROWB), GB_ROWB, tid);
      lb.store(sB + (buf ^ 1) * (GB_BN * GB_ROWB), GB_ROWB, tid);
    }
    __syncthreads();
  }

  // ---- epilogue: lane l, register v -> row 8*(v/4) + 4*(l/32) + v%4, column l%32 ----
#pragma unroll
  for (int i = 0; i < GB_TM; ++i)
#pragma unroll
    for (int j = 0; j < GB_TN; ++j) {
      const int col = n0 + wn * GB_WTN + j * 32 + l32;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * GB_WTM + i * 32 + 8 * (v / 4) + 4 * lh + (v % 4);
#if GB_EDGE
        if (row < GB_M && col < GB_N)
#endif
        {
#if GB_OUT_BF16
          C[(long)row * GB_N + col] = (kcg_u16)kcg_f32_to_bf16_bits(acc[i][j][v]);
#else
          C[(long)row * GB_N + col] = acc[i][j][v];
#endif
        }
      }
    }
}
#undef GB_LOAD_A
#undef GB_LOAD_B
#undef GB_NT
#undef GB_WTM
#undef GB_WTN
#undef GB_TM
#undef GB_TN
#undef GB_ROWB
#undef GB_KT
#undef GB_GUARD
