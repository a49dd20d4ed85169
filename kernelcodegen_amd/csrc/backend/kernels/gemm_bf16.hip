// ---- bf16 GEMM / batched GEMM on v_mfma_f32_32x32x16_bf16 --------------------
// C[b] = op(A[b]) * op(B[b]); bf16 operands, fp32 accumulate, fp32 or bf16 out.
// Parameters:
//   GB_NAME   kernel symbol
//   GB_M GB_N GB_K GB_BATCH      problem (row-major, dense, static)
//   GB_TA / GB_TB                1: operand stored column-major (A as [K][M], B as [N][K])
//   GB_BM GB_BN GB_BK            workgroup tile, GB_BK a multiple of 16
//   GB_WM GB_WN                  wavefronts along M and N; block = 64*GB_WM*GB_WN
//   GB_GROUP_M                   tile rows per L2 strip
//   GB_STAGES                    1 or 2 sets of staging registers = tiles in flight from global memory
//   GB_INTERLEAVE                1: deal each k-step's memory instructions out between its MFMAs
//   GB_EDGE                      1: ragged tiles, guard loads and stores
//   GB_OUT_BF16                  1: C is bf16, else fp32
//   GB_RELU                      1: fused max(0, .) epilogue
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
#ifndef KCG_TL_LINES
#define KCG_TL_LINES 1
#endif
typedef unsigned short kcg_u16;
template <bool B> struct KcgBool { static constexpr bool v = B; };

// 16-byte chunks, contiguous along k in global memory.  Tile rows x BK.
// One unit = one chunk per lane.
template <int ROWS, int BK, int NT, bool GUARD>
struct KcgKLoader {
  static constexpr int CPR = BK / 8;
  static constexpr int CHUNKS = ROWS * CPR;
  static constexpr int PER = (CHUNKS + NT - 1) / NT;
  static constexpr int WEIGHT = 1;                    // feeding work of one unit, in 16-byte loads
  kcg_u32x4 r[PER];
  __device__ __forceinline__ void load_unit(int i, const kcg_u16* __restrict__ g, long ld, int row0, int k0,
                                            int row_lim, int k_lim, int tid) {
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
  __device__ __forceinline__ void store_unit(int i, char* s, int row_bytes, int tid) const {
    const int q = i * NT + tid;
    if (CHUNKS % NT == 0 || q < CHUNKS) {
      const int rr = q / CPR, c = q % CPR;
      *(kcg_u32x4*)(s + rr * row_bytes + c * 16) = r[i];
    }
  }
};

// KR(k) x 8(m|n) blocks, contiguous along m|n in global memory, transposed in
// registers.  Tile is COLS (m|n) x BK.  KR = 8: a lane owns a whole 8x8 block
// and writes eight 16-byte k-chunks; KR = 4 (chosen when there is at most one
// 8x8 block per lane): a lane owns half a block and writes eight 8-byte halves.
// One unit = one block (or half block) per lane.
template <int COLS, int BK, int NT, bool GUARD>
struct KcgTLoader {
  static constexpr int KR = ((BK / 8) * (COLS / 8) > NT) ? 8 : 4;
  static constexpr int WEIGHT = KR;                   // feeding work of one unit, in 16-byte loads
  static constexpr int KB = BK / KR;                  // (half) blocks along k
  static constexpr int BLOCKS = KB * (COLS / 8);
  static constexpr int PER = (BLOCKS + NT - 1) / NT;
  // Lane -> block.  Where the shape allows, a wavefront takes 8 blocks along k by 8 along m|n, so that each of
  // its load instructions covers whole 128-byte lines (8 rows x 8 chunks); otherwise blocks are dealt along k first.
  static constexpr bool LINES = KCG_TL_LINES && KB % 8 == 0 && (COLS / 8) % 8 == 0 && BLOCKS % 64 == 0;
  static __device__ __forceinline__ void block_of(int q, int& kb, int& cb) {
    if (LINES) {
      const int w = q >> 6, l = q & 63;
      kb = (w % (KB / 8)) * 8 + (l & 7);
      cb = (w / (KB / 8)) * 8 + (l >> 3);
    } else {
      kb = q % KB;
      cb = q / KB;
    }
  }
  kcg_u32x4 r[PER][KR];
  __device__ __forceinline__ void load_unit(int i, const kcg_u16* __restrict__ g, long ld, int col0, int k0,
                                            int col_lim, int k_lim, int tid) {
    const int q = i * NT + tid;
    int kb, cb;
    block_of(q, kb, cb);
#pragma unroll
    for (int kk = 0; kk < KR; ++kk) {
      kcg_u32x4 v = {0u, 0u, 0u, 0u};
      if (BLOCKS % NT == 0 || q < BLOCKS) {
        const int k = k0 + kb * KR + kk;
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
  __device__ __forceinline__ void store_unit(int i, char* s, int row_bytes, int tid) const {
    const int q = i * NT + tid;
    if (BLOCKS % NT == 0 || q < BLOCKS) {
      int kb, cb;
      block_of(q, kb, cb);
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        // column c of the block: halves c%2 of dword c/2 of each of the KR k rows
        unsigned o[KR / 2];
#pragma unroll
        for (int e = 0; e < KR / 2; ++e) {
          const unsigned lo = r[i][2 * e][c / 2], hi = r[i][2 * e + 1][c / 2];
          o[e] = (c & 1) ? __builtin_amdgcn_perm(hi, lo, 0x07060302u)
                         : __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        }
        char* d = s + (cb * 8 + c) * row_bytes + kb * (2 * KR);
        if (KR == 8) {
          kcg_u32x4 w = {o[0], o[1], o[KR / 2 - 2], o[KR / 2 - 1]};
          *(kcg_u32x4*)d = w;
        } else {
          kcg_u32x2 w = {o[0], o[1]};
          *(kcg_u32x2*)d = w;
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
  typedef KcgKLoader<GB_BM, GB_BK, GB_NT, GB_GUARD> LoaderA;
#define GB_LOAD_A(s, i, k0) la[s].load_unit((i), A, GB_K, m0, (k0), GB_M, GB_K, tid)
#else
  typedef KcgTLoader<GB_BM, GB_BK, GB_NT, GB_GUARD> LoaderA;
#define GB_LOAD_A(s, i, k0) la[s].load_unit((i), A, GB_M, m0, (k0), GB_M, GB_K, tid)
#endif
#if GB_TB == 1
  typedef KcgKLoader<GB_BN, GB_BK, GB_NT, GB_GUARD> LoaderB;
#define GB_LOAD_B(s, i, k0) lb[s].load_unit((i), B, GB_K, n0, (k0), GB_N, GB_K, tid)
#else
  typedef KcgTLoader<GB_BN, GB_BK, GB_NT, GB_GUARD> LoaderB;
#define GB_LOAD_B(s, i, k0) lb[s].load_unit((i), B, GB_N, n0, (k0), GB_N, GB_K, tid)
#endif
  // Staging registers between global memory and LDS: tile j waits in set j % GB_STAGES.
  LoaderA la[GB_STAGES];
  LoaderB lb[GB_STAGES];
  constexpr int PA = LoaderA::PER, PB = LoaderB::PER, UNITS = PA + PB;
  constexpr int WA = LoaderA::WEIGHT, WB = LoaderB::WEIGHT, WORK = PA * WA + PB * WB;
  constexpr int KS = GB_BK / 16;                 // MFMA k-steps per tile
  constexpr int FS = KS > 1 ? KS - 1 : 1;        // k-steps that carry feeding work

  kcg_f32x16 acc[GB_TM][GB_TN];
#pragma unroll
  for (int i = 0; i < GB_TM; ++i)
#pragma unroll
    for (int j = 0; j < GB_TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // Prologue: tile 0 through set 0 into LDS buffer 0, then tiles 1..GB_STAGES
  // into their staging sets.
#pragma unroll
  for (int u = 0; u < PA; ++u) GB_LOAD_A(0, u, 0);
#pragma unroll
  for (int u = 0; u < PB; ++u) GB_LOAD_B(0, u, 0);
#pragma unroll
  for (int u = 0; u < PA; ++u) la[0].store_unit(u, sA, GB_ROWB, tid);
#pragma unroll
  for (int u = 0; u < PB; ++u) lb[0].store_unit(u, sB, GB_ROWB, tid);
#pragma unroll
  for (int j = 1; j <= GB_STAGES; ++j)
    if (j < GB_KT) {
#pragma unroll
      for (int u = 0; u < PA; ++u) GB_LOAD_A(j % GB_STAGES, u, j * GB_BK);
#pragma unroll
      for (int u = 0; u < PB; ++u) GB_LOAD_B(j % GB_STAGES, u, j * GB_BK);
    }
  __syncthreads();

  const char* fA = sA + (wm * GB_WTM + l32) * GB_ROWB + lh * 16;
  const char* fB = sB + (wn * GB_WTN + l32) * GB_ROWB + lh * 16;
  kcg_bf16x8 fa[2][GB_TM], fb[2][GB_TN];
#pragma unroll
  for (int i = 0; i < GB_TM; ++i) fa[0][i] = *(const kcg_bf16x8*)(fA + i * 32 * GB_ROWB);
#pragma unroll
  for (int j = 0; j < GB_TN; ++j) fb[0][j] = *(const kcg_bf16x8*)(fB + j * 32 * GB_ROWB);

  // Iteration kt multiplies tile kt out of LDS buffer kt%2.  Meanwhile, spread
  // over its first k-steps, the staging set that holds tile kt+1 is written to
  // the other LDS buffer and, register by register, immediately reloaded with
  // tile kt+1+GB_STAGES: every global load has GB_STAGES whole iterations to
  // arrive.  The fragment reads run one k-step ahead of the MFMAs.  The single
  // barrier of the iteration sits before the last k-step: by then every
  // wavefront has finished reading this buffer and writing the other, so the
  // first fragments of tile kt+1 are fetched under the last step's MFMAs.  The
  // scheduling fences pin this order.  The body is instantiated per parity of
  // kt (LDS buffer and staging set become compile-time constants) and once more
  // for the last iterations, where the feeding work is conditional.
  auto iteration = [&](const int kt, auto par_c, auto steady_c) {
    constexpr int buf = decltype(par_c)::v ? 1 : 0;
    constexpr bool steady = decltype(steady_c)::v;
    constexpr int set = (buf + 1) % GB_STAGES;
    const bool feed = steady || kt + 1 < GB_KT;               // tile kt+1 exists: write it to LDS
    const bool fetch = steady || kt + 1 + GB_STAGES < GB_KT;  // tile kt+1+GB_STAGES exists: load it
    const char* cA = fA + buf * (GB_BM * GB_ROWB);
    const char* cB = fB + buf * (GB_BN * GB_ROWB);
    char* nA = sA + (buf ^ 1) * (GB_BM * GB_ROWB);
    char* nB = sB + (buf ^ 1) * (GB_BN * GB_ROWB);
    const int k2 = (kt + 1 + GB_STAGES) * GB_BK;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      __builtin_amdgcn_sched_barrier(0);
      if (ks + 1 < KS) {
#pragma unroll
        for (int i = 0; i < GB_TM; ++i) fa[nxt][i] = *(const kcg_bf16x8*)(cA + i * 32 * GB_ROWB + (ks + 1) * 32);
#pragma unroll
        for (int j = 0; j < GB_TN; ++j) fb[nxt][j] = *(const kcg_bf16x8*)(cB + j * 32 * GB_ROWB + (ks + 1) * 32);
      }
      if (ks < FS) {
#pragma unroll
        for (int u = 0; u < UNITS; ++u)
          if ((u < PA ? u * WA : PA * WA + (u - PA) * WB) * FS / WORK == ks) {   // units dealt to the steps by weight
            if (u < PA) {
              if (feed) la[set].store_unit(u, nA, GB_ROWB, tid);
              if (fetch) GB_LOAD_A(set, u, k2);
            } else {
              if (feed) lb[set].store_unit(u - PA, nB, GB_ROWB, tid);
              if (fetch) GB_LOAD_B(set, u - PA, k2);
            }
          }
      }
      if (ks == KS - 1) {
        __syncthreads();
        if (feed) {
#pragma unroll
          for (int i = 0; i < GB_TM; ++i)
            fa[nxt][i] = *(const kcg_bf16x8*)(fA + (buf ^ 1) * (GB_BM * GB_ROWB) + i * 32 * GB_ROWB);
#pragma unroll
          for (int j = 0; j < GB_TN; ++j)
            fb[nxt][j] = *(const kcg_bf16x8*)(fB + (buf ^ 1) * (GB_BN * GB_ROWB) + j * 32 * GB_ROWB);
        }
      }
#if !GB_INTERLEAVE
      __builtin_amdgcn_sched_barrier(0);
#endif
#pragma unroll
      for (int i = 0; i < GB_TM; ++i)
#pragma unroll
        for (int j = 0; j < GB_TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[cur][i], fb[cur][j], acc[i][j], 0, 0, 0);
#if GB_INTERLEAVE
      // One wavefront per SIMD: nothing else fills the issue slots while an MFMA
      // occupies the pipe, so the step's LDS, global-memory and permute
      // instructions are dealt out between its MFMAs instead of ahead of them.
#pragma unroll
      for (int m = 0; m < GB_TM * GB_TN; ++m) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
        __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);   // permutes / address arithmetic
        __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);   // one LDS write
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // one global load
      }
#endif
    }
    __builtin_amdgcn_sched_barrier(0);
    if (KS & 1) {      // odd number of k-steps: the prefetched fragments sit in set 1, move them to set 0
#pragma unroll
      for (int i = 0; i < GB_TM; ++i) fa[0][i] = fa[1][i];
#pragma unroll
      for (int j = 0; j < GB_TN; ++j) fb[0][j] = fb[1][j];
    }
  };
  int kt = 0;
  for (; kt + 2 + GB_STAGES < GB_KT; kt += 2) {      // both iterations of the pair feed and fetch
    iteration(kt, KcgBool<false>{}, KcgBool<true>{});
    iteration(kt + 1, KcgBool<true>{}, KcgBool<true>{});
  }
  for (; kt < GB_KT; ++kt) {
    if (kt & 1) iteration(kt, KcgBool<true>{}, KcgBool<false>{});
    else iteration(kt, KcgBool<false>{}, KcgBool<false>{});
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
          C[(long)row * GB_N + col] = (kcg_u16)kcg_f32_to_bf16_bits(GB_RELU ? fmaxf(acc[i][j][v], 0.0f) : acc[i][j][v]);
#else
          C[(long)row * GB_N + col] = GB_RELU ? fmaxf(acc[i][j][v], 0.0f) : acc[i][j][v];
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
