// ---- fp8 (e4m3) GEMM / batched GEMM on v_mfma_f32_32x32x64_f8f6f4 --------------
// C[b] = scale_a * scale_b * op(A[b]) * op(B[b]); fp8 e4m3 operands with one
// fp32 scale per tensor, fp32 accumulate, fp32 or bf16 out.  Parameters:
//   GF_NAME   kernel symbol
//   GF_M GF_N GF_K GF_BATCH      problem (dense, static)
//   GF_TA / GF_TB                1: operand stored column-major (A as [K][M], B as [N][K]);
//                                the k-contiguous forms (GF_TA=0, GF_TB=1) need no transposition
//   GF_BM GF_BN GF_BK            workgroup tile, GF_BK a multiple of 64
//   GF_WM GF_WN                  wavefronts along M and N; block = 64*GF_WM*GF_WN
//   GF_GROUP_M                   tile rows per L2 strip
//   GF_EDGE                      1: ragged tiles, guard loads and stores
//   GF_OUT_BF16                  1: C is bf16, else fp32
//   GF_RELU                      1: fused max(0, .) epilogue
//   GF_STAGES                    1 or 2 sets of staging registers = tiles in flight from global memory
//   GF_PREFETCH                  1: fragment reads run one k-step ahead (two fragment sets), 0: read at use
//   GF_ROTATE                    1 (GF_PREFETCH = 0, at least two k-steps per tile): a fragment is read again, for the
//                                next k-step, right behind the last MFMA that uses it (see "Rotating fragments")
//   GF_PINGPONG                  1 (GF_BK = 64, eight wavefronts, whole tiles): the two wavefronts of a SIMD run half a
//                                k-tile out of step, one in its memory phase while the other multiplies (see the loop)
//   GF_BTR                       1 (GF_TB = 0 only): B tiles lie in LDS as they lie in memory, [k][n], and the MFMA
//                                fragments come from transposing LDS reads (see "B as it lies" below); 0: B is
//                                transposed in registers on the way in
//   GF_SCALE_PTR                 0: the scales are two trailing fp32 kernel arguments, (A, B, C, float, float);
//                                1: they are read from device memory, one fp32 each, (A, B, C, const float*, const float*):
//                                   the order of a BatchedMatmul function that carries them as graph values;
//                                2: the same with the result last, (A, B, const float*, const float*, C): the order
//                                   of a Matmul function (inputs, then the output it allocates)
//
// One v_mfma_f32_32x32x64_f8f6f4 takes per lane 32 consecutive-k bytes of row
// (A) / column (B) lane%32, k half lane/32.  The LDS tiles are k-contiguous
// rows padded by 16 bytes, read as two ds_read_b128 per fragment.  An operand
// that is contiguous along m or n in memory is transposed byte-wise in
// registers on the way in (4x4 byte blocks, v_perm_b32).  The pipeline
// is the one of the bf16 kernel: staging registers written to the other LDS
// buffer and reloaded during the first k-steps, fragment reads one k-step
// ahead, one barrier before the last k-step.
#ifndef KCG_GEMM8_HELPERS
#define KCG_GEMM8_HELPERS
template <bool B> struct KcgBool8 { static constexpr bool v = B; };

// 16-byte chunks (16 fp8 values), contiguous along k in global memory.
template <int ROWS, int BK, int NT, bool GUARD>
struct KcgKLoader8 {
  static constexpr int CPR = BK / 16;
  static constexpr int CHUNKS = ROWS * CPR;
  static constexpr int PER = (CHUNKS + NT - 1) / NT;
  kcg_u32x4 r[PER];
  __device__ __forceinline__ void load_unit(int i, const unsigned char* __restrict__ g, long ld, int row0, int k0,
                                            int row_lim, int k_lim, int tid) {
    const int q = i * NT + tid;
    kcg_u32x4 v = {0u, 0u, 0u, 0u};
    if (!GUARD && CHUNKS % NT == 0 && NT % CPR == 0 && (long)(NT / CPR + 1) * ld < 0x7fffffffL) {
      // Address = a part that is the same for every lane (tile, unit, k-tile: scalar registers) plus a 32-bit
      // lane part that all units share: one address register for the whole loader instead of two per unit.
      const unsigned lane_part = (unsigned)(tid / CPR) * (unsigned)ld + (unsigned)(tid % CPR) * 16u;
      const unsigned char* unit_part = g + (long)(row0 + i * (NT / CPR)) * ld + k0;
      r[i] = *(const kcg_u32x4*)(unit_part + lane_part);
      return;
    }
    if (CHUNKS % NT == 0 || q < CHUNKS) {
      const int rr = q / CPR, c = q % CPR;
      const unsigned char* p = g + (long)(row0 + rr) * ld + (k0 + c * 16);
      if (!GUARD) {
        v = *(const kcg_u32x4*)p;
      } else if (row0 + rr < row_lim) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const unsigned b = (k0 + c * 16 + j < k_lim) ? (unsigned)p[j] : 0u;
          v[j / 4] |= b << (8 * (j % 4));
        }
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

// KR(k) x 16(m|n) byte blocks, contiguous along m|n in global memory, transposed in registers:
// a lane loads KR rows of 16 bytes and writes, for each of the 16 columns, its KR consecutive-k
// bytes.  KR = 8 when such blocks keep at least half the lanes busy, else 4: with eight rows a wavefront's load
// covers 64 bytes of each row instead of 32 (6 % on the 4096 x 11008 x 4096 product with operands in HBM) and
// its 8-byte LDS stores stay conflict free, at the price of idle lanes.
template <int COLS, int BK, int NT, bool GUARD>
struct KcgTLoader8 {
  static constexpr int KR = ((BK / 8) * (COLS / 16) * 2 >= NT) ? 8 : 4;
  static constexpr int KB = BK / KR;
  static constexpr int BLOCKS = KB * (COLS / 16);
  static constexpr int PER = (BLOCKS + NT - 1) / NT;
  kcg_u32x4 r[PER][KR];
  __device__ __forceinline__ void load_unit(int i, const unsigned char* __restrict__ g, long ld, int col0, int k0,
                                            int col_lim, int k_lim, int tid) {
    const int q = i * NT + tid;
    const int kb = q % KB, cb = q / KB;
#pragma unroll
    for (int kk = 0; kk < KR; ++kk) {
      kcg_u32x4 v = {0u, 0u, 0u, 0u};
      if (BLOCKS % NT == 0 || q < BLOCKS) {
        const int k = k0 + kb * KR + kk;
        const unsigned char* p = g + (long)k * ld + (col0 + cb * 16);
        if (!GUARD) {
          v = *(const kcg_u32x4*)p;
        } else if (k < k_lim) {
#pragma unroll
          for (int j = 0; j < 16; ++j) {
            const unsigned b = (col0 + cb * 16 + j < col_lim) ? (unsigned)p[j] : 0u;
            v[j / 4] |= b << (8 * (j % 4));
          }
        }
      }
      r[i][kk] = v;
    }
  }
  __device__ __forceinline__ void store_unit(int i, char* s, int row_bytes, int tid) const {
    const int q = i * NT + tid;
    if (BLOCKS % NT == 0 || q < BLOCKS) {
      const int kb = q % KB, cb = q / KB;
#pragma unroll
      for (int d = 0; d < 4; ++d) {            // dword d of every row: columns 4d .. 4d+3
        unsigned col[4][KR / 4];               // col[c][g] = bytes k = 4g .. 4g+3 of column 4d + c
#pragma unroll
        for (int gq = 0; gq < KR / 4; ++gq) {
          const unsigned r0 = r[i][4 * gq][d], r1 = r[i][4 * gq + 1][d], r2 = r[i][4 * gq + 2][d], r3 = r[i][4 * gq + 3][d];
          const unsigned t0 = __builtin_amdgcn_perm(r1, r0, 0x05010400u), t1 = __builtin_amdgcn_perm(r1, r0, 0x07030602u);
          const unsigned u0 = __builtin_amdgcn_perm(r3, r2, 0x05010400u), u1 = __builtin_amdgcn_perm(r3, r2, 0x07030602u);
          col[0][gq] = __builtin_amdgcn_perm(u0, t0, 0x05040100u);
          col[1][gq] = __builtin_amdgcn_perm(u0, t0, 0x07060302u);
          col[2][gq] = __builtin_amdgcn_perm(u1, t1, 0x05040100u);
          col[3][gq] = __builtin_amdgcn_perm(u1, t1, 0x07060302u);
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          char* dst = s + (cb * 16 + 4 * d + c) * row_bytes + kb * KR;
          if (KR == 8) {
            kcg_u32x2 w = {col[c][0], col[c][KR / 4 - 1]};
            *(kcg_u32x2*)dst = w;
          } else {
            *(unsigned*)dst = col[c][0];
          }
        }
      }
    }
  }
};
#endif  // KCG_GEMM8_HELPERS


#ifndef KCG_LD32
#define KCG_LD32
// 32 consecutive bytes of LDS as the eight dwords of one f8f6f4 MFMA operand.
__device__ __forceinline__ kcg_i32x8 kcg_ld32(const char* p) {
  const kcg_i32x4 lo = *(const kcg_i32x4*)p, hi = *(const kcg_i32x4*)(p + 16);
  kcg_i32x8 r = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return r;
}
#endif
#define GF_NT (64 * GF_WM * GF_WN)
#define GF_WTM (GF_BM / GF_WM)
#define GF_WTN (GF_BN / GF_WN)
#define GF_TM (GF_WTM / 32)
#define GF_TN (GF_WTN / 32)
#define GF_ROWB (GF_BK + 16)
#ifndef GF_BTR
#define GF_BTR 0
#endif
#if GF_BTR && GF_TB
#error "GF_BTR is for a B operand stored [K][N]"
#endif
// B as it lies.  A B tile is copied row by row, sB[k][n], rows of GF_BN bytes padded by 32.  One ds_read_b64_tr_b8
// (probed on the device, its operation is in no header here): within each group of 16 lanes, lane r supplies the address
// of 8 bytes, row r of a 16 x 8 byte matrix M, and lane i receives M[2 j + i / 8][i % 8], j = 0..7.  With the even lanes
// r = 2 j pointing at sB[k + j][n .. n + 7] and the odd lanes r = 2 j + 1 at sB[k + j][n + 8 .. n + 15], lane i receives the
// eight consecutive k of column n + i: a quarter of an MFMA operand, four reads per fragment.  The 32 lanes that are
// served together read eight rows of 32 bytes; with the pad the rows fall on eight disjoint sets of eight banks.
#define GF_BROWB (GF_BN + 32)
#define GF_SB_BYTES (GF_BTR ? 2 * GF_BK * GF_BROWB : 2 * GF_BN * GF_ROWB)
#define GF_KT ((GF_K + GF_BK - 1) / GF_BK)
#define GF_GUARD ((GF_EDGE != 0) | ((GF_K % 16) != 0) | ((GF_TA != 0) & ((GF_M % 16) != 0)) | ((GF_TB == 0) & ((GF_N % 16) != 0)))

#if (GF_BM % (32 * GF_WM)) || (GF_BN % (32 * GF_WN)) || (GF_BK % 64)
#error "tile shape does not divide into 32x32x64 MFMA tiles"
#endif

#ifndef GF_STAGGER
#define GF_STAGGER 0
#define GF_STAGGER_DEFAULTED 1
#endif
#ifndef GF_SCALE_PTR
#define GF_SCALE_PTR 0
#define GF_SCALE_PTR_DEFAULTED
#endif
#if GF_OUT_BF16
#define GF_C_T unsigned short
#else
#define GF_C_T float
#endif
extern "C" __global__ __launch_bounds__(GF_NT)
#if GF_SCALE_PTR == 2
void GF_NAME(const unsigned char* __restrict__ A, const unsigned char* __restrict__ B,
             const float* __restrict__ scale_a_p, const float* __restrict__ scale_b_p, GF_C_T* __restrict__ C) {
  const float scale_a = *scale_a_p, scale_b = *scale_b_p;
#elif GF_SCALE_PTR == 1
void GF_NAME(const unsigned char* __restrict__ A, const unsigned char* __restrict__ B, GF_C_T* __restrict__ C,
             const float* __restrict__ scale_a_p, const float* __restrict__ scale_b_p) {
  const float scale_a = *scale_a_p, scale_b = *scale_b_p;
#else
void GF_NAME(const unsigned char* __restrict__ A, const unsigned char* __restrict__ B, GF_C_T* __restrict__ C,
             float scale_a, float scale_b) {
#endif
  __shared__ __attribute__((aligned(16))) char kcg_smem[2 * GF_BM * GF_ROWB + GF_SB_BYTES];
  char* sA = kcg_smem;                                  // [2][GF_BM][GF_ROWB]
  char* sB = kcg_smem + 2 * GF_BM * GF_ROWB;            // [2][GF_BN][GF_ROWB], or [2][GF_BK][GF_BROWB] (GF_BTR)
  constexpr int B_ROWB = GF_BTR ? GF_BROWB : GF_ROWB;          // pitch of a row of the B tile in LDS
  constexpr int B_BUF = GF_BTR ? GF_BK * GF_BROWB : GF_BN * GF_ROWB;   // bytes of one B buffer

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / GF_WN;
  const int wn = wave % GF_WN;
  const int l32 = lane & 31;
  const int lh = lane >> 5;

#if GF_STAGGER
  // Out of step on purpose.  All workgroups of a launch start together and take the same time for a tile, so all of
  // them write their results at the same moment, a burst that the memory takes several microseconds to absorb while
  // no matrix instruction runs.  The workgroups of the first round (one per compute unit) therefore start up to
  // 7 * GF_STAGGER sleeps of 4096 cycles apart, in eight classes per XCD; the rounds after them inherit the offsets.
  if (blockIdx.x < 256 && blockIdx.y == 0) {
    const int steps = (int)((blockIdx.x >> 3) & 7) * GF_STAGGER;
    for (int d = 0; d < steps; ++d) __builtin_amdgcn_s_sleep(64);
  }
#endif
  const int tiles_m = (GF_M + GF_BM - 1) / GF_BM;
  const int tiles_n = (GF_N + GF_BN - 1) / GF_BN;
  int tile_m, tile_n;
  kcg_tile_coords(blockIdx.x, tiles_m, tiles_n, GF_GROUP_M, tile_m, tile_n);
  const int m0 = tile_m * GF_BM;
  const int n0 = tile_n * GF_BN;
  const long batch = blockIdx.y;
  A += batch * (long)GF_M * GF_K;
  B += batch * (long)GF_K * GF_N;
  C += batch * (long)GF_M * GF_N;

#if GF_TA == 0
  typedef KcgKLoader8<GF_BM, GF_BK, GF_NT, GF_GUARD> LoaderA;
#define GF_LOAD_A(s, i, k0) la[s].load_unit((i), A, GF_K, m0, (k0), GF_M, GF_K, tid)
#else
  typedef KcgTLoader8<GF_BM, GF_BK, GF_NT, GF_GUARD> LoaderA;
#define GF_LOAD_A(s, i, k0) la[s].load_unit((i), A, GF_M, m0, (k0), GF_M, GF_K, tid)
#endif
#if GF_TB == 1
  typedef KcgKLoader8<GF_BN, GF_BK, GF_NT, GF_GUARD> LoaderB;
#define GF_LOAD_B(s, i, k0) lb[s].load_unit((i), B, GF_K, n0, (k0), GF_N, GF_K, tid)
#elif GF_BTR
  // rows of the tile = k, 16-byte chunks along n: the k-contiguous loader with the roles of the two extents exchanged
  typedef KcgKLoader8<GF_BK, GF_BN, GF_NT, GF_GUARD> LoaderB;
#define GF_LOAD_B(s, i, k0) lb[s].load_unit((i), B, GF_N, (k0), n0, GF_K, GF_N, tid)
#else
  typedef KcgTLoader8<GF_BN, GF_BK, GF_NT, GF_GUARD> LoaderB;
#define GF_LOAD_B(s, i, k0) lb[s].load_unit((i), B, GF_N, n0, (k0), GF_N, GF_K, tid)
#endif
  // Staging registers between global memory and LDS: tile j waits in set j % GF_STAGES.
  LoaderA la[GF_STAGES];
  LoaderB lb[GF_STAGES];
  constexpr int PA = LoaderA::PER, PB = LoaderB::PER, UNITS = PA + PB;
  constexpr int KS = GF_BK / 64;                 // MFMA k-steps per tile
  constexpr int FS = KS > 1 ? KS - 1 : 1;        // k-steps that carry feeding work

  kcg_f32x16 acc[GF_TM][GF_TN];
#pragma unroll
  for (int i = 0; i < GF_TM; ++i)
#pragma unroll
    for (int j = 0; j < GF_TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // Prologue: tile 0 through set 0 into LDS buffer 0, then tiles 1..GF_STAGES
  // into their staging sets.
#pragma unroll
  for (int u = 0; u < PA; ++u) GF_LOAD_A(0, u, 0);
#pragma unroll
  for (int u = 0; u < PB; ++u) GF_LOAD_B(0, u, 0);
#pragma unroll
  for (int u = 0; u < PA; ++u) la[0].store_unit(u, sA, GF_ROWB, tid);
#pragma unroll
  for (int u = 0; u < PB; ++u) lb[0].store_unit(u, sB, B_ROWB, tid);
#pragma unroll
  for (int j = 1; j <= GF_STAGES; ++j)
    if (j < GF_KT) {
#pragma unroll
      for (int u = 0; u < PA; ++u) GF_LOAD_A(j % GF_STAGES, u, j * GF_BK);
#pragma unroll
      for (int u = 0; u < PB; ++u) GF_LOAD_B(j % GF_STAGES, u, j * GF_BK);
    }
  __syncthreads();

  const char* fA = sA + (wm * GF_WTM + l32) * GF_ROWB + lh * 32;
#if GF_BTR
  // this lane's address for the transposing reads of k-step 0, column tile 0, first quarter: row 32 lh + (lane % 16) / 2,
  // columns 16 ((lane / 16) % 2) + 8 (lane % 2) .. + 7 of the wavefront's strip
  typedef __attribute__((address_space(3))) char* kcg_lds_ptr8;
  typedef int kcg_i32x2_tr __attribute__((ext_vector_type(2)));
  const kcg_lds_ptr8 fB = (kcg_lds_ptr8)sB + (32 * lh + (lane & 15) / 2) * GF_BROWB + wn * GF_WTN + 16 * ((lane >> 4) & 1) + 8 * (lane & 1);
  // fragment of column tile j, k-step ks out of the buffer at byte offset `buf`
  auto read_fb = [&](int buf, int j, int ks) __attribute__((always_inline)) {
    kcg_i32x8 r;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const kcg_i32x2_tr v = __builtin_amdgcn_ds_read_tr8_b64_v2i32(
          (__attribute__((address_space(3))) kcg_i32x2_tr*)(fB + buf + (ks * 64 + 8 * q) * GF_BROWB + j * 32));
      r[2 * q] = v[0];
      r[2 * q + 1] = v[1];
    }
    return r;
  };
#else
  const char* fB = sB + (wn * GF_WTN + l32) * GF_ROWB + lh * 32;
  auto read_fb = [&](int buf, int j, int ks) __attribute__((always_inline)) {
    return kcg_ld32(fB + buf + j * 32 * GF_ROWB + ks * 64);
  };
#endif
  kcg_i32x8 fa[1 + GF_PREFETCH][GF_TM], fb[1 + GF_PREFETCH][GF_TN];
#if GF_ROTATE
  // Rotating fragments.  A fragment takes eight registers, a second set of the six of a k-step 48 more than the kernel
  // has; read at the start of the step that uses them, the fragments arrive while nothing but the other wavefront of
  // the SIMD can run.  The MFMAs of a step go row by row over the wavefront's tiles, so the A fragment of row i has its
  // last use in MFMA (i, last column) and the B fragment of column j in MFMA (last row, j): each is read again for the
  // NEXT k-step into the same registers right behind that MFMA, four to five MFMAs (256-320 cycles) ahead of its first
  // use there.  The barrier of a tile stands at the start of its last k-step: every wavefront has then issued (and, for
  // the barrier's own wait, received) its last reads of this buffer and has written its share of the other one, from
  // which the last step's re-reads take the first fragments of the next tile.
#pragma unroll
  for (int i = 0; i < GF_TM; ++i) fa[0][i] = kcg_ld32(fA + i * 32 * GF_ROWB);
#pragma unroll
  for (int j = 0; j < GF_TN; ++j) fb[0][j] = read_fb(0, j, 0);
#endif
#if GF_PREFETCH
#pragma unroll
  for (int i = 0; i < GF_TM; ++i) fa[0][i] = kcg_ld32(fA + i * 32 * GF_ROWB);
#pragma unroll
  for (int j = 0; j < GF_TN; ++j) fb[0][j] = read_fb(0, j, 0);
#endif

  // Iteration kt multiplies tile kt out of LDS buffer kt%2.  Meanwhile, spread
  // over its first k-steps, the staging set that holds tile kt+1 is written to
  // the other LDS buffer and, register by register, immediately reloaded with
  // tile kt+1+GF_STAGES: every global load has GF_STAGES whole iterations to
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
    constexpr int set = (buf + 1) % GF_STAGES;
    const bool feed = steady || kt + 1 < GF_KT;               // tile kt+1 exists: write it to LDS
    const bool fetch = steady || kt + 1 + GF_STAGES < GF_KT;  // tile kt+1+GF_STAGES exists: load it
    const char* cA = fA + buf * (GF_BM * GF_ROWB);
    constexpr int cB = buf * B_BUF, oB = (buf ^ 1) * B_BUF;      // this buffer and the other one, as byte offsets
    char* nA = sA + (buf ^ 1) * (GF_BM * GF_ROWB);
    char* nB = sB + oB;
    const int k2 = (kt + 1 + GF_STAGES) * GF_BK;
#if GF_ROTATE
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      __builtin_amdgcn_sched_barrier(0);
      if (ks == KS - 1) __syncthreads();
      if (ks < FS) {
#pragma unroll
        for (int u = 0; u < UNITS; ++u)
          if (u * FS / UNITS == ks) {
            if (u < PA) {
              if (feed) la[set].store_unit(u, nA, GF_ROWB, tid);
              if (fetch) GF_LOAD_A(set, u, k2);
            } else {
              if (feed) lb[set].store_unit(u - PA, nB, B_ROWB, tid);
              if (fetch) GF_LOAD_B(set, u - PA, k2);
            }
          }
      }
      const bool more = ks + 1 < KS || feed;                       // there is a next k-step to read fragments for
      const char* rA = ks + 1 < KS ? cA + (ks + 1) * 64 : fA + (buf ^ 1) * (GF_BM * GF_ROWB);
      const int rB = ks + 1 < KS ? cB : oB, rks = ks + 1 < KS ? ks + 1 : 0;
#pragma unroll
      for (int i = 0; i < GF_TM; ++i)
#pragma unroll
        for (int j = 0; j < GF_TN; ++j) {
          __builtin_amdgcn_sched_barrier(0);
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[0][i], fb[0][j], acc[i][j], 0, 0, 0, 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
          if (more && j == GF_TN - 1) fa[0][i] = kcg_ld32(rA + i * 32 * GF_ROWB);
          if (more && i == GF_TM - 1) fb[0][j] = read_fb(rB, j, rks);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    return;
#endif
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int cur = GF_PREFETCH ? (ks & 1) : 0, nxt = GF_PREFETCH ? (cur ^ 1) : 0;
      __builtin_amdgcn_sched_barrier(0);
      if (!GF_PREFETCH) {
#pragma unroll
        for (int i = 0; i < GF_TM; ++i) fa[0][i] = kcg_ld32(cA + i * 32 * GF_ROWB + ks * 64);
#pragma unroll
        for (int j = 0; j < GF_TN; ++j) fb[0][j] = read_fb(cB, j, ks);
      } else if (ks + 1 < KS) {
#pragma unroll
        for (int i = 0; i < GF_TM; ++i) fa[nxt][i] = kcg_ld32(cA + i * 32 * GF_ROWB + (ks + 1) * 64);
#pragma unroll
        for (int j = 0; j < GF_TN; ++j) fb[nxt][j] = read_fb(cB, j, ks + 1);
      }
      if (ks < FS) {
#pragma unroll
        for (int u = 0; u < UNITS; ++u)
          if (u * FS / UNITS == ks) {
            if (u < PA) {
              if (feed) la[set].store_unit(u, nA, GF_ROWB, tid);
              if (fetch) GF_LOAD_A(set, u, k2);
            } else {
              if (feed) lb[set].store_unit(u - PA, nB, B_ROWB, tid);
              if (fetch) GF_LOAD_B(set, u - PA, k2);
            }
          }
      }
      if (ks == KS - 1 && !GF_PREFETCH) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < GF_TM; ++i)
#pragma unroll
          for (int j = 0; j < GF_TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[0][i], fb[0][j], acc[i][j], 0, 0, 0, 0, 0, 0);
        __syncthreads();      // the MFMAs above have consumed the last fragments of this buffer
      } else if (ks == KS - 1) {
        __syncthreads();
        if (feed) {
#pragma unroll
          for (int i = 0; i < GF_TM; ++i)
            fa[nxt][i] = kcg_ld32(fA + (buf ^ 1) * (GF_BM * GF_ROWB) + i * 32 * GF_ROWB);
#pragma unroll
          for (int j = 0; j < GF_TN; ++j)
            fb[nxt][j] = read_fb(oB, j, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if (GF_PREFETCH || ks < KS - 1) {
#pragma unroll
        for (int i = 0; i < GF_TM; ++i)
#pragma unroll
          for (int j = 0; j < GF_TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[cur][i], fb[cur][j], acc[i][j], 0, 0, 0, 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (GF_PREFETCH && (KS & 1)) {      // odd number of k-steps: the prefetched fragments sit in set 1, move them to set 0
#pragma unroll
      for (int i = 0; i < GF_TM; ++i) fa[0][i] = fa[1][i];
#pragma unroll
      for (int j = 0; j < GF_TN; ++j) fb[0][j] = fb[1][j];
    }
  };
#if GF_PINGPONG
  // Two groups of wavefronts, half a k-tile out of step (GF_BK = 64: one k-step per tile).  Left to themselves the
  // two wavefronts of a SIMD do the same thing at the same time -- both wait for their fragments, both want the matrix
  // pipe, both issue their loads and stores -- and each part's time adds up.  Here a wavefront alternates between a
  // memory phase (its share of tile kt+1 from the staging registers into the other LDS buffer, the loads of tile
  // kt+1+GF_STAGES, the fragment reads of tile kt) and a matrix phase (the MFMAs of tile kt), every phase ends in a
  // workgroup barrier, and the second half of the wavefronts (the other wavefront of every SIMD) passes one barrier
  // more before it starts: while one group multiplies, the other moves data.  Buffer (kt+1) % 2 is written in the two
  // phases in which the groups have their memory phase of tile kt, and read in those of tile kt+1, a barrier later;
  // the fragments of tile kt-1, its previous content, were read a barrier earlier.
  {
    const bool late = wave >= GF_NT / 128;
    auto phase_pair = [&](const int kt, auto par_c, auto steady_c) {
      constexpr int buf = decltype(par_c)::v ? 1 : 0;
      constexpr bool steady = decltype(steady_c)::v;
      constexpr int set = (buf + 1) % GF_STAGES;
      const bool feed = steady || kt + 1 < GF_KT;
      const bool fetch = steady || kt + 1 + GF_STAGES < GF_KT;
      char* nA = sA + (buf ^ 1) * (GF_BM * GF_ROWB);
      char* nB = sB + (buf ^ 1) * B_BUF;
      const int k2 = (kt + 1 + GF_STAGES) * GF_BK;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < UNITS; ++u) {
        if (u < PA) {
          if (feed) la[set].store_unit(u, nA, GF_ROWB, tid);
          if (fetch) GF_LOAD_A(set, u, k2);
        } else {
          if (feed) lb[set].store_unit(u - PA, nB, B_ROWB, tid);
          if (fetch) GF_LOAD_B(set, u - PA, k2);
        }
      }
#pragma unroll
      for (int i = 0; i < GF_TM; ++i) fa[0][i] = kcg_ld32(fA + buf * (GF_BM * GF_ROWB) + i * 32 * GF_ROWB);
#pragma unroll
      for (int j = 0; j < GF_TN; ++j) fb[0][j] = read_fb(buf * B_BUF, j, 0);
      __syncthreads();
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < GF_TM; ++i)
#pragma unroll
        for (int j = 0; j < GF_TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[0][i], fb[0][j], acc[i][j], 0, 0, 0, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();
    };
    if (late) __syncthreads();
    int kt = 0;
    for (; kt + 2 + GF_STAGES < GF_KT; kt += 2) {
      phase_pair(kt, KcgBool8<false>{}, KcgBool8<true>{});
      phase_pair(kt + 1, KcgBool8<true>{}, KcgBool8<true>{});
    }
    for (; kt < GF_KT; ++kt) {
      if (kt & 1) phase_pair(kt, KcgBool8<true>{}, KcgBool8<false>{});
      else phase_pair(kt, KcgBool8<false>{}, KcgBool8<false>{});
    }
    if (!late) __syncthreads();
  }
#else
  int kt = 0;
  for (; kt + 2 + GF_STAGES < GF_KT; kt += 2) {      // both iterations of the pair feed and fetch
    iteration(kt, KcgBool8<false>{}, KcgBool8<true>{});
    iteration(kt + 1, KcgBool8<true>{}, KcgBool8<true>{});
  }
  for (; kt < GF_KT; ++kt) {
    if (kt & 1) iteration(kt, KcgBool8<true>{}, KcgBool8<false>{});
    else iteration(kt, KcgBool8<false>{}, KcgBool8<false>{});
  }
#endif

  const float scale = scale_a * scale_b;
  // ---- epilogue: lane l, register v -> row 8*(v/4) + 4*(l/32) + v%4, column l%32 ----
#pragma unroll
  for (int i = 0; i < GF_TM; ++i)
#pragma unroll
    for (int j = 0; j < GF_TN; ++j) {
      const int col = n0 + wn * GF_WTN + j * 32 + l32;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * GF_WTM + i * 32 + 8 * (v / 4) + 4 * lh + (v % 4);
#if GF_EDGE
        if (row < GF_M && col < GF_N)
#endif
        {
#if GF_OUT_BF16
          C[(long)row * GF_N + col] = (unsigned short)kcg_f32_to_bf16_bits(GF_RELU ? fmaxf(acc[i][j][v] * scale, 0.0f) : acc[i][j][v] * scale);
#else
          C[(long)row * GF_N + col] = GF_RELU ? fmaxf(acc[i][j][v] * scale, 0.0f) : acc[i][j][v] * scale;
#endif
        }
      }
    }
}
#undef GF_LOAD_A
#undef GF_LOAD_B
#undef GF_NT
#undef GF_WTM
#undef GF_WTN
#undef GF_TM
#undef GF_TN
#undef GF_ROWB
#undef GF_BROWB
#undef GF_SB_BYTES
#undef GF_BTR
#undef GF_KT
#undef GF_GUARD
#undef GF_C_T
#ifdef GF_SCALE_PTR_DEFAULTED
#undef GF_SCALE_PTR
#undef GF_SCALE_PTR_DEFAULTED
#endif
#ifdef GF_STAGGER_DEFAULTED
#undef GF_STAGGER
#undef GF_STAGGER_DEFAULTED
#endif
