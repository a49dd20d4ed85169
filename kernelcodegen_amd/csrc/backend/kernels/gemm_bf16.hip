// ---- bf16 / fp16 GEMM / batched GEMM on v_mfma_f32_32x32x16_{bf16,f16} ---------
// C[b] = op(A[b]) * op(B[b]); 16-bit float operands, fp32 accumulate, fp32 or 16-bit out.
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
//   GB_F16                       1: the operands (and a 16-bit result) are IEEE half instead of bf16; the tiles
//                                move as 16-bit patterns either way, only the MFMA and the result's rounding differ
//   GB_OUT_BF16                  1: C has the operands' 16-bit type, else fp32
//   GB_RELU                      1: fused max(0, .) epilogue
//   GB_STAGE_C                   1: results are turned round in LDS and stored as whole rows of the tile (see the
//                                epilogue); 2: with the non-temporal hint
//   GB_SK_UNITS                  0: one workgroup per tile.  > 0: the tiles that do not fill a whole round of
//                                GB_SK_UNITS workgroups (the tail) are split along k between GB_SK_UNITS extra
//                                workgroups; the kernel then takes a fourth pointer, a workspace
//   GB_SK_FULL                   number of workgroups that compute one whole tile each (GB_SK_UNITS > 0)
//
// Tail split (GB_SK_UNITS > 0, on request only: it measured slower than one workgroup per tile on the shapes
// tried).  GB_SK_FULL workgroups compute whole tiles and the k-iterations of the
// remaining tiles, laid end to end, are cut into GB_SK_UNITS equal runs, one per extra workgroup; a run covers
// the end of one tile and the start of the next (two segments).  A workgroup writes the accumulators of a
// segment to its slot of the workspace, makes them visible (device-scope fence) and counts itself in on the
// tile's counter; the workgroup that finds all others counted in adds the slots up in k order (so the sum
// does not depend on who arrives last) and stores the tile.  Nobody waits for anybody.  Workspace: 4096 bytes
// of counters (zero before the first launch; every launch leaves them zero), then GB_SK_UNITS * 2 slots of
// GB_BM * GB_BN floats.  When the tile count and the unit count are multiples of eight, runs and tiles are
// formed per XCD (workgroup id mod 8), so that a tile's contributors share an L2.
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
template <int V> struct KcgInt { static constexpr int v = V; };

// 16-byte chunks, contiguous along k in global memory.  Tile rows x BK.
// One unit = one chunk per lane.
// SPLIT forms every address as one 32-bit lane part, shared by all units, plus a part that is the same for every
// lane (scalar registers for global memory, an immediate for LDS).  It saves vector registers where the kernel
// around it is short of them and costs some where it is not, so the kernel chooses.
// SWZ (rows of exactly eight chunks, no padding): chunk c of row r is stored at chunk position c ^ ((r / 2) % 8), the
// layout the 16x16x32 MFMA fragments are read from (see GB_M16 in the kernel).
// QUADS (with SWZ): the values of k are regrouped inside each run of 32 so that chunk position q of the run holds the
// two runs of four values 4 q .. 4 q + 3 and 16 + 4 q .. 16 + 4 q + 3: what lane group q of a 16x16x32 fragment must
// hold when the other operand's fragments come from transposing LDS reads of rows 4 q .. and 16 + 4 q .. (two groups
// served together then read eight consecutive rows).  A chunk from memory, values 8 c .. 8 c + 7 of its run, goes out
// as two 8-byte halves to positions 2 (c % 2) and 2 (c % 2) + 1, half c / 2.
template <int ROWS, int BK, int NT, bool GUARD, bool SPLIT = false, bool SWZ = false, bool QUADS = false, bool OPAQUE = SWZ>
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
    if (SPLIT && !GUARD && CHUNKS % NT == 0 && NT % CPR == 0 && (long)(NT / CPR + 1) * ld * 2 < 0x7fffffffL) {
      unsigned lane_part = ((unsigned)(tid / CPR) * (unsigned)ld + (unsigned)(tid % CPR) * 8u) * 2u;
      // kept opaque where registers are short: the compiler otherwise keeps one 64-bit sum per unit across the k loop
      if (OPAQUE) asm volatile("" : "+v"(lane_part));
      const char* unit_part = (const char*)(g + (long)(row0 + i * (NT / CPR)) * ld + k0);
      r[i] = *(const kcg_u32x4*)(unit_part + lane_part);
      return;
    }
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
    static_assert(!SWZ || (CPR == 8 && NT % 128 == 0 && CHUNKS % NT == 0), "swizzled rows hold eight chunks and a unit covers whole groups of 16 rows");
    if (SPLIT && CHUNKS % NT == 0 && NT % CPR == 0) {
      typedef __attribute__((address_space(3))) char* lds_ptr;
      if (QUADS) {
        static_assert(!QUADS || SWZ, "regrouped chunks are part of the swizzled layout");
        const unsigned c = (unsigned)(tid % CPR), pos = (c & 4u) + 2u * (c & 1u), half = (c >> 1) & 1u;
        const unsigned first = (unsigned)(tid / CPR) * (unsigned)row_bytes + ((pos ^ (((unsigned)(tid / CPR) >> 1) & 7u)) * 16u) + half * 8u;
        const kcg_u32x2 lo = {r[i][0], r[i][1]}, hi = {r[i][2], r[i][3]};
        *(__attribute__((address_space(3))) kcg_u32x2*)((lds_ptr)s + first + i * (NT / CPR) * row_bytes) = lo;
        *(__attribute__((address_space(3))) kcg_u32x2*)((lds_ptr)s + (first ^ 16u) + i * (NT / CPR) * row_bytes) = hi;
        return;
      }
      const unsigned col = SWZ ? ((unsigned)(tid % CPR) ^ (((unsigned)(tid / CPR) >> 1) & 7u)) : (unsigned)(tid % CPR);
      const unsigned lane_part = (unsigned)(tid / CPR) * (unsigned)row_bytes + col * 16u;
      *(__attribute__((address_space(3))) kcg_u32x4*)((lds_ptr)s + lane_part + i * (NT / CPR) * row_bytes) = r[i];
      return;
    }
    static_assert(!QUADS || (SPLIT && CHUNKS % NT == 0 && NT % CPR == 0), "regrouped chunks need the split form");
    if (CHUNKS % NT == 0 || q < CHUNKS) {
      const int rr = q / CPR, c = SWZ ? ((q % CPR) ^ ((rr >> 1) & 7)) : q % CPR;
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

// GB_M16 1: the products run on v_mfma_f32_16x16x32 instead of v_mfma_f32_32x32x16.  One instruction then takes 32
// values of k and touches a quarter of the accumulators: per result the fp32 accumulators are read and written half
// as often, which is what the part's power limit rewards (a register-only loop on N(0,1) operands sustains
// 1.94 PFLOP/s with this shape against 1.74 with the other, 1.66 against 1.52 with the fragment reads from LDS).
// Lane l of a fragment holds row (A) / column (B) l % 16, values 8 (l / 16) .. + 7 of the step's 32 along k, one
// ds_read_b128.  The k-contiguous LDS rows are 128 bytes without padding (GB_BK = 64) and chunk c of row r lies at
// chunk position c ^ ((r / 2) % 8): the sixteen lanes that the LDS serves in one pass (lanes 0-3, 12-15 and 20-27
// of a half-wave, then the rest) then read sixteen different groups of four banks, and a store of whole rows stays a
// permutation within each row.  A fragment set of a k-step is twice the size of the other shape's, so only the A
// fragments have a second set; each B fragment is read again for the next step right behind its last MFMA.
#ifndef GB_M16
#define GB_M16 0
#define GB_M16_DEFAULTED 1
#endif
#ifndef GB_STAGE_C
#define GB_STAGE_C 0
#define GB_STAGE_C_DEFAULTED 1
#endif
#ifndef GB_D2L
#define GB_D2L 0
#define GB_D2L_DEFAULTED 1
#endif
#define GB_NT (64 * GB_WM * GB_WN)
#define GB_WTM (GB_BM / GB_WM)
#define GB_WTN (GB_BN / GB_WN)
#if GB_M16
#define GB_FR 16
#define GB_KSTEP 32
#define GB_ROWB (GB_BK * 2)
#define GB_ACC kcg_f32x4
#define GB_ACCN 4
#else
#define GB_FR 32
#define GB_KSTEP 16
#define GB_ROWB (GB_BK * 2 + 16)
#define GB_ACC kcg_f32x16
#define GB_ACCN 16
#endif
#define GB_TM (GB_WTM / GB_FR)
#define GB_TN (GB_WTN / GB_FR)
#define GB_KT ((GB_K + GB_BK - 1) / GB_BK)
// A B operand that is contiguous along n in memory (row-major [K][N]) is copied into LDS as it is, sB[k][n], and its
// MFMA operand fragments come from transposing LDS reads (ds_read_b64_tr_b16; within each group of 16 lanes, lane r
// supplies the address of four consecutive 16-bit values, row r of a 16 x 4 matrix M, and lane i receives
// M[4 j + i / 4][i % 4], j = 0..3: with lane r pointing at B[k0 + r / 4][n0 + 4 (r % 4) ..], lane i receives the four
// consecutive k of column n0 + i).  The 32 lanes served together read four k rows of 64 bytes; rows are padded by
// GB_BPAD bytes, chosen by the emitter so that the pitch is 64 modulo 256 and those rows fall on disjoint banks.
// GB_BTR 0 transposes such an operand in registers on the way in instead (KcgTLoader), as A still is.
#ifndef GB_BTR
#define GB_BTR (GB_TB == 0)
#define GB_BTR_DEFAULTED 1
#endif
#ifndef GB_BPAD
#define GB_BPAD 32
#endif
#define GB_BROWB (GB_BN * 2 + (GB_D2L ? 0 : GB_BPAD))               // bytes per k row of sB[k][n]
#define GB_BBUF (GB_BTR ? GB_BK * GB_BROWB : GB_BN * GB_ROWB)        // bytes of one B buffer
// The walk along k may start anywhere when no load is guarded, the tile is not split along k and K is whole tiles.  It
// does (see rot_k in the kernel) when both operands are contiguous along k, where it was measured to gain 15-20 %; with
// row-major [K][N] weights it gains nothing (their rows are read 512 bytes at a time at a pitch that is no power of two).
#ifndef GB_KROT_ON
#define GB_KROT_ON (GB_TA == 0 && GB_TB == 1)
#define GB_KROT_DEFAULTED
#endif
#define GB_KROT (GB_KROT_ON && !GB_GUARD && GB_SK_UNITS == 0 && GB_K % GB_BK == 0)
#define GB_GUARD ((GB_EDGE != 0) | ((GB_K % 8) != 0) | ((GB_TA != 0) & ((GB_M % 8) != 0)) | ((GB_TB == 0) & ((GB_N % 8) != 0)))

#ifndef GB_F16
#define GB_F16 0
#define GB_F16_DEFAULTED 1
#endif
// GB_SETPRIO n > 0: a wavefront raises its issue priority to n for the MFMAs of a k-step and drops it to 0 for the
// step's memory instructions (two wavefronts share a SIMD: the one in its memory phase then yields to the one that
// has matrix work).  Measured, not the default.
#ifndef GB_STAGGER
#define GB_STAGGER 0
#define GB_STAGGER_DEFAULTED 1
#endif
#ifndef GB_SETPRIO
#define GB_SETPRIO 0
#define GB_SETPRIO_DEFAULTED 1
#endif
#if GB_F16
typedef _Float16 kcg_f16x8 __attribute__((ext_vector_type(8)));
#define GB_FRAG kcg_f16x8
#if GB_M16
#define GB_MFMA __builtin_amdgcn_mfma_f32_16x16x32_f16
#else
#define GB_MFMA __builtin_amdgcn_mfma_f32_32x32x16_f16
#endif
#define GB_TO16(x) __builtin_bit_cast(unsigned short, (_Float16)(x))
#else
#define GB_FRAG kcg_bf16x8
#if GB_M16
#define GB_MFMA __builtin_amdgcn_mfma_f32_16x16x32_bf16
#else
#define GB_MFMA __builtin_amdgcn_mfma_f32_32x32x16_bf16
#endif
#define GB_TO16(x) ((kcg_u16)kcg_f32_to_bf16_bits(x))
#endif
#ifndef GB_SK_UNITS
#define GB_SK_UNITS 0
#define GB_SK_FULL 0
#define GB_SK_DEFAULTED 1
#endif
#define GB_TILES (((GB_M + GB_BM - 1) / GB_BM) * ((GB_N + GB_BN - 1) / GB_BN))
#define GB_SK_TAIL (GB_TILES - GB_SK_FULL)                         // tiles that are split along k
#define GB_SK_XCD ((GB_SK_UNITS % 8 == 0) && (GB_SK_FULL % 8 == 0) && (GB_SK_TAIL % 8 == 0) && (GB_TILES % 8 == 0))
#define GB_SK_GROUPS (GB_SK_XCD ? 8 : 1)                          // independent runs of tiles and units
#define GB_SK_GTILES (GB_SK_TAIL / GB_SK_GROUPS)                   // tail tiles per group
#define GB_SK_GUNITS (GB_SK_UNITS / GB_SK_GROUPS)                  // units per group
#define GB_SK_PER0 ((GB_SK_GTILES * GB_KT + GB_SK_GUNITS - 1) / (GB_SK_GUNITS > 0 ? GB_SK_GUNITS : 1))
#define GB_SK_PER (GB_SK_PER0 + (GB_SK_PER0 & 1))                    // k-iterations per unit, even

#if (GB_BM % (32 * GB_WM)) || (GB_BN % (32 * GB_WN)) || (GB_BK % 16)
#error "tile shape does not divide into 32x32x16 MFMA tiles"
#endif
#if GB_D2L && (!GB_M16 || (GB_BTR && GB_BN != 256))
#error "direct loads into LDS: only with the 16x16x32 form; row-major weights need 256-column tiles"
#endif
#if GB_M16 && (GB_BK != 64 || GB_TA != 0 || (GB_TB == 0 && !GB_BTR) || GB_GUARD || GB_SK_UNITS > 0 || GB_STAGES != 1 || GB_NT % 128 || GB_BM % (GB_NT / 8) || (GB_TB == 1 && GB_BN % (GB_NT / 8)))
#error "the 16x16x32 form needs whole 64-deep k-tiles, a k-contiguous A, unguarded loads, no tail split and one staging set"
#endif
#if GB_SK_UNITS > 0 && (GB_BATCH != 1 || GB_SK_TAIL <= 0 || GB_SK_TAIL > 1024 || GB_SK_PER > GB_KT || GB_SK_PER < 2)
#error "tail split: needs one batch, 1..1024 tail tiles and at most one tile's k-iterations per unit"
#endif
#if GB_SK_UNITS > 0 && ((GB_KT % 2) || (GB_SK_PER % 2) || GB_STAGES != 1 || (GB_K % GB_BK))
#error "tail split: needs an even number of whole k-tiles per tile and per unit, and one staging set"
#endif

#if GB_STAGE_C && (!GB_M16 || GB_BM != 256 || GB_BN != 256 || GB_WM != 4 || GB_WN != 2 || GB_EDGE || GB_SK_UNITS > 0)
#error "gemm_bf16: results go through LDS (GB_STAGE_C) only from whole 256 x 256 tiles of the 16x16x32 form, 4 x 2 wavefronts"
#endif
extern "C" __global__ __launch_bounds__(GB_NT)
void GB_NAME(const kcg_u16* __restrict__ A, const kcg_u16* __restrict__ B,
#if GB_OUT_BF16
             kcg_u16* __restrict__ C
#else
             float* __restrict__ C
#endif
#if GB_SK_UNITS > 0
             , unsigned* __restrict__ W
#endif
) {
  __shared__ __attribute__((aligned(16))) char kcg_smem[2 * GB_BM * GB_ROWB + 2 * GB_BBUF];
#if GB_SK_UNITS > 0
  __shared__ unsigned kcg_sk_arrived;
#endif
  char* sA = kcg_smem;                                  // [2][GB_BM][GB_ROWB]
  char* sB = kcg_smem + 2 * GB_BM * GB_ROWB;            // [2][GB_BN][GB_ROWB], or [2][GB_BK][GB_BROWB] (GB_BTR)

#if GB_STAGGER
  // Out of step on purpose.  All workgroups of a launch start together and take the same time for a tile, so all of
  // them write their results at the same moment, a burst that the memory takes several microseconds to absorb while
  // no matrix instruction runs.  The workgroups of the first round (one per compute unit) therefore start up to
  // 7 * GB_STAGGER sleeps of 4096 cycles apart, in eight classes per XCD; the rounds after them inherit the offsets.
  if (blockIdx.x < 256 && blockIdx.y == 0) {
    const int steps = (int)((blockIdx.x >> 3) & 7) * GB_STAGGER;
    for (int d = 0; d < steps; ++d) __builtin_amdgcn_s_sleep(64);
  }
#endif
  const int tiles_m = (GB_M + GB_BM - 1) / GB_BM;
  const int tiles_n = (GB_N + GB_BN - 1) / GB_BN;
  const long batch = blockIdx.y;
  A += batch * (long)GB_M * GB_K;
  B += batch * (long)GB_K * GB_N;
  C += batch * (long)GB_M * GB_N;

  // What this workgroup computes: k-iterations [kb, ke) of tile `pid` (a position in the order that
  // kcg_tile_coords walks), once for a whole-tile workgroup, up to twice for a tail unit.
#if GB_SK_UNITS > 0
  const bool sk_unit = (int)blockIdx.x >= GB_SK_FULL;
  const int sk_u = (int)blockIdx.x - GB_SK_FULL;
  const int sk_group = GB_SK_XCD ? (sk_u & 7) : 0;                 // XCD of the unit
  const int sk_lu = GB_SK_XCD ? (sk_u >> 3) : sk_u;                 // unit within its group
  const int sk_g0 = sk_lu * GB_SK_PER;                              // first k-iteration of the run, in the group's iteration space
  const int sk_g1 = (sk_g0 + GB_SK_PER) < GB_SK_GTILES * GB_KT ? (sk_g0 + GB_SK_PER) : GB_SK_GTILES * GB_KT;
  const int num_segments = !sk_unit ? 1 : (sk_g1 <= sk_g0 ? 0 : ((sk_g1 - 1) / GB_KT - sk_g0 / GB_KT + 1));
#else
  const int num_segments = 1;
#endif
  for (int segment = 0; segment < num_segments; ++segment) {
  int tid = threadIdx.x;
#if GB_SK_UNITS > 0
  // Everything a segment derives from the thread index is derived again for the next one: values kept in
  // registers from one segment to the next would be live across the k loop, which has no register to spare.
  asm volatile("" : "+v"(tid));
#endif
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / GB_WN;
  const int wn = wave % GB_WN;
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  int pid = blockIdx.x, kb = 0, ke = GB_KT;
#if GB_SK_UNITS > 0
  int sk_lt = 0;                                                    // tail tile within the group
  if (sk_unit) {
    sk_lt = sk_g0 / GB_KT + segment;
    kb = segment == 0 ? sk_g0 - sk_lt * GB_KT : 0;
    ke = (sk_g1 - sk_lt * GB_KT) < GB_KT ? (sk_g1 - sk_lt * GB_KT) : GB_KT;
    pid = GB_SK_FULL + (GB_SK_XCD ? sk_lt * 8 + sk_group : sk_lt);
  }
#endif
  const int len = ke - kb;
  int tile_m, tile_n;
  kcg_tile_coords(pid, tiles_m, tiles_n, GB_GROUP_M, tile_m, tile_n);
  const int m0 = tile_m * GB_BM;
  const int n0 = tile_n * GB_BN;
  // Where this workgroup's walk along k starts.  At any moment all workgroups of a launch are at about the same k, and
  // with a row pitch that is a power of two (K = 4096: 8 KB rows) the lines they ask for then differ only in address
  // bits far above the ones that select the memory channel: every request of that moment goes to the same few
  // channels.  The workgroups of XCD x (ids are dealt round-robin to the 8 XCDs) therefore start x/8 of the way along k
  // and wrap around, which spreads each moment's requests over the channels and leaves the sharing of operand panels
  // inside an XCD's L2 as it was.  Measured on 4096x11008x4096 with k-contiguous weights: 0.376 -> 0.313 ms.  The
  // sum over k is taken in the rotated order, so results differ in the last bits between XCDs (and from the unrotated
  // order), deterministically.
#if GB_KROT
  const int rot_k = (int)(blockIdx.x & 7) * GB_KT / 8 * GB_BK;
#define GB_KPOS(k0) (((k0) + rot_k) % GB_K)
#else
#define GB_KPOS(k0) (k0)
#endif

#if GB_TA == 0
  typedef KcgKLoader<GB_BM, GB_BK, GB_NT, GB_GUARD, GB_BTR != 0 || GB_M16 != 0, GB_M16 != 0, GB_M16 != 0 && GB_BTR != 0 && !GB_D2L> LoaderA;
#define GB_LOAD_A(s, i, k0) la[s].load_unit((i), As, GB_K, m0, GB_KPOS(k0), GB_M, k_lim, tid)
  const kcg_u16* __restrict__ As = A + (long)kb * GB_BK;                 // the segment's first k column
#else
  typedef KcgTLoader<GB_BM, GB_BK, GB_NT, GB_GUARD> LoaderA;
#define GB_LOAD_A(s, i, k0) la[s].load_unit((i), As, GB_M, m0, GB_KPOS(k0), GB_M, k_lim, tid)
  const kcg_u16* __restrict__ As = A + (long)kb * GB_BK * GB_M;          // the segment's first k row
#endif
#if GB_TB == 1
  typedef KcgKLoader<GB_BN, GB_BK, GB_NT, GB_GUARD, GB_M16 != 0, GB_M16 != 0> LoaderB;
#define GB_LOAD_B(s, i, k0) lb[s].load_unit((i), Bs, GB_K, n0, GB_KPOS(k0), GB_N, k_lim, tid)
  const kcg_u16* __restrict__ Bs = B + (long)kb * GB_BK;
#elif GB_BTR
  typedef KcgKLoader<GB_BK, GB_BN, GB_NT, GB_GUARD, true, false, false, GB_M16 != 0> LoaderB;        // rows are k, contiguous along n: a plain copy
#define GB_LOAD_B(s, i, k0) lb[s].load_unit((i), Bs, GB_N, GB_KPOS(k0), n0, k_lim, GB_N, tid)
  const kcg_u16* __restrict__ Bs = B + (long)kb * GB_BK * GB_N;
#else
  typedef KcgTLoader<GB_BN, GB_BK, GB_NT, GB_GUARD> LoaderB;
#define GB_LOAD_B(s, i, k0) lb[s].load_unit((i), Bs, GB_N, n0, GB_KPOS(k0), GB_N, k_lim, tid)
  const kcg_u16* __restrict__ Bs = B + (long)kb * GB_BK * GB_N;
#endif
  const int k_lim = GB_K - kb * GB_BK;                                   // k values left from the segment's start
  // Staging registers between global memory and LDS: tile j waits in set j % GB_STAGES.
  LoaderA la[GB_STAGES];
  LoaderB lb[GB_STAGES];
  constexpr int PA = LoaderA::PER, PB = LoaderB::PER, UNITS = PA + PB;
  constexpr int WA = LoaderA::WEIGHT, WB = LoaderB::WEIGHT, WORK = PA * WA + PB * WB;
  constexpr int KS = GB_BK / GB_KSTEP;           // MFMA k-steps per tile
  constexpr int FS = KS > 1 ? KS - 1 : 1;        // k-steps that carry feeding work

  GB_ACC acc[GB_TM][GB_TN];
#pragma unroll
  for (int i = 0; i < GB_TM; ++i)
#pragma unroll
    for (int j = 0; j < GB_TN; ++j)
#pragma unroll
      for (int v = 0; v < GB_ACCN; ++v) acc[i][j][v] = 0.0f;

#if GB_D2L
  // Operand tiles go from global memory straight into LDS (global_load_lds_dwordx4): one instruction of a wavefront
  // moves 1 KiB, eight rows of 128 bytes, to 1 KiB of consecutive LDS, lane i to byte 16 i.  The swizzle of the rows
  // is applied on the source side: the lane that fills position p of row r fetches chunk p ^ ((r / 2) % 8) of that
  // row, still within the row's one 128-byte line.  No staging registers, no LDS store instructions; a tile's loads
  // are issued behind the barrier that frees its buffer and awaited in front of the next barrier.
  constexpr int UA = GB_BM / 8 / (GB_NT / 64);                                     // instructions per wavefront and tile
  constexpr int UB = GB_BTR ? GB_BK / 2 / (GB_NT / 64) : GB_BN / 8 / (GB_NT / 64);
  static_assert(UA % 2 == 0 && GB_BM % (8 * (GB_NT / 64)) == 0, "direct loads: whole, even numbers of 8-row groups per wavefront");
  static_assert(GB_BTR ? (UB == 4 && GB_NT == 512) : (UB % 2 == 0 && GB_BN % (8 * (GB_NT / 64)) == 0), "direct loads of B: four blocks per wavefront");
  // The instruction is written out: through the builtin the compiler, which cannot tell that the transposing reads
  // that follow touch the other buffer, puts a wait for all outstanding loads in front of each of them.  Here it sees
  // neither the LDS write nor the counter; the waits are the explicit ones in front of the barriers.  The address is a
  // 64-bit scalar base (the same for the whole wavefront) plus a 32-bit lane offset; M0 carries the LDS address.
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  auto lds_dma = [&](const char* base, unsigned lane_off, char* dst) __attribute__((always_inline)) {
    const unsigned l = __builtin_amdgcn_readfirstlane((unsigned)(size_t)(__attribute__((address_space(3))) char*)dst);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" :: "v"(lane_off), "s"(base), "s"(l) : "memory");
  };
  const unsigned d2l_lane = (unsigned)(lane >> 3) * (unsigned)(GB_K * 2) + (unsigned)(((lane & 7) ^ (lane >> 4)) * 16);
  auto d2l = [&](const kcg_u16* g, int row0, int k0, char* sbuf, int t, int upw) __attribute__((always_inline)) {
    const int grp = wave_u * upw + t;                      // group of eight rows within the tile; its parity is that of t
    lds_dma((const char*)(g + (long)(row0 + grp * 8) * GB_K + k0), d2l_lane ^ (unsigned)((t & 1) * 64), sbuf + grp * 8 * GB_ROWB);
  };
#if GB_BTR
  // Row-major weights: a tile row is 512 bytes of consecutive n, one instruction moves two k rows.  Rows are not
  // padded; the 32-byte granule g of row k lies at granule g ^ f(k), f(k) = k % 4 + 4 ((k / 8) % 2): the eight k rows
  // that the transposing reads of two lane groups take together (k0 .. k0 + 3 and k0 + 8 .. k0 + 11) then fall on
  // disjoint banks.  Block b = 4 wave + t holds rows 2 b and 2 b + 1: f = (i / 32) + 2 (t % 2) + 4 (wave % 2).
  const unsigned d2l_lane_b = (unsigned)(lane >> 5) * (unsigned)(GB_N * 2) +
                              (((((unsigned)(lane & 31) >> 1) ^ (unsigned)(lane >> 5) ^ (4u * (wave & 1))) << 1) | (unsigned)(lane & 1)) * 16u;
  auto d2l_b = [&](int k0, char* sbuf, int t) __attribute__((always_inline)) {
    const int blk = wave_u * UB + t;
    lds_dma((const char*)(Bs + (long)(k0 + blk * 2) * GB_N + n0), d2l_lane_b ^ (unsigned)((t & 1) * 64), sbuf + blk * 2 * GB_BROWB);
  };
#endif
  auto d2l_unit = [&](int u, int k0, int buf) __attribute__((always_inline)) {
    if (u < UA) d2l(As, m0, GB_KPOS(k0), sA + buf * (GB_BM * GB_ROWB), u, UA);
#if GB_BTR
    else d2l_b(GB_KPOS(k0), sB + buf * GB_BBUF, u - UA);
#else
    else d2l(Bs, n0, GB_KPOS(k0), sB + buf * GB_BBUF, u - UA, UB);
#endif
  };
#pragma unroll
  for (int u = 0; u < UA + UB; ++u) d2l_unit(u, 0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);                       // vmcnt(0): tile 0 has landed
  __syncthreads();
  if (1 < len) {
#pragma unroll
    for (int u = 0; u < UA + UB; ++u) d2l_unit(u, GB_BK, 1);
  }
#else
  // Prologue: tile 0 through set 0 into LDS buffer 0, then tiles 1..GB_STAGES
  // into their staging sets.
#pragma unroll
  for (int u = 0; u < PA; ++u) GB_LOAD_A(0, u, 0);
#pragma unroll
  for (int u = 0; u < PB; ++u) GB_LOAD_B(0, u, 0);
#pragma unroll
  for (int u = 0; u < PA; ++u) la[0].store_unit(u, sA, GB_ROWB, tid);
#pragma unroll
  for (int u = 0; u < PB; ++u) lb[0].store_unit(u, sB, GB_BTR ? GB_BROWB : GB_ROWB, tid);
#pragma unroll
  for (int j = 1; j <= GB_STAGES; ++j)
    if (GB_SK_UNITS > 0 || j < len) {       // a split segment has at least two k-iterations
#pragma unroll
      for (int u = 0; u < PA; ++u) GB_LOAD_A(j % GB_STAGES, u, j * GB_BK);
#pragma unroll
      for (int u = 0; u < PB; ++u) GB_LOAD_B(j % GB_STAGES, u, j * GB_BK);
    }
  __syncthreads();
#endif

#if GB_M16
  // lane l: row l % 16 of a fragment, chunk 4 ks + l / 16 of the row, at its swizzled position (the row's number
  // inside its group of 16 decides the swizzle: the tiles of a wavefront start at multiples of 16 rows).  With two
  // k-steps per tile the two positions differ in one address bit.
  const int l16 = lane & 15, lq = lane >> 4;
  const int kpos0 = (lq ^ ((l16 >> 1) & 7)) * 16;
  const char* fA = sA + (wm * GB_WTM + l16) * GB_ROWB;
  const char* fB = sB + (wn * GB_WTN + l16) * GB_ROWB;
#define GB_KOFF(ks) (kpos0 ^ ((ks) * 64))
#else
  const char* fA = sA + (wm * GB_WTM + l32) * GB_ROWB + lh * 16;
  const char* fB = sB + (wn * GB_WTN + l32) * GB_ROWB + lh * 16;
#define GB_KOFF(ks) ((ks) * 32)
#endif
#if GB_BTR
  // this lane's address inside a block of 16 k x 32 n of sB[k][n], in the LDS address space so that the reads of a
  // buffer differ from one base register by immediates only
  typedef __attribute__((address_space(3))) char* kcg_lds_ptr;
  typedef short kcg_s16x4 __attribute__((ext_vector_type(4)));
#if GB_M16
  // group q = lane / 16 of a 16x16x32 fragment takes k 4 q .. 4 q + 3 and 16 + 4 q .. 16 + 4 q + 3 of the step (A is laid
  // out to match, see KcgKLoader), all four groups the same 16 columns: the two groups that a read serves together
  // take eight consecutive rows of 32 bytes, which a pitch of 32 modulo 256 bytes puts on disjoint banks
#if GB_D2L
  // natural k order (group q holds k 8 q .. 8 q + 7), unpadded rows with swizzled 32-byte granules (see d2l_b)
  const kcg_lds_ptr bT = (kcg_lds_ptr)sB + (8 * (lane >> 4) + (lane & 15) / 4) * GB_BROWB + 8 * (lane & 3);
  const int bswz = ((lane & 15) >> 2) + 4 * ((lane >> 4) & 1);
  int boff[GB_TN];
#pragma unroll
  for (int j = 0; j < GB_TN; ++j) boff[j] = ((wn * GB_WTN / 16 + j) ^ bswz) * 32;
#else
  const kcg_lds_ptr bT = (kcg_lds_ptr)sB + (4 * (lane >> 4) + (lane & 15) / 4) * GB_BROWB + (wn * GB_WTN + 4 * (lane & 3)) * 2;
#endif
#else
  const kcg_lds_ptr bT = (kcg_lds_ptr)sB + (8 * lh + (lane & 15) / 4) * GB_BROWB + (wn * GB_WTN + 16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
#endif
#endif
  // fragment j of k-step ks out of B buffer buf
  auto read_fb = [&](int buf, int ks, int j) __attribute__((always_inline)) -> GB_FRAG {
#if GB_BTR
#if GB_M16 && GB_D2L
    const kcg_lds_ptr p = bT + buf * GB_BBUF + ks * GB_KSTEP * GB_BROWB + boff[j];
#else
    const kcg_lds_ptr p = bT + buf * GB_BBUF + ks * GB_KSTEP * GB_BROWB + j * (2 * GB_FR);
#endif
    const kcg_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) kcg_s16x4*)p);
    const kcg_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) kcg_s16x4*)(p + (GB_M16 && !GB_D2L ? 16 : 4) * GB_BROWB));
    return __builtin_bit_cast(GB_FRAG, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
#else
    return *(const GB_FRAG*)(fB + buf * GB_BBUF + j * GB_FR * GB_ROWB + GB_KOFF(ks));
#endif
  };
  GB_FRAG fa[2][GB_TM], fb[2][GB_TN];      // the 16x16x32 form uses one set of B fragments
#pragma unroll
  for (int i = 0; i < GB_TM; ++i) fa[0][i] = *(const GB_FRAG*)(fA + i * GB_FR * GB_ROWB + GB_KOFF(0));
#pragma unroll
  for (int j = 0; j < GB_TN; ++j) fb[0][j] = read_fb(0, 0, j);

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
  // mode_c: 1 = steady state (tile kt+1 is written to LDS, tile kt+1+GB_STAGES loaded), 2 = write only,
  // 3 = neither (the last iteration), 0 = decided at run time from the iteration count.
  auto iteration = [&](const int kt, auto par_c, auto mode_c) {
    constexpr int buf = decltype(par_c)::v ? 1 : 0;
    constexpr int mode = decltype(mode_c)::v;
    constexpr bool steady = mode == 1;
    constexpr int set = (buf + 1) % GB_STAGES;
    const bool feed = mode == 0 ? kt + 1 < len : mode != 3;               // tile kt+1 exists: write it to LDS
    const bool fetch = mode == 0 ? kt + 1 + GB_STAGES < len : mode == 1;  // tile kt+1+GB_STAGES exists: load it
    const char* cA = fA + buf * (GB_BM * GB_ROWB);
    char* nA = sA + (buf ^ 1) * (GB_BM * GB_ROWB);
    char* nB = sB + (buf ^ 1) * GB_BBUF;
    const int k2 = (kt + 1 + GB_STAGES) * GB_BK;
#if GB_M16
    // The MFMAs of a step go column by column over the wavefront's tiles: the B fragment of column j has its last use
    // in MFMA (last row, j) and is read again for the next k-step right behind it, GB_TM * (GB_TN - 1) MFMAs ahead of its
    // first use there (in the tile's last step: for the first step of the next tile, out of the other buffer).  The A
    // fragments of the next step go into their second set at the start of the step.  The tile's barrier stands at the
    // start of its last step.  Feeding: with direct loads (GB_D2L) the instructions that bring tile kt+2 into the buffer
    // that the barrier has just freed are dealt out between the columns of the last step (all of them right behind the
    // barrier measured 5 % slower), and the wait for tile kt+1 stands in front of the barrier; through registers, the
    // LDS stores of tile kt+1 and the loads of tile kt+2 go between the columns of the first step (GB_M16_DEAL) or in
    // front of it.
#ifndef GB_M16_DEAL
#define GB_M16_DEAL 1
#endif
    static_assert(KS % 2 == 0, "the A fragment sets alternate per k-step");
    auto feed_unit = [&](int u) __attribute__((always_inline)) {
      if (u < PA) {
        if (feed) la[set].store_unit(u, nA, GB_ROWB, tid);
        if (fetch) GB_LOAD_A(set, u, k2);
      } else {
        if (feed) lb[set].store_unit(u - PA, nB, GB_BTR ? GB_BROWB : GB_ROWB, tid);
        if (fetch) GB_LOAD_B(set, u - PA, k2);
      }
    };
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      const bool last = ks == KS - 1;
      __builtin_amdgcn_sched_barrier(0);
      if (!last) {
#pragma unroll
        for (int i = 0; i < GB_TM; ++i) fa[nxt][i] = *(const GB_FRAG*)(cA + i * GB_FR * GB_ROWB + GB_KOFF(ks + 1));
      }
      if (!GB_D2L && !GB_M16_DEAL && ks < FS) {
#pragma unroll
        for (int u = 0; u < UNITS; ++u)
          if ((u < PA ? u * WA : PA * WA + (u - PA) * WB) * FS / WORK == ks) feed_unit(u);
      }
      if (last) {
#if GB_D2L
        __builtin_amdgcn_s_waitcnt(0x0F70);                 // vmcnt(0): this wavefront's share of tile kt+1 has landed
#endif
        __syncthreads();
        if (feed) {
#pragma unroll
          for (int i = 0; i < GB_TM; ++i)
            fa[nxt][i] = *(const GB_FRAG*)(fA + (buf ^ 1) * (GB_BM * GB_ROWB) + i * GB_FR * GB_ROWB + GB_KOFF(0));
        }
      }
#pragma unroll
      for (int j = 0; j < GB_TN; ++j) {
#pragma unroll
        for (int i = 0; i < GB_TM; ++i) {
          __builtin_amdgcn_sched_barrier(0);
          acc[i][j] = GB_MFMA(fa[cur][i], fb[0][j], acc[i][j], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (!last) fb[0][j] = read_fb(buf, ks + 1, j);
        else if (feed) fb[0][j] = read_fb(buf ^ 1, 0, j);
#if GB_D2L
        if (last && kt + 2 < len) {
#pragma unroll
          for (int u = 0; u < UA + UB; ++u)
            if (u * GB_TN / (UA + UB) == j) d2l_unit(u, (kt + 2) * GB_BK, buf);
        }
#else
        if (GB_M16_DEAL && ks < FS) {
#pragma unroll
          for (int u = 0; u < UNITS; ++u)
            if ((u < PA ? u * WA : PA * WA + (u - PA) * WB) * FS / WORK == ks &&
                (u - (ks * UNITS + FS - 1) / FS + UNITS) % UNITS * GB_TN / UNITS == j) feed_unit(u);
        }
#endif
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    return;
#endif
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      __builtin_amdgcn_sched_barrier(0);
      if (ks + 1 < KS) {
#pragma unroll
        for (int i = 0; i < GB_TM; ++i) fa[nxt][i] = *(const GB_FRAG*)(cA + i * 32 * GB_ROWB + (ks + 1) * 32);
#pragma unroll
        for (int j = 0; j < GB_TN; ++j) fb[nxt][j] = read_fb(buf, ks + 1, j);
      }
      if (ks < FS) {
#pragma unroll
        for (int u = 0; u < UNITS; ++u)
          if ((u < PA ? u * WA : PA * WA + (u - PA) * WB) * FS / WORK == ks) {   // units dealt to the steps by weight
            if (u < PA) {
              if (feed) la[set].store_unit(u, nA, GB_ROWB, tid);
              if (fetch) GB_LOAD_A(set, u, k2);
            } else {
              if (feed) lb[set].store_unit(u - PA, nB, GB_BTR ? GB_BROWB : GB_ROWB, tid);
              if (fetch) GB_LOAD_B(set, u - PA, k2);
            }
          }
      }
      if (ks == KS - 1) {
        __syncthreads();
        if (feed) {
#pragma unroll
          for (int i = 0; i < GB_TM; ++i)
            fa[nxt][i] = *(const GB_FRAG*)(fA + (buf ^ 1) * (GB_BM * GB_ROWB) + i * 32 * GB_ROWB);
#pragma unroll
          for (int j = 0; j < GB_TN; ++j)
            fb[nxt][j] = read_fb(buf ^ 1, 0, j);
        }
      }
#if !GB_INTERLEAVE
      __builtin_amdgcn_sched_barrier(0);
#endif
#if GB_SETPRIO
      __builtin_amdgcn_s_setprio(GB_SETPRIO);
#endif
#pragma unroll
      for (int i = 0; i < GB_TM; ++i)
#pragma unroll
        for (int j = 0; j < GB_TN; ++j)
          acc[i][j] = GB_MFMA(fa[cur][i], fb[cur][j], acc[i][j], 0, 0, 0);
#if GB_SETPRIO
      __builtin_amdgcn_s_setprio(0);
#endif
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
  int kt = 0;                                         // counts from the segment's first k-iteration
  for (; kt + 2 + GB_STAGES < len; kt += 2) {        // both iterations of the pair feed and fetch
    iteration(kt, KcgBool<false>{}, KcgInt<1>{});
    iteration(kt + 1, KcgBool<true>{}, KcgInt<1>{});
  }
#if GB_SK_UNITS > 0
  // a split segment has an even number of iterations (and one staging set): two are left, of known kinds
  iteration(kt, KcgBool<false>{}, KcgInt<2>{});
  iteration(kt + 1, KcgBool<true>{}, KcgInt<3>{});
#else
  for (; kt < len; ++kt) {
    if (kt & 1) iteration(kt, KcgBool<true>{}, KcgInt<0>{});
    else iteration(kt, KcgBool<false>{}, KcgInt<0>{});
  }
#endif

#if GB_SK_UNITS > 0
  // ---- a segment that is not a whole tile: slot, fence, count in; the last one in adds up and goes on to the stores ----
  bool store_tile = true;
  if (len < GB_KT) {
    typedef float kcg_f32x4 __attribute__((ext_vector_type(4)));
    kcg_f32x4* slots = (kcg_f32x4*)(W + 1024);
    constexpr long SLOT = (long)GB_BM * GB_BN / 4;               // float4 per slot
    kcg_f32x4* mine = slots + (long)(sk_u * 2 + segment) * SLOT;
#pragma unroll
    for (int i = 0; i < GB_TM; ++i)
#pragma unroll
      for (int j = 0; j < GB_TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          kcg_f32x4 v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
          mine[((i * GB_TN + j) * 4 + q) * GB_NT + tid] = v;
        }
    __threadfence();
    __syncthreads();
    // the units whose runs overlap this tile's k-iterations, in k order
    const int first_unit = (sk_lt * GB_KT) / GB_SK_PER;
    const int last_unit = (sk_lt * GB_KT + GB_KT - 1) / GB_SK_PER;
    unsigned* counter = W + (pid - GB_SK_FULL);
    if (tid == 0) kcg_sk_arrived = atomicAdd(counter, 1u);
    __syncthreads();
    store_tile = kcg_sk_arrived == (unsigned)(last_unit - first_unit);
    if (store_tile) {
      __threadfence();
      if (tid == 0) atomicExch(counter, 0u);                      // the next launch finds the counter at zero
      for (int unit = first_unit; unit <= last_unit; ++unit) {
        const int their_first_tile = (unit * GB_SK_PER) / GB_KT;
        const int their_u = GB_SK_XCD ? unit * 8 + sk_group : unit;
        const kcg_f32x4* theirs = slots + (long)(their_u * 2 + (sk_lt - their_first_tile)) * SLOT;
#pragma unroll
        for (int i = 0; i < GB_TM; ++i)
#pragma unroll
          for (int j = 0; j < GB_TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const kcg_f32x4 v = theirs[((i * GB_TN + j) * 4 + q) * GB_NT + tid];
#pragma unroll
              for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] = (unit == first_unit ? 0.0f : acc[i][j][4 * q + e]) + v[e];
            }
      }
    }
  }
  if (store_tile)
#endif
  {
  // ---- epilogue: lane l, register v -> row 8*(v/4) + 4*(l/32) + v%4, column l%32 (32x32 tiles);
  //      row 4*(l/16) + v, column l%16 (16x16 tiles) ----
#if GB_STAGE_C
  // Whole rows.  Out of the 16 x 16 accumulator tiles a store instruction writes 16 values of each of four rows (64
  // bytes in fp32, 32 in a 16-bit type: two bytes a lane), and the pieces of a 128-byte line leave at different times.
  // Here the 256 x 256 tile goes through LDS, the k loop's 128 KiB: in two halves of 128 rows as fp32 (the wavefront's
  // tile rows 0-1, then 2-3: every wavefront takes part in both), at once in a 16-bit type.  Row r of the staged part is
  // 256 values, its chunk c of 16 values at chunk c ^ ((r / 4) % 4), so that the four rows a wavefront writes at a time
  // fall on different banks; then every lane stores 16 bytes of a row, a wavefront one or two whole rows at a time
  // (GB_STAGE_C 2: with the non-temporal hint).  16-bit results gain 2-3 % (4096 x 11008 x 4096: 0.280 against 0.287 ms);
  // fp32 results, whose pieces are 64 bytes already, gain nothing in this kernel and keep the plain epilogue.
  {
#if GB_OUT_BF16
    typedef kcg_u16 stage_t;
#else
    typedef float stage_t;
#endif
    constexpr int ES = (int)sizeof(stage_t), PASSES = ES == 4 ? 2 : 1, RP = 256 / PASSES;    // rows per pass
    constexpr int LPR = 256 * ES / 16, RPI = 64 / LPR, EPL = 16 / ES;                        // lanes per row, rows per instruction, values per lane
    stage_t* stage = (stage_t*)kcg_smem;
    const int lq = lane >> 4, l16 = lane & 15;
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
      __syncthreads();
#pragma unroll
      for (int ii = 0; ii < GB_TM / PASSES; ++ii)
#pragma unroll
        for (int j = 0; j < GB_TN; ++j)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int i = pass * (GB_TM / PASSES) + ii;
            const float r = GB_RELU ? fmaxf(acc[i][j][v], 0.0f) : acc[i][j][v];
            const int row = wm * (GB_WTM / PASSES) + 16 * ii + 4 * lq + v, col = wn * GB_WTN + 16 * j + l16;
#if GB_OUT_BF16
            stage[row * 256 + (col ^ (16 * lq))] = GB_TO16(r);
#else
            stage[row * 256 + (col ^ (16 * lq))] = r;
#endif
          }
      __syncthreads();
#pragma unroll
      for (int x = 0; x < RP / 8 / RPI; ++x) {
        const int row = wave * (RP / 8) + x * RPI + lane / LPR;
        const int col = (lane % LPR) * EPL;
        const kcg_f32x4 val = *(const kcg_f32x4*)(stage + row * 256 + (col ^ (16 * ((row >> 2) & 3))));
        const int trow = PASSES == 2 ? (row / (GB_WTM / 2)) * GB_WTM + (GB_WTM / 2) * pass + row % (GB_WTM / 2) : row;
#if GB_STAGE_C == 2
        __builtin_nontemporal_store(val, (kcg_f32x4*)(C + (long)(m0 + trow) * GB_N + n0 + col));
#else
        *(kcg_f32x4*)(C + (long)(m0 + trow) * GB_N + n0 + col) = val;
#endif
      }
    }
  }
#else
#pragma unroll
  for (int i = 0; i < GB_TM; ++i)
#pragma unroll
    for (int j = 0; j < GB_TN; ++j) {
      const int col = n0 + wn * GB_WTN + j * GB_FR + (GB_M16 ? (lane & 15) : l32);
#pragma unroll
      for (int v = 0; v < GB_ACCN; ++v) {
        const int row = GB_M16 ? m0 + wm * GB_WTM + i * 16 + 4 * (lane >> 4) + v
                               : m0 + wm * GB_WTM + i * 32 + 8 * (v / 4) + 4 * lh + (v % 4);
#if GB_EDGE
        if (row < GB_M && col < GB_N)
#endif
        {
#if GB_OUT_BF16
          C[(long)row * GB_N + col] = GB_TO16(GB_RELU ? fmaxf(acc[i][j][v], 0.0f) : acc[i][j][v]);
#else
          C[(long)row * GB_N + col] = GB_RELU ? fmaxf(acc[i][j][v], 0.0f) : acc[i][j][v];
#endif
        }
      }
    }
#endif   // GB_STAGE_C
  }
#if GB_SK_UNITS > 0
  if (segment + 1 < num_segments) __syncthreads();   // the next segment reuses the LDS tiles and kcg_sk_arrived
#endif
  }   // segment
}
#undef GB_LOAD_A
#undef GB_LOAD_B
#undef GB_KOFF
#undef GB_FR
#undef GB_KSTEP
#undef GB_ACC
#undef GB_ACCN
#ifdef GB_M16_DEFAULTED
#undef GB_M16
#undef GB_M16_DEFAULTED
#endif
#ifdef GB_D2L_DEFAULTED
#undef GB_D2L
#undef GB_D2L_DEFAULTED
#endif
#ifdef GB_STAGE_C_DEFAULTED
#undef GB_STAGE_C
#undef GB_STAGE_C_DEFAULTED
#endif
#undef GB_NT
#undef GB_WTM
#undef GB_WTN
#undef GB_TM
#undef GB_TN
#undef GB_ROWB
#undef GB_KT
#undef GB_GUARD
#undef GB_BROWB
#undef GB_BPAD
#undef GB_BBUF
#ifdef GB_BTR_DEFAULTED
#undef GB_BTR
#undef GB_BTR_DEFAULTED
#endif
#undef GB_KROT
#ifdef GB_KROT_DEFAULTED
#undef GB_KROT_ON
#undef GB_KROT_DEFAULTED
#endif
#undef GB_KPOS
#undef GB_TILES
#undef GB_SK_TAIL
#undef GB_SK_XCD
#undef GB_SK_GROUPS
#undef GB_SK_GTILES
#undef GB_SK_GUNITS
#undef GB_SK_PER
#undef GB_SK_PER0
#undef GB_FRAG
#undef GB_MFMA
#undef GB_TO16
#ifdef GB_F16_DEFAULTED
#undef GB_F16
#undef GB_F16_DEFAULTED
#endif
#ifdef GB_SETPRIO_DEFAULTED
#undef GB_SETPRIO
#undef GB_SETPRIO_DEFAULTED
#endif
#ifdef GB_SK_DEFAULTED
#undef GB_SK_UNITS
#undef GB_SK_FULL
#undef GB_SK_DEFAULTED
#endif
#ifdef GB_STAGGER_DEFAULTED
#undef GB_STAGGER
#undef GB_STAGGER_DEFAULTED
#endif
