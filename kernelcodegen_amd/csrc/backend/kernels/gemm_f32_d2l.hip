// ---- fp32 GEMM on v_mfma_f32_32x32x2_f32, operand tiles straight from global memory into LDS ----------------------
// C[b] = A[b] * B[b]: A [M][K], B [K][N], C [M][N], all row-major fp32; whole 256 x 256 x 16 tiles only (the emitter
// falls back to gemm_f32.hip for every other case).  Parameters:
//   GD_NAME                      kernel symbol
//   GD_M GD_N GD_K GD_BATCH      problem: multiples of 256, 256 and 16
//   GD_GROUP_M                   tile rows per L2 strip
//   GD_RELU                      1: fused max(0, .) epilogue
//
// Sixteen wavefronts (4 x 4) of 64 x 64 results = 2 x 2 MFMA tiles of 32 x 32.  What gemm_f32.hip spends between
// global memory and LDS - a float4 per operand and thread in registers, four scattered LDS stores to turn a
// k-contiguous row of A into the k-major tile - is not there: a k-tile is two global_load_lds_dwordx4 per wavefront,
// one 1 KiB block of each operand, and both tiles lie in LDS as they lie in memory.
//
// A in LDS: 256 rows of 64 bytes (16 k), no padding; the 16-byte chunk c (four k) of row m lies at position
// c ^ ((m / 4) % 4).  A lane of an MFMA holds row m = lane % 32 and, with one ds_read_b128, the four k of chunk
// 2 u + lane / 32 (u = 0, 1: the halves of the k-tile); the sixteen lanes that such a read serves in one pass (rows
// 0-3, 12-15, 20-27 of a 32-row block, then the rest) then fall on sixteen different groups of four banks.  The swizzle
// is applied on the source side of the load: lane i of a block writes 16 bytes at 16 i, that is position i % 4 of row
// i / 4, and fetches the chunk that belongs there.
// B in LDS: 16 rows (k) of 1 KiB, as in memory; a lane reads one float of row k at column n = lane % 32 of its block.
// An MFMA sums over the two k that its two half-waves hold; which two is free as long as both operands agree: MFMA e
// of half u takes k = 8 u + e from the lower half-wave and 8 u + 4 + e from the upper.
//
// Pipeline.  One barrier per k-tile, in front of the MFMAs of its second half: by then a wavefront has read all its
// fragments of the tile (so the buffer is free) and has waited for its own two loads of the next tile (so that tile is
// complete once everyone has arrived).  Behind it the first half's fragments of the next tile are read; the loads of
// the tile after next start at the top of the next tile.  Fragments are read half a k-tile ahead into a second set.
#ifndef KCG_GEMM32D_HELPERS
#define KCG_GEMM32D_HELPERS
template <bool B> struct KcgBool32d { static constexpr bool v = B; };
#endif
#if (GD_M % 256) || (GD_N % 256) || (GD_K % 16)
#error "gemm_f32_d2l: whole 256 x 256 x 16 tiles only"
#endif
#define GD_KT (GD_K / 16)

extern "C" __global__ __launch_bounds__(1024)
void GD_NAME(const float* __restrict__ A, const float* __restrict__ B, float* __restrict__ C) {
  constexpr int TILE = 256 * 16 * 4;                      // bytes of an operand tile
  constexpr int B_AT = 2 * TILE;                          // A's two buffers, then B's two
  __shared__ __attribute__((aligned(1024))) char kcg_smem[4 * TILE];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int wm = wave >> 2, wn = wave & 3;
  const int l32 = lane & 31, lh = lane >> 5;

  const int tiles_m = GD_M / 256, tiles_n = GD_N / 256;
  int tile_m, tile_n;
  kcg_tile_coords(blockIdx.x, tiles_m, tiles_n, GD_GROUP_M, tile_m, tile_n);
  // (the division in kcg_tile_coords runs on the vector unit: the tile origins go back into scalar registers here, the
  // load instructions below take their base addresses from there)
  const int m0 = __builtin_amdgcn_readfirstlane(tile_m * 256), n0 = __builtin_amdgcn_readfirstlane(tile_n * 256);
  const long batch = blockIdx.y;
  A += batch * (long)GD_M * GD_K;
  B += batch * (long)GD_K * GD_N;
  C += batch * (long)GD_M * GD_N;

  // ---- loads: wavefront w moves rows 16 w .. 16 w + 15 of the A tile and row (k) w of the B tile ----
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)kcg_smem;
  const unsigned lds_wave = __builtin_amdgcn_readfirstlane(lds_base + wave_u * 1024);
  const unsigned a_lane = (unsigned)(lane >> 2) * (unsigned)(GD_K * 4) + (unsigned)(((lane & 3) ^ ((lane >> 4) & 3)) * 16);
  const unsigned b_lane = (unsigned)lane * 16u;
  const char* rowsA = (const char*)(A + (long)(m0 + wave_u * 16) * GD_K);
  const char* rowsB = (const char*)(B + (long)wave_u * GD_N + n0);
  auto dma = [&](int kt, int buf) __attribute__((always_inline)) {
    unsigned w = lds_wave;
    asm volatile("" : "+s"(w));                            // the two sums are formed here each time, not kept
    const unsigned dst_a = w + (unsigned)(buf * TILE), dst_b = w + (unsigned)(B_AT + buf * TILE);
    const char* src_a = rowsA + (long)kt * 64;
    const char* src_b = rowsB + (long)kt * 16 * GD_N * 4;
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(a_lane), "s"(src_a), "s"(dst_a) : "memory");
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(b_lane), "s"(src_b), "s"(dst_b) : "memory");
  };

  // ---- fragments of half u of the tile in buffer buf ----
  const int ma = wm * 64 + l32;                            // the lane's row of A's first block; the second is 32 further
  const int sw = (ma >> 2) & 3;                            // the same for both blocks: 32 rows are eight groups of four
  const char* fA = kcg_smem + ma * 64;
  const char* fB = kcg_smem + B_AT + lh * 4096 + (wn * 64 + l32) * 4;
  auto read_fragments = [&](int buf, int u, kcg_f32x4 (&a)[2], float (&b)[2][4]) __attribute__((always_inline)) {
    const int pos = ((2 * u + lh) ^ sw) * 16;
#pragma unroll
    for (int i = 0; i < 2; ++i) a[i] = *(const kcg_f32x4*)(fA + buf * TILE + i * 32 * 64 + pos);
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) b[j][e] = *(const float*)(fB + buf * TILE + (8 * u + e) * 1024 + j * 128);
  };

  kcg_f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // ---- prologue: tile 0 into buffer 0, wait, first fragments ----
  dma(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);                      // vmcnt(0)
  __syncthreads();
  kcg_f32x4 fa[2][2];
  float fb[2][2][4];
  read_fragments(0, 0, fa[0], fb[0]);

  auto half = [&](kcg_f32x4 (&a)[2], float (&b)[2][4]) __attribute__((always_inline)) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][e], b[j][e], acc[i][j], 0, 0, 0);
  };
  auto tile = [&](const int kt, auto par_c) {
    constexpr int par = decltype(par_c)::v ? 1 : 0;
    const bool more = kt + 1 < GD_KT;
    if (more) dma(kt + 1, par ^ 1);                        // the other buffer is free since the last barrier
    __builtin_amdgcn_sched_barrier(0);
    read_fragments(par, 1, fa[1], fb[1]);
    half(fa[0], fb[0]);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0F70);                    // vmcnt(0): this wavefront's blocks of tile kt+1 have landed
    __syncthreads();                                       // (its wait for LDS covers the last fragment reads of tile kt)
    if (more) read_fragments(par ^ 1, 0, fa[0], fb[0]);
    half(fa[1], fb[1]);
    __builtin_amdgcn_sched_barrier(0);
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
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn * 64 + j * 32 + l32;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 64 + i * 32 + 8 * (v / 4) + 4 * lh + (v % 4);
        float o = acc[i][j][v];
#if GD_RELU
        o = fmaxf(0.0f, o);
#endif
        C[(long)row * GD_N + col] = o;
      }
    }
}
#undef GD_KT
