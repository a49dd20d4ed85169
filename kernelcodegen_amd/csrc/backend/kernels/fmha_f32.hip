// ---- fused attention forward in fp32 on v_mfma_f32_32x32x2_f32 ----------------
// O[b, h] = softmax(scale * Q[b, h] K[b, h]^T [+ causal mask]) V[b, h]; Q, K, V, O are [B][H][S][D] fp32, dense.
// Both products run on the full-precision fp32 MFMA and the probabilities stay fp32, so the result keeps the fp32
// bar (1e-5 relative Frobenius against fp64) that the unfused nests of the Frontend meet (reference graph:
// test/test.cc:107-147, BatchMatmul NT -> Softmax -> BatchMatmul NN on fp32 tensors).
// Parameters:
//   FF_NAME                kernel symbol
//   FF_B FF_H FF_S FF_D    problem; FF_D a multiple of 32; any FF_S >= 1
//   FF_WAVES               wavefronts per workgroup, 32 queries each (FF_BR = 32 * FF_WAVES queries per workgroup)
//   FF_BC                  keys per LDS tile, a multiple of 32
//   FF_CAUSAL              1: key j contributes to query i only if j <= i
//   FF_C                   softmax scale times log2(e), a float literal (the exponentials are taken in base 2)
//   FF_OCC                 workgroups per CU the register allocation has to leave room for
//   FF_D2L                 1 (whole tiles only: FF_S a multiple of FF_BR and FF_BC; FF_D 64 or 128): the K and V tiles go
//                          from global memory straight into LDS, two buffers each, one barrier per tile (see below)
//
// A wavefront owns 32 queries and computes the TRANSPOSED score tile S^T = K Q^T, 32 keys x 32 queries: K rows from
// LDS are the MFMA's A operand, the wavefront's own Q rows (registers, scaled once) its B operand.  Lane l then holds,
// for query l % 32, the scores of keys 8 (v / 4) + 4 (l / 32) + v % 4, v = 0..15: a row maximum or row sum is 16
// values of one lane plus one exchange between the two half-waves.  The same 16 registers, once they hold the
// probabilities, are directly the B operand of O^T += V^T P^T: the sum over the 32 keys of a tile may run in any
// order, so step v takes the keys the two half-waves hold in register v, and the A operand reads V[that key][d] from
// LDS.  No value of S or P ever leaves the registers.
//
// K's k-steps are ordered likewise: the half-wave l / 32 reads d = 8 g + 4 (l / 32) + {0..3} as one 16-byte LDS
// read that feeds four MFMAs.  K rows are padded to FF_D + 4 floats (16 consecutive keys' 16-byte reads fall into 16
// different groups of four banks), V rows to FF_D + 8 (the two half-waves of a V read take rows four keys apart,
// which that pitch puts 32 banks apart).
//
// FF_D2L.  A K or V tile is FF_BC rows of FF_D floats that lie one behind the other in memory, so it is FF_BC FF_D / 256
// blocks of 1 KiB, each one global_load_lds_dwordx4 of a wavefront (lane i writes 16 bytes at 16 i of the block); the
// blocks of both tiles are dealt round-robin to the wavefronts.  The next tile is loaded into the other buffer while
// this one is multiplied: no staging registers, no LDS stores, and one barrier per tile instead of two with the load
// between them.  Rows are not padded; the lane that fills a position fetches the chunk that belongs there:
//   K: the 16-byte chunk c of row r lies at chunk c ^ (r % 16) (the sixteen rows whose 16-byte reads are served in one
//      pass, rows 0-3, 12-15, 20-27 of a 32-row block and then the rest, fall on sixteen groups of four banks);
//   V: the 32 floats [32 j, 32 j + 32) of row r lie at j ^ ((r / 4) % 2): the two half-waves of a V read take rows four
//      keys apart, which this puts 32 banks apart.
//
// Without FF_D2L the K and V tiles are loaded by the whole workgroup between two barriers; two workgroups per CU (FF_OCC = 2) keep
// the matrix pipes busy while one of them loads.  Workgroups are numbered so that all query tiles of a head run on
// one XCD (ids are dealt round-robin to the 8 XCDs): a head's K and V come from HBM once.
#define FF_NT (64 * FF_WAVES)
#define FF_BR (32 * FF_WAVES)
#ifndef FF_D2L
#define FF_D2L 0
#define FF_D2L_DEFAULTED
#endif
#if FF_D2L
#define FF_KROW FF_D
#define FF_VROW FF_D
#else
#define FF_KROW (FF_D + 4)
#define FF_VROW (FF_D + 8)
#endif
#define FF_NQ ((FF_S + FF_BR - 1) / FF_BR)
// FF_PAIR 1 (causal mask, an even number of query tiles, the last of which may be partly filled): a workgroup takes two query tiles of its head one after
// the other, tile FF_NQ - 1 - j and then tile j, so that every workgroup walks FF_NQ + 1 groups of keys; the grid is half
// as large.  Without it a head's workgroups differ FF_NQ-fold in length.
#ifndef FF_PAIR
#define FF_PAIR 0
#define FF_PAIR_DEFAULTED
#endif
#if FF_PAIR && (!FF_CAUSAL || (FF_NQ % 2) != 0)
#error "fmha_f32: FF_PAIR needs the causal mask and an even number of query tiles"
#endif
#define FF_SLOTS (FF_PAIR ? FF_NQ / 2 : FF_NQ)
#define FF_RAGGED ((FF_S % FF_BR) != 0 || (FF_S % FF_BC) != 0)
#if (FF_D % 32) || (FF_BC % 32) || FF_WAVES < 1 || FF_WAVES > 16
#error "fmha_f32: head dim and key tile must be multiples of 32, 1..16 wavefronts"
#endif
#if FF_D2L && (FF_RAGGED || (FF_D != 64 && FF_D != 128))
#error "fmha_f32: direct loads into LDS need whole tiles and a head dim of 64 or 128"
#endif

extern "C" __global__ __launch_bounds__(FF_NT, FF_OCC)
void FF_NAME(const float* __restrict__ Q, const float* __restrict__ K, const float* __restrict__ V, float* __restrict__ O) {
#if FF_D2L
  __shared__ __attribute__((aligned(1024))) float sKV[4 * FF_BC * FF_D];   // K's two buffers, then V's two
#else
  __shared__ __attribute__((aligned(16))) float sK[FF_BC * FF_KROW];
  __shared__ __attribute__((aligned(16))) float sV[FF_BC * FF_VROW];
#endif
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, lh = lane >> 5;
  constexpr int HEADS = FF_B * FF_H;
  int head, slot;
  {
    const int bid = blockIdx.x;
    if (HEADS % 8 == 0) { head = (bid & 7) + 8 * (bid / (8 * FF_SLOTS)); slot = (bid >> 3) % FF_SLOTS; }
    else { head = bid / FF_SLOTS; slot = bid % FF_SLOTS; }
  }
  const long base = (long)head * FF_S * FF_D;
  const float* __restrict__ q = Q + base;
  const float* __restrict__ k = K + base;
  const float* __restrict__ v = V + base;
  float* __restrict__ o = O + base;
#pragma unroll 1
  for (int pass = 0; pass < (FF_PAIR ? 2 : 1); ++pass) {
  // under the mask the query tiles with the most keys start first; a pair's second tile is the short one
  const int qt = FF_CAUSAL ? (FF_PAIR && pass ? slot : FF_NQ - 1 - slot) : slot;
  const int q0 = qt * FF_BR + wave * 32;            // the wavefront's first query
  const int qrow = q0 + l32;                        // this lane's query: column of both accumulator tiles
  const float NEG_INF = -__builtin_inff();

  // Q as the B operand of step (g, j): B[k = l / 32][n = l % 32] = Q[qrow][8 g + 4 (l / 32) + j], times scale log2(e)
  kcg_f32x4 qf[FF_D / 8];
  {
    const int r = (FF_RAGGED && qrow >= FF_S) ? FF_S - 1 : qrow;     // a row past the end reads the last one; never stored
    const float* qp = q + (long)r * FF_D + 4 * lh;
#pragma unroll
    for (int g = 0; g < FF_D / 8; ++g) qf[g] = *(const kcg_f32x4*)(qp + 8 * g) * FF_C;
  }
  kcg_f32x16 acc[FF_D / 32];
#pragma unroll
  for (int db = 0; db < FF_D / 32; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[db][e] = 0.0f;
  float m = NEG_INF, l = 0.0f;        // running maximum (base-2 exponent units) and this half-wave's part of the running sum

  // keys the workgroup walks: all of them, or up to its last query under the mask
  const int last_query = (qt * FF_BR + FF_BR - 1) < (FF_S - 1) ? (qt * FF_BR + FF_BR - 1) : (FF_S - 1);
  const int kend = FF_CAUSAL ? last_query + 1 : FF_S;
#if FF_D2L
  constexpr int TILE_B = FF_BC * FF_D * 4;            // bytes of a tile
  constexpr int NBLK = TILE_B / 1024;                 // blocks of 1 KiB per tile
  constexpr int CPR = FF_D / 4, RPB = 1024 / (FF_D * 4);   // 16-byte chunks per row, rows per block
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) char*)sKV;
  // lane i of a block: row i / CPR of the block, position i % CPR; the chunk it fetches is that position swizzled with the
  // row's number in the tile, RPB b + i / CPR for block b: the part that depends on b is applied per block below
  const unsigned k_lane = (unsigned)(lane / CPR) * (unsigned)(FF_D * 4) + (unsigned)(((lane % CPR) ^ (lane / CPR)) * 16);
  const unsigned v_lane = (unsigned)lane * 16u;
  const char* kbytes = (const char*)k;
  const char* vbytes = (const char*)v;
  auto dma_tile = [&](int k0, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int x = 0; x < (2 * NBLK + FF_WAVES - 1) / FF_WAVES; ++x) {
      const int blk = wave_u + x * FF_WAVES;          // wave-uniform: K's blocks, then V's
      if ((2 * NBLK) % FF_WAVES == 0 || blk < 2 * NBLK) {
        const bool is_k = blk < NBLK;
        const int b = is_k ? blk : blk - NBLK;
        const unsigned dst = __builtin_amdgcn_readfirstlane(lds_base + (unsigned)((is_k ? 0 : 2 * TILE_B) + buf * TILE_B + b * 1024));
        const char* src = (is_k ? kbytes : vbytes) + (long)k0 * (FF_D * 4) + (long)b * 1024;
        // K: chunk ^ ((RPB b) % 16); V: the halves of 32 floats (8 chunks) exchanged in rows 4-7 of every eight
        const unsigned lane_off = is_k ? k_lane ^ (unsigned)(((RPB * b) % 16) * 16)
                                       : v_lane ^ (unsigned)((((RPB * b + (int)(lane / CPR)) >> 2) & 1) * 128);
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(lane_off), "s"(src), "s"(dst) : "memory");
      }
    }
  };
  dma_tile(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0F70);                 // vmcnt(0)
  __syncthreads();
  int buf = 0;
#endif
  for (int k0 = 0; k0 < kend; k0 += FF_BC) {
#if FF_D2L
    if (k0 + FF_BC < kend) dma_tile(k0 + FF_BC, buf ^ 1);     // the other buffer is free since the last barrier
    const float* sK = sKV + buf * (FF_BC * FF_D);
    const float* sV = sKV + (2 + buf) * (FF_BC * FF_D);
#else
    __syncthreads();                                  // everybody has finished with the tile before
    constexpr int VECS = FF_BC * (FF_D / 4);          // 16-byte vectors per tile
#pragma unroll
    for (int i0 = 0; i0 < VECS; i0 += FF_NT) {
      const int i = i0 + tid;
      if (VECS % FF_NT == 0 || i < VECS) {
        const int row = i / (FF_D / 4), c = i % (FF_D / 4);
        int gr = k0 + row;
        if (FF_RAGGED && gr >= FF_S) gr = FF_S - 1;  // keys past the end are masked below
        const kcg_f32x4 kv = *(const kcg_f32x4*)(k + (long)gr * FF_D + 4 * c);
        const kcg_f32x4 vv = *(const kcg_f32x4*)(v + (long)gr * FF_D + 4 * c);
        *(kcg_f32x4*)(sK + row * FF_KROW + 4 * c) = kv;
        *(kcg_f32x4*)(sV + row * FF_VROW + 4 * c) = vv;
      }
    }
    __syncthreads();
#endif
#pragma unroll 1
    for (int sub = 0; sub < FF_BC / 32; ++sub) {
      const int kb = k0 + sub * 32;                   // first key of the 32 this step takes
      if (kb >= kend) break;
      if (FF_CAUSAL && kb > q0 + 31) break;           // wholly behind this wavefront's queries (the same for all its lanes)
      // ---- S^T = K Q^T ----
      kcg_f32x16 s;
#pragma unroll
      for (int e = 0; e < 16; ++e) s[e] = 0.0f;
#if FF_D2L
      const float* kr = sK + (sub * 32 + l32) * FF_KROW;
#else
      const float* kr = sK + (sub * 32 + l32) * FF_KROW + 4 * lh;
#endif
#pragma unroll
      for (int g = 0; g < FF_D / 8; ++g) {
#if FF_D2L
        const kcg_f32x4 kf = *(const kcg_f32x4*)(kr + 4 * ((2 * g + lh) ^ (l32 & 15)));
#else
        const kcg_f32x4 kf = *(const kcg_f32x4*)(kr + 8 * g);
#endif
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[0], qf[g][0], s, 0, 0, 0);
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[1], qf[g][1], s, 0, 0, 0);
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[2], qf[g][2], s, 0, 0, 0);
        s = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[3], qf[g][3], s, 0, 0, 0);
      }
      // ---- mask: keys behind the query, keys past the end ----
      if ((FF_CAUSAL && kb + 31 > q0) || (FF_RAGGED && kb + 32 > FF_S)) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = kb + 8 * (e / 4) + 4 * lh + (e % 4);
          if ((FF_CAUSAL && key > qrow) || (FF_RAGGED && key >= FF_S)) s[e] = NEG_INF;
        }
      }
      // ---- online softmax; the first key is never masked, so the maximum is finite from the first tile on ----
      float tm = s[0];
#pragma unroll
      for (int e = 1; e < 16; ++e) tm = fmaxf(tm, s[e]);
      tm = fmaxf(tm, __shfl_xor(tm, 32, KCG_WAVE));
      const float mn = fmaxf(m, tm);
      const float alpha = __builtin_amdgcn_exp2f(m - mn);
      float ps = 0.0f;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        s[e] = __builtin_amdgcn_exp2f(s[e] - mn);
        ps += s[e];
      }
      l = l * alpha + ps;
      m = mn;
#pragma unroll
      for (int db = 0; db < FF_D / 32; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[db][e] *= alpha;
      // ---- O^T += V^T P^T: step e sums over the keys that the half-waves hold in register e ----
      const float* vr = sV + (sub * 32 + 4 * lh) * FF_VROW + l32;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float* vk = vr + (8 * (e / 4) + (e % 4)) * FF_VROW;
#pragma unroll
        for (int db = 0; db < FF_D / 32; ++db)
          acc[db] = __builtin_amdgcn_mfma_f32_32x32x2f32(vk[FF_D2L ? (db ^ lh) * 32 : db * 32], s[e], acc[db], 0, 0, 0);
      }
    }
#if FF_D2L
    __builtin_amdgcn_s_waitcnt(0x0F70);               // vmcnt(0): this wavefront's blocks of the next tile have landed
    __syncthreads();                                  // everybody has finished with this tile, and the next is complete
    buf ^= 1;
#endif
  }
  // ---- O = acc / sum; lane: query qrow, head-dim positions db * 32 + 8 t + 4 (l / 32) + {0..3} ----
  l += __shfl_xor(l, 32, KCG_WAVE);
  if (!FF_RAGGED || qrow < FF_S) {
    float* op = o + (long)qrow * FF_D + 4 * lh;
#pragma unroll
    for (int db = 0; db < FF_D / 32; ++db)
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        kcg_f32x4 r = {acc[db][4 * t] / l, acc[db][4 * t + 1] / l, acc[db][4 * t + 2] / l, acc[db][4 * t + 3] / l};
        *(kcg_f32x4*)(op + db * 32 + 8 * t) = r;
      }
  }
  }   // pass: every wavefront has left the last tile behind the loop's last barrier, so the next pass may refill the buffers
}
#undef FF_NT
#undef FF_BR
#undef FF_KROW
#undef FF_VROW
#undef FF_NQ
#undef FF_SLOTS
#ifdef FF_PAIR_DEFAULTED
#undef FF_PAIR
#undef FF_PAIR_DEFAULTED
#endif
#undef FF_RAGGED
#ifdef FF_D2L_DEFAULTED
#undef FF_D2L
#undef FF_D2L_DEFAULTED
#endif
