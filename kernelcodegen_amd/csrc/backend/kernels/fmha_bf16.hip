// ---- fused attention forward, bf16 operands, fp32 softmax and accumulation ----
// O[b,h] = softmax(scale * Q[b,h] K[b,h]^T  (+ causal mask)) V[b,h]
// Q, K, V, O: [B, H, S, D] row-major.  Parameters:
//   FA_NAME, FA_B, FA_H, FA_S, FA_D      FA_D a multiple of 32
//   FA_BR     query rows per workgroup = 32 * FA_QW * number of wavefronts
//   FA_QW     32-query blocks per wavefront (1 or 2).  With 2, every K and V^T fragment read from LDS
//             feeds two MFMAs, a workgroup of 256 queries is four wavefronts with one per SIMD and 512
//             registers each, and the steady state runs in the step-pipelined form described below.
//   FA_BC     keys per LDS tile, a multiple of 32
//   FA_CAUSAL 1: keys j <= i only       FA_C  scale * log2(e) as an fp32 literal
//   FA_OUT_BF16
//   FA_OCC    workgroups per CU the register allocation has to leave room for
//
// Every wavefront owns 32 * FA_QW query rows and computes, per 32 of them, the TRANSPOSED score tile
//   S^T[key, query] = K . Q^T      (A operand = K rows from LDS, B operand = Q rows kept in registers)
// so that one lane holds ONE query column: its 16 accumulator registers per
// 32-key tile are 16 keys of that query, and the row maximum / row sum of the
// online softmax need only in-lane work plus one exchange between the two
// half-waves.  The probabilities stay in registers and become the B operand of
//   O^T[d, query] += V^T . P^T     (A operand = V^T from LDS)
// The accumulator layout (lane l, register v -> row 8*(v/4) + 4*(l/32) + v%4)
// fixes which 8 keys a half-wave contributes to one 16-deep MFMA step:
//   key(step s, half h, position p) = 16*s + 8*(p/4) + 4*h + p%4   (inside a 32-key tile)
// V tiles are copied into LDS as they are; the transposing LDS read (see "V in LDS" below) delivers exactly those
// keys of a column to a lane, so that the A operand of a step is two 8-byte reads.
//
// Pipeline.  On this part a wavefront's VALU work hides under MFMAs only when
// both are interleaved in its own instruction stream (about four VALU
// instructions per 32x32x16 MFMA); VALU work of one wavefront does not overlap
// with MFMAs of another on the same SIMD.  The softmax of tile t therefore runs
// between the MFMAs of the two products that do not depend on it: O += P(t-1)
// V(t-1) and S(t+1) = K(t+1) Q^T.  Iteration t:
//   global loads of K(t+2), V(t+1)
//   second half of tile t-1's exponentials, then max / rescale decision of tile t,
//                                         interleaved with  O^T += V(t-1)^T P(t-1)^T
//   first half of tile t's exp2, row sum, bf16 packing
//                                         interleaved with  S(t+1)^T = K(t+1) Q^T
//   LDS stores of K(t+2), V(t+1); one barrier
// K lives in two LDS buffers (tile t+1 read, t+2 written), V in three (t-1 read,
// t resident, t+1 written).
// With FA_QW 2 the iterations in which all three pieces are present run as a chain of short steps fenced
// against each other: a step issues the LDS reads of the NEXT step's two A fragments, runs four MFMAs
// from the two fragments read one step earlier, and carries an even share of the softmax's VALU work.
#ifndef KCG_INT_TAG
#define KCG_INT_TAG
template <int N> struct KcgInt { static constexpr int v = N; };
template <int I, int N, class F> __device__ __forceinline__ void kcg_static_for(F&& f) {
  if constexpr (I < N) {
    f(KcgInt<I>{});
    kcg_static_for<I + 1, N>(f);
  }
}
#endif
#ifndef FA_QW
#define FA_QW 1
#endif
#ifndef FA_PAIR
#define FA_PAIR 1
#endif
#ifndef FA_PERSIST
#define FA_PERSIST 0
#endif
#define FA_WAVES (FA_BR / (32 * FA_QW))
#define FA_NT (64 * FA_WAVES)
// FA_D2L 1 (head dim 128, 64-key tiles, eight wavefronts, no ragged edge): the K and V tiles go from global memory straight
// into LDS (global_load_lds_dwordx4; one instruction of a wavefront moves 1 KiB, four rows of 256 bytes, lane i to byte
// 16 i), so there are no staging registers and no LDS stores.  The rows are then not padded but swizzled, and the
// swizzle is applied on the source side (the lane that fills a position fetches the chunk that belongs there):
//   K: the 16-byte chunk c of key row r lies at position c ^ (r % 16): the sixteen lanes that a ds_read_b128 serves in
//      one pass (rows 0-3, 12-15 and 20-27 of a 32-row fragment, then the rest, all at one chunk) read sixteen positions;
//   V: the 64-byte granule g (32 values of d) of key row r lies at granule g ^ (r % 4): the four key rows that a
//      transposing read's 32 lanes take together fall on disjoint banks.
// A tile's loads are issued where the register form issued its global loads, at the start of the iteration that has
// the target buffer free, and are awaited in front of that iteration's barrier.
#ifndef FA_D2L
#define FA_D2L 0
#define FA_D2L_DEFAULTED
#endif
#define FA_SROWB (FA_D * 2 + 16)          // bytes per row of a wavefront's result tile when it is turned round in LDS
#define FA_KROWB (FA_D * 2 + (FA_D2L ? 0 : 16))          // bytes per K row in LDS
#ifndef FA_VPAD
#define FA_VPAD 32
#endif
#define FA_VROWB (FA_D * 2 + (FA_D2L ? 0 : FA_VPAD))     // bytes per key row of V in LDS (see "V in LDS" below)
#define FA_KTILES (FA_BC / 32)            // 32-key tiles per LDS tile
#define FA_DTILES (FA_D / 32)
#define FA_KSTEPS (FA_D / 16)             // MFMA steps of the score product
#define FA_KCHUNKS (FA_BC * (FA_D / 8))   // 16-byte chunks of a K tile
#define FA_KPER ((FA_KCHUNKS + FA_NT - 1) / FA_NT)
#define FA_VBUF (FA_BC * FA_VROWB)         // bytes of one V buffer
// V in LDS.  A V tile is copied as it is, [key][d] like K (16-byte chunks, plain stores).  The A operand of
// O^T += V^T P^T wants, in lane (d, key group h) of step s, the eight keys 16 s + 4 h + {0..3} and 16 s + 8 + 4 h + {0..3} of
// column d: that is what two ds_read_b64_tr_b16 deliver.  Of that instruction (probed on the device, its operation
// is in no header here): within each group of 16 lanes, lane r supplies the address of four consecutive 16-bit values,
// "row r" of a 16 x 4 matrix M, and lane i receives M[4 j + i / 4][i % 4], j = 0..3.  With lane r pointing at V[key0 + r / 4]
// [d0 + 4 (r % 4) ..], lane i receives V[key0 + 0..3][d0 + i]: four consecutive keys of its own column.  Rows are padded
// by 32 bytes: the four key rows a group reads then fall on four disjoint sets of eight banks.
#ifndef FA_FAST_CAUSAL
#define FA_FAST_CAUSAL 1
#endif
// FA_RAGGED: the sequence length is no multiple of the tiles.  The last query tile and the last key tile are then
// partly outside the tensors: their loads take row FA_S - 1 instead of a row past the end, scores of keys past the end
// are masked like keys behind the diagonal, and result rows past the end are not written.  Such a kernel runs every
// tile in the general form of the iteration (the number of key tiles may be odd, and the last one is masked).
#define FA_RAGGED ((FA_S % FA_BC) != 0 || (FA_S % FA_BR) != 0)
#define FA_FAST (!FA_RAGGED && FA_BC == 64 && FA_D % 64 == 0 && \
                 (FA_CAUSAL ? (FA_FAST_CAUSAL && FA_QW == 1 && FA_BR % (2 * FA_BC) == 0) : (FA_S / FA_BC) % 2 == 0))
// The epilogue turns each wavefront's 32-query result tile round in LDS (rows padded like the K tile's) when the result
// is bf16 and the tiles fit into the buffers nobody reads any more after the last iteration's barrier: both K buffers and
// the two V buffers that do not hold the last tile.
// A persistent workgroup has filled those buffers with the next job's tiles by then; it stages in LDS of its own,
// if the compute unit has that much.
#define FA_LDS_TILES (2 * FA_BC * FA_KROWB + 3 * FA_VBUF)
#define FA_STAGE_OWN (FA_PERSIST && FA_LDS_TILES + FA_WAVES * FA_STAGE_B <= 160 * 1024)
#define FA_STAGE_B (32 * FA_SROWB)
#define FA_STAGE_NK (2 * FA_BC * FA_KROWB / FA_STAGE_B)
#define FA_STAGE_NV (FA_VBUF / FA_STAGE_B)
#ifndef FA_STAGE_O
#define FA_STAGE_O (FA_OUT_BF16 && (FA_STAGE_OWN || FA_STAGE_NK + 2 * FA_STAGE_NV >= FA_WAVES))
#endif
#ifndef FA_AHEAD
#define FA_AHEAD 2                        // steps between a fragment read and the MFMAs that use it
#endif

// FA_F16 1: Q, K, V (and a 16-bit result) are IEEE half instead of bf16; everything else is the same kernel
#ifndef FA_F16
#define FA_F16 0
#define FA_F16_DEFAULTED
#endif
#if FA_F16
typedef _Float16 kcg_fa_f16x8 __attribute__((ext_vector_type(8)));
#define FA_FRAG kcg_fa_f16x8
#define FA_MFMA __builtin_amdgcn_mfma_f32_32x32x16_f16
#define FA_PACK2 kcg_pack_f16x2
#else
#define FA_FRAG kcg_bf16x8
#define FA_MFMA __builtin_amdgcn_mfma_f32_32x32x16_bf16
#define FA_PACK2 kcg_pack_bf16x2
#endif

#if (FA_D % 32) || (FA_BC % 32) || (FA_BR % (32 * FA_QW))
#error "fmha: D, BC must be multiples of 32, BR of 32 * QW"
#endif
#if FA_RAGGED && FA_PERSIST
#error "fmha: a persistent workgroup needs a sequence length that is a multiple of the tiles"
#endif
#if FA_D2L && (FA_RAGGED || FA_D != 128 || FA_BC != 64 || FA_NT != 512)
#error "fmha: direct loads into LDS need head dim 128, 64-key tiles, eight wavefronts and whole tiles"
#endif

extern "C" __global__ __launch_bounds__(FA_NT, FA_OCC)
void FA_NAME(const unsigned short* __restrict__ Q, const unsigned short* __restrict__ K,
             const unsigned short* __restrict__ V,
#if FA_OUT_BF16
             unsigned short* __restrict__ O
#else
             float* __restrict__ O
#endif
) {
  __shared__ __attribute__((aligned(1024))) char smem[FA_LDS_TILES + (FA_STAGE_O && FA_STAGE_OWN ? FA_WAVES * FA_STAGE_B : 0)];
  char* sK = smem;                                   // [2][FA_BC][FA_KROWB]
  char* sV = smem + 2 * FA_BC * FA_KROWB;            // [3][FA_BC][FA_VROWB]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int lh = lane >> 5;
  // V^T fragment reads (transposing): this lane's address inside a block of 16 keys x 32 d, see "V in LDS"
  // (FA_D2L: plus the lane's part of the granule swizzle, key row % 4 = (lane % 16) / 4, in address bits 6-7, where the
  // d tile of a read is then XORed in)
  const int vtr = (4 * lh + (lane & 15) / 4) * FA_VROWB + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2 + (FA_D2L ? ((lane & 15) / 4) * 64 : 0);
  typedef short kcg_s16x4 __attribute__((ext_vector_type(4)));
  // (addresses are formed in the LDS address space: a cast of every generic pointer would stand between the reads and
  // their immediate offsets)
  typedef __attribute__((address_space(3))) char* kcg_lds_ptr;
  const kcg_lds_ptr sV3 = (kcg_lds_ptr)sV + vtr;
  // The lane's address in V buffer `buf`, in a register of its own: the reads of a tile then differ from it by
  // immediates only (left to itself the compiler keeps one address per read and adjusts all of them every iteration).
  auto v_tile_base = [&](int buf) __attribute__((always_inline)) {
    kcg_lds_ptr p = sV3 + buf * FA_VBUF;
    asm volatile("" : "+v"(p));
    return p;
  };
  auto read_vt = [&](kcg_lds_ptr tile, int block) __attribute__((always_inline)) {     // block: offset of key 16 s of the step, d 32 i of the tile
#if FA_D2L
    // block = key group * 16 rows + d tile * 64 bytes: the rows are added, the d tile is XORed into the granule bits
    const kcg_lds_ptr p = (kcg_lds_ptr)(((unsigned)(size_t)(tile + (block / FA_VROWB) * FA_VROWB)) ^ (unsigned)(block % FA_VROWB));
#else
    const kcg_lds_ptr p = tile + block;
#endif
    const kcg_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) kcg_s16x4*)p);
    const kcg_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) kcg_s16x4*)(p + 8 * FA_VROWB));
    return __builtin_bit_cast(FA_FRAG, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  };

  // Workgroup id -> (query tile, batch*head).  Consecutive ids go round-robin to
  // the 8 XCDs: with the id's low 3 bits selecting the head, every query tile of
  // one head runs on one XCD and shares that head's K and V in its L2.
  constexpr int NQ = (FA_S + FA_BR - 1) / FA_BR;
  constexpr int BH = FA_B * FA_H;
  // Under a causal mask query tile i needs i+1 key-tile groups.  A workgroup takes a pair of query tiles whose key
  // tiles add up to NQ + 1, so that all workgroups do the same amount of work:
  //   FA_PAIR 1: (NQ-1-p, p) of the SAME head (needs an even NQ).  The NQ/2 workgroups of a head walk its keys together
  //              in their first job, but start their second jobs one after the other, each from key 0 again: by then the
  //              head's first keys have left the L2 (measured: 1.44 times the algorithmic bytes at S 2048, D 128).
  //   FA_PAIR 2: (NQ-1-j, j) of two DIFFERENT heads A and B (needs an even number of heads): NQ workgroups share the two
  //              heads.  They walk A's keys together from key 0 (tile NQ-1-j stops after NQ-j key tiles), and enter B
  //              one key tile apart, the one with the longest walk first, so that every key tile of B is read by the next
  //              workgroup one tile's time after the one before it: both heads' K and V come from HBM once.
  constexpr bool CROSS = FA_CAUSAL && FA_PAIR == 2 && BH % 2 == 0;
  constexpr bool PAIR = FA_CAUSAL && FA_PAIR == 1 && NQ % 2 == 0;
  constexpr int NSLOT = CROSS ? NQ : (PAIR ? NQ / 2 : NQ);
  // A workgroup works through the items blockIdx.x, blockIdx.x + gridDim.x, ... (FA_PERSIST: the grid is the number of
  // compute units; else one item each), an item being a query tile or a pair of them: its jobs.  While the last key tile
  // of a job is in the softmax, the first tiles of the next job are fetched: K(0), K(1), V(0) into the LDS buffers that
  // are free by then and the queries into the fragment registers, so that a job's prologue waits for no memory.
  constexpr int PASSES = (PAIR || CROSS) ? 2 : 1;
  constexpr int NGROUP = CROSS ? BH / 2 : BH;         // heads, or pairs of heads, that the items are dealt over
  constexpr int ITEMS = NSLOT * NGROUP;
  auto job_coords = [&](int job, int& qt, long& bh) __attribute__((always_inline)) {
    const int item = blockIdx.x + (job / PASSES) * gridDim.x, pass = job % PASSES;
    int slot, grp;
    if (NGROUP % 8 == 0) {
      const int r = item >> 3;
      slot = r % NSLOT;
      grp = (r / NSLOT) * 8 + (item & 7);
    } else {
      slot = item % NSLOT;
      grp = item / NSLOT;
    }
    // under a causal mask the query tile with the most keys goes first
    if (CROSS) {
      qt = pass == 0 ? NQ - 1 - slot : slot;
      bh = 2 * grp + pass;
    } else {
      qt = !FA_CAUSAL ? slot : (PAIR ? (pass == 0 ? NQ - 1 - slot : slot) : NQ - 1 - slot);
      bh = grp;
    }
  };
  const int njobs = ((ITEMS - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x) * PASSES;
  // number of tiles certainly even (under the mask also for a ragged length: see num_tiles)
  constexpr bool EVEN = FA_CAUSAL ? (FA_BR % (2 * FA_BC) == 0) : (FA_RAGGED || (FA_S / FA_BC) % 2 == 0);
  constexpr bool PREFETCH = FA_PERSIST && EVEN;
  // With PREFETCH the key tiles of a workgroup's jobs form one stream: tile T of a job with T tiles is tile 0 of the
  // next job.  The loads run on across the boundary; the last iteration of a job computes the first scores of the next
  // one (with that job's queries) beside its own softmax; and the first iteration of a job adds the last tile of the job
  // before it to that job's accumulators beside its own softmax, then writes that job's result and clears them.  Only
  // the first job of a workgroup has a prologue and only the last one a drain.
  bool carry = false;        // the job before this one has left its last tile's probabilities and its accumulators behind
  bool carry_active = false; // and this wavefront took part in that tile
  int prev_qt = 0;
  long prev_bh = 0;
  int voff = 0;              // key tile t of the job lives in V buffer (t + voff) % 3

  FA_FRAG fq[FA_QW][FA_KSTEPS];
  kcg_u32x4 rk[FA_KPER], rk1[FA_KPER];
  kcg_u32x4 rv[FA_KPER];

  for (int job = 0; job < njobs; ++job) {
  int qt;
  long bh;
  job_coords(job, qt, bh);
  const unsigned short* q_ = Q + bh * (long)FA_S * FA_D;
  const unsigned short* k_ = K + bh * (long)FA_S * FA_D;
  const unsigned short* v_ = V + bh * (long)FA_S * FA_D;
  const int q0 = qt * FA_BR + wave * (32 * FA_QW);   // first query of this wavefront
  const int myq = q0 + l32;                          // the query this lane's columns belong to, in block 0; +32 per block
  // the job after this one
  const bool has_next = PREFETCH && job + 1 < njobs;
  int nqt = 0;
  long nbh = 0;
  if (has_next) job_coords(job + 1, nqt, nbh);
  const unsigned short* nq_ = Q + nbh * (long)FA_S * FA_D;
  const unsigned short* nk_ = K + nbh * (long)FA_S * FA_D;
  const unsigned short* nv_ = V + nbh * (long)FA_S * FA_D;

  // Q fragments: B operand of S^T = K Q^T, lane = (query l32, d group lh).  The queries are
  // multiplied by scale * log2(e) once here, so the first product yields base-2 exponents directly.
  // The loads are issued here and the scaling happens in the prologue, once the first K and V tiles are on their way too.
  // (the lane's row and d group from a copy of the thread id the compiler cannot see through: see write_out)
  auto load_q = [&](const unsigned short* head, int qtile) __attribute__((always_inline)) {
    int tid_q = tid;
    asm volatile("" : "+v"(tid_q));
#if FA_RAGGED
    const int row0 = qtile * FA_BR + (tid_q >> 6) * (32 * FA_QW) + (tid_q & 31);
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw) {
      const int row = row0 + 32 * qw < FA_S ? row0 + 32 * qw : FA_S - 1;
#pragma unroll
      for (int ks = 0; ks < FA_KSTEPS; ++ks)
        fq[qw][ks] = *(const FA_FRAG*)((const char*)head + (unsigned)((row * FA_D + ((tid_q >> 5) & 1) * 8 + ks * 16) * 2));
    }
#else
    const unsigned short* lane_rows = head + (long)(qtile * FA_BR + (tid_q >> 6) * (32 * FA_QW) + (tid_q & 31)) * FA_D + ((tid_q >> 5) & 1) * 8;
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw)
#pragma unroll
      for (int ks = 0; ks < FA_KSTEPS; ++ks)
        fq[qw][ks] = *(const FA_FRAG*)(lane_rows + (long)(32 * qw) * FA_D + ks * 16);
#endif
  };
  if (!carry) load_q(q_, qt);
  auto scale_q = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw)
#pragma unroll
      for (int ks = 0; ks < FA_KSTEPS; ++ks) {
#if FA_F16
        typedef float kcg_fa_f32x8 __attribute__((ext_vector_type(8)));
        fq[qw][ks] = __builtin_convertvector(__builtin_convertvector(fq[qw][ks], kcg_fa_f32x8) * FA_C, FA_FRAG);
#else
        const kcg_u32x4 raw = __builtin_bit_cast(kcg_u32x4, fq[qw][ks]);
        kcg_u32x4 scaled;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          scaled[e] = FA_PACK2(__builtin_bit_cast(float, raw[e] << 16) * FA_C,
                               __builtin_bit_cast(float, raw[e] & 0xffff0000u) * FA_C);
        fq[qw][ks] = __builtin_bit_cast(FA_FRAG, scaled);
#endif
      }
  };

  kcg_f32x16 oacc[FA_QW][FA_DTILES];
  float m_run[FA_QW];        // reference point of the exponentials, a base-2 exponent; same in both half-waves
  float l_run[FA_QW];        // running sum of exp2(score - m_run) over this half-wave's keys
  auto clear_sums = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw) {
      l_run[qw] = 0.0f;
#pragma unroll
      for (int i = 0; i < FA_DTILES; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[qw][i][v] = 0.0f;
    }
  };

  constexpr int t_lo = 0;
  constexpr int ALL_TILES = (FA_S + FA_BC - 1) / FA_BC;
  // Past the end of a ragged sequence there is at most one more tile, which makes the count even (under the mask: where
  // the count up to the diagonal is).  The parity known at compile time is what keeps the two sets of score registers
  // apart without copies.  All keys of that tile are masked, or it concerns no wavefront; its loads repeat the last row.
  constexpr int ALL_EVEN = FA_RAGGED && (!FA_CAUSAL || FA_BR % (2 * FA_BC) == 0) ? ALL_TILES + ALL_TILES % 2 : ALL_TILES;
#if FA_CAUSAL
  const int to_diagonal = (qt * FA_BR + FA_BR + FA_BC - 1) / FA_BC;   // tiles that contain a key <= last query
  const int num_tiles = FA_RAGGED && to_diagonal > ALL_EVEN ? ALL_EVEN : to_diagonal;
#else
  const int num_tiles = ALL_EVEN;
#endif

  auto load_k_into = [&](const unsigned short* k_, int t, kcg_u32x4 (&rk)[FA_KPER]) __attribute__((always_inline)) {
    // address = a pointer every lane shares + a 32-bit offset of the lane's own that is the same for every tile: the
    // lane keeps one register for it, not a 64-bit address per load
    const char* tile = (const char*)k_ + (long)t * (FA_BC * FA_D * 2);
#pragma unroll
    for (int i = 0; i < FA_KPER; ++i) {
      const int c = i * FA_NT + tid;
      if (FA_KCHUNKS % FA_NT == 0 || c < FA_KCHUNKS) {
        if (FA_RAGGED) {
          const int row = c / (FA_D / 8), ch = c % (FA_D / 8);
          // (a head is below 4 GiB: the pointer all lanes share plus a 32-bit offset, as in the other forms)
          const int key = t * FA_BC + row < FA_S ? t * FA_BC + row : FA_S - 1;
          rk[i] = *(const kcg_u32x4*)((const char*)k_ + (unsigned)(key * (FA_D * 2) + ch * 16));
        } else if (FA_NT % (FA_D / 8) == 0) {
          const unsigned mine = (unsigned)((tid / (FA_D / 8)) * (FA_D * 2) + (tid % (FA_D / 8)) * 16);
          rk[i] = *(const kcg_u32x4*)(tile + (long)i * (FA_NT / (FA_D / 8)) * (FA_D * 2) + mine);
        } else {
          const int row = c / (FA_D / 8), ch = c % (FA_D / 8);
          rk[i] = *(const kcg_u32x4*)(tile + (unsigned)(row * (FA_D * 2) + ch * 16));
        }
      }
    }
  };
  auto load_v_from = [&](const unsigned short* v_, int t) __attribute__((always_inline)) { load_k_into(v_, t, rv); };
#if FA_D2L
  // Direct loads.  A tile is 16 blocks of four rows; block 2 wave + u (u = 0, 1) is this wavefront's.  Lane i fills row
  // i / 16 of its block, position i % 16.  K: it fetches chunk (i % 16) ^ (row % 16), row % 16 = 4 (block % 4) + i / 16;
  // V: chunk (((i % 16) / 4) ^ (i / 16)) * 4 + i % 4.  The instruction is written out (scalar base, 32-bit lane offset,
  // M0 = LDS address): through the builtin the compiler waits for every outstanding load in front of the transposing
  // reads, which it cannot tell apart from the landing tile.
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const unsigned smem_lds = (unsigned)(size_t)(__attribute__((address_space(3))) char*)smem;
  auto lds_dma = [&](const char* base, unsigned lane_off, unsigned dst) __attribute__((always_inline)) {
    const unsigned m = __builtin_amdgcn_readfirstlane(dst);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" :: "v"(lane_off), "s"(base), "s"(m) : "memory");
  };
  const unsigned dma_k_lane = (unsigned)((lane >> 4) * (FA_D * 2)) + (unsigned)((((lane & 15) ^ (lane >> 4)) ^ (8 * (wave & 1))) * 16);
  const unsigned dma_v_lane = (unsigned)((lane >> 4) * (FA_D * 2)) + (unsigned)(((((lane & 15) >> 2) ^ (lane >> 4)) * 4 + (lane & 3)) * 16);
  auto dma_k_tile = [&](const unsigned short* k_, int t) __attribute__((always_inline)) {      // tile t of a head into K buffer t % 2
    const char* tile = (const char*)k_ + (long)t * (FA_BC * FA_D * 2) + wave_u * (8 * FA_D * 2);
#pragma unroll
    for (int u = 0; u < 2; ++u)
      lds_dma(tile + u * (4 * FA_D * 2), dma_k_lane ^ (unsigned)(u * 64), smem_lds + (t & 1) * (FA_BC * FA_KROWB) + (wave_u * 2 + u) * (4 * FA_KROWB));
  };
  auto dma_v_tile = [&](const unsigned short* v_, int t, int buf) __attribute__((always_inline)) {
    const char* tile = (const char*)v_ + (long)t * (FA_BC * FA_D * 2) + wave_u * (8 * FA_D * 2);
#pragma unroll
    for (int u = 0; u < 2; ++u)
      lds_dma(tile + u * (4 * FA_D * 2), dma_v_lane, smem_lds + 2 * FA_BC * FA_KROWB + buf * FA_VBUF + (wave_u * 2 + u) * (4 * FA_VROWB));
  };
#endif
  // tile t of the stream: of this job, or past its end of the next one
  auto load_k = [&](int t) __attribute__((always_inline)) {
#if FA_D2L
    if (t < num_tiles) dma_k_tile(k_, t);
    else if (has_next) { const unsigned short* n_ = nk_; const int tt = t - num_tiles; const char* tile = (const char*)n_ + (long)tt * (FA_BC * FA_D * 2) + wave_u * (8 * FA_D * 2);
#pragma unroll
      for (int u = 0; u < 2; ++u)
        lds_dma(tile + u * (4 * FA_D * 2), dma_k_lane ^ (unsigned)(u * 64), smem_lds + (t & 1) * (FA_BC * FA_KROWB) + (wave_u * 2 + u) * (4 * FA_KROWB));
    }
#else
    if (t < num_tiles) load_k_into(k_, t, rk);
    else if (has_next) load_k_into(nk_, t - num_tiles, rk);
#endif
  };
  auto load_v = [&](int t) __attribute__((always_inline)) {
#if FA_D2L
    if (t < num_tiles) dma_v_tile(v_, t, (t + voff + 3) % 3);
    else if (has_next) dma_v_tile(nv_, t - num_tiles, (t + voff + 3) % 3);
#else
    if (t < num_tiles) load_v_from(v_, t);
    else if (has_next) load_v_from(nv_, t - num_tiles);
#endif
  };
  auto store_k_from = [&](int t, const kcg_u32x4 (&rk)[FA_KPER]) __attribute__((always_inline)) {   // tile t into K buffer t%2
    char* dk = sK + (t & 1) * (FA_BC * FA_KROWB);
#pragma unroll
    for (int i = 0; i < FA_KPER; ++i) {
      const int c = i * FA_NT + tid;
      if (FA_KCHUNKS % FA_NT == 0 || c < FA_KCHUNKS) {
        const int row = c / (FA_D / 8), ch = c % (FA_D / 8);
        *(kcg_u32x4*)(dk + row * FA_KROWB + ch * 16) = rk[i];
      }
    }
  };
#if FA_D2L
  auto store_k = [&](int) __attribute__((always_inline)) {};        // the tile was loaded straight into its buffer
#else
  auto store_k = [&](int t) __attribute__((always_inline)) { store_k_from(t, rk); };
#endif
  auto store_v_buf = [&](int buf) __attribute__((always_inline)) {     // the tile in rv into a V buffer, as it is
    char* dv = sV + buf * FA_VBUF;
#pragma unroll
    for (int i = 0; i < FA_KPER; ++i) {
      const int c = i * FA_NT + tid;
      if (FA_KCHUNKS % FA_NT == 0 || c < FA_KCHUNKS) {
        const int row = c / (FA_D / 8), ch = c % (FA_D / 8);
        *(kcg_u32x4*)(dv + row * FA_VROWB + ch * 16) = rv[i];
      }
    }
  };
#if FA_D2L
  auto store_v = [&](int) __attribute__((always_inline)) {};
  // in front of a barrier: this wavefront's shares of the tiles on their way have landed
  auto tiles_landed = [&]() __attribute__((always_inline)) { __builtin_amdgcn_s_waitcnt(0x0F70); };     // vmcnt(0)
#else
  auto store_v = [&](int t) __attribute__((always_inline)) { store_v_buf((t + voff + 3) % 3); };
  auto tiles_landed = [&]() __attribute__((always_inline)) {};
#endif

  constexpr int KH = (FA_KTILES + 1) / 2;     // sub-tiles whose exponentials run beside the next tile's score product
  kcg_f32x16 s0[FA_QW][FA_KTILES], s1[FA_QW][FA_KTILES];   // exponents of the tile in softmax and of the tile after it
  kcg_u32x4 pk[FA_QW][FA_KTILES][2];         // probabilities of one tile as bf16 pairs: B operands of the second product
  // Tile t concerns this wavefront unless every one of its keys lies after every query of the wavefront.
  // (`masked_c`: whether the run in progress contains tiles behind the diagonal at all.)
  auto active = [&](int t, auto masked_c) { return decltype(masked_c)::v == 0 || t * FA_BC <= q0 + 32 * FA_QW - 1; };

  // S^T = K(t) Q^T - m_run into `sc`: per query block FA_KTILES tiles of 32 keys x 32 queries.  Every register
  // of a lane belongs to the lane's query, so starting the accumulators at -m_run subtracts the reference
  // point for free.
  auto scores = [&](int t, kcg_f32x16 (&sc)[FA_QW][FA_KTILES]) {
    const char* cK = sK + (t & 1) * (FA_BC * FA_KROWB) + l32 * FA_KROWB + (FA_D2L ? (lh ^ (l32 & 15)) : lh) * 16;
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw)
#pragma unroll
      for (int kt = 0; kt < FA_KTILES; ++kt)
#pragma unroll
        for (int v = 0; v < 16; ++v) sc[qw][kt][v] = -m_run[qw];
#pragma unroll
    for (int ks = 0; ks < FA_KSTEPS; ++ks)
#pragma unroll
      for (int kt = 0; kt < FA_KTILES; ++kt) {
#if FA_D2L
        const FA_FRAG fk = *(const __attribute__((address_space(3))) FA_FRAG*)((kcg_lds_ptr)(((unsigned)(size_t)(kcg_lds_ptr)cK) ^ (unsigned)(ks * 32)) + kt * 32 * FA_KROWB);
#else
        const FA_FRAG fk = *(const FA_FRAG*)(cK + kt * 32 * FA_KROWB + ks * 32);
#endif
#pragma unroll
        for (int qw = 0; qw < FA_QW; ++qw)
          sc[qw][kt] = FA_MFMA(fk, fq[qw][ks], sc[qw][kt], 0, 0, 0);
      }
  };
  // O^T += V(t)^T P^T with the probabilities in pk
  auto weighted_sum = [&](int t) {
    const kcg_lds_ptr vb = v_tile_base((t + voff + 3) % 3);
#pragma unroll
    for (int kt = 0; kt < FA_KTILES; ++kt)
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int g = kt * 2 + s;       // this lane reads chunk 2 g + lh of row 32 i + l32
#pragma unroll
        for (int i = 0; i < FA_DTILES; ++i) {
          const FA_FRAG fv = read_vt(vb, g * 16 * FA_VROWB + i * 64);
#pragma unroll
          for (int qw = 0; qw < FA_QW; ++qw)
            oacc[qw][i] = FA_MFMA(fv, __builtin_bit_cast(FA_FRAG, pk[qw][kt][s]),
                                                                  oacc[qw][i], 0, 0, 0);
        }
      }
  };
  // First half of the online softmax of tile t (exponents relative to m_run in `sc`): mask, then per query
  // block the maximum over this half-wave's keys.
  auto row_max_local = [&](int t, kcg_f32x16 (&sc)[FA_QW][FA_KTILES], float (&m_half)[FA_QW], auto may_mask_c) {
#if FA_CAUSAL
    const int j0 = t * FA_BC;
    if (decltype(may_mask_c)::v != 0 && j0 + FA_BC - 1 > q0) {   // wave-uniform: only tiles that cross the diagonal need the mask
#pragma unroll
      for (int qw = 0; qw < FA_QW; ++qw)
#pragma unroll
        for (int kt = 0; kt < FA_KTILES; ++kt)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int key = j0 + kt * 32 + 8 * (v / 4) + 4 * lh + (v % 4);
            if (key > myq + 32 * qw) sc[qw][kt][v] = -__builtin_inff();
          }
    }
#endif
#if FA_RAGGED
    if (t * FA_BC + FA_BC > FA_S) {      // the last key tile: keys past the end of the sequence
#pragma unroll
      for (int qw = 0; qw < FA_QW; ++qw)
#pragma unroll
        for (int kt = 0; kt < FA_KTILES; ++kt)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int key = t * FA_BC + kt * 32 + 8 * (v / 4) + 4 * lh + (v % 4);
            if (key >= FA_S) sc[qw][kt][v] = -__builtin_inff();
          }
    }
#endif
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw) {
      float m_tile = -__builtin_inff();
#pragma unroll
      for (int kt = 0; kt < FA_KTILES; ++kt)
#pragma unroll
        for (int v = 0; v < 16; ++v) m_tile = fmaxf(m_tile, sc[qw][kt][v]);
      m_half[qw] = m_tile;
    }
  };
  // The maximum over all keys of the tile, which is how far the reference point would have to move up.
  auto row_max = [&](int t, kcg_f32x16 (&sc)[FA_QW][FA_KTILES], float (&m_rel)[FA_QW], auto masked_c) {
    row_max_local(t, sc, m_rel, masked_c);
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw) m_rel[qw] = fmaxf(m_rel[qw], __shfl_xor(m_rel[qw], 32, KCG_WAVE));
  };
  // The reference point m_run only has to keep exp2 in range, not to be the exact maximum.  The
  // first tile of a run sets it to the tile's maximum (that tile holds a key <= every query of every
  // wavefront it concerns, so that maximum is finite); afterwards it moves, and the accumulators are rescaled, only when some column's
  // maximum exceeds it by more than 8, i.e. a probability above 2^8, which is rare.  The exponents
  // already in `sc` were taken relative to the old reference point and are shifted along.
  auto rescale = [&](int t, float (&m_rel)[FA_QW], kcg_f32x16 (&sc)[FA_QW][FA_KTILES]) {
    bool grow = false;
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw) grow = grow || m_rel[qw] > 8.0f;
    if (t == t_lo || __builtin_amdgcn_ballot_w64(grow) != 0) {
#pragma unroll
      for (int qw = 0; qw < FA_QW; ++qw) {
        const float delta = t == t_lo ? m_rel[qw] : fmaxf(m_rel[qw], 0.0f);
        m_run[qw] += delta;
#pragma unroll
        for (int kt = 0; kt < FA_KTILES; ++kt)
#pragma unroll
          for (int v = 0; v < 16; ++v) sc[qw][kt][v] -= delta;
        if (t != t_lo) {      // nothing is accumulated before the first tile
          const float alpha = __builtin_amdgcn_exp2f(-delta);
          l_run[qw] *= alpha;
#pragma unroll
          for (int i = 0; i < FA_DTILES; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) oacc[qw][i][v] *= alpha;
        }
      }
      return true;
    }
    return false;
  };
  // Second half, for the 32-key sub-tiles [kt0, kt1): exponentials, row sum, packing to bf16 into pk.
  auto exponentials = [&](kcg_f32x16 (&sc)[FA_QW][FA_KTILES], auto kt0_c, auto kt1_c) {
    constexpr int kt0 = decltype(kt0_c)::v, kt1 = decltype(kt1_c)::v;
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw) {
      float l_tile = 0.0f;
#pragma unroll
      for (int kt = kt0; kt < kt1; ++kt)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const float p = __builtin_amdgcn_exp2f(sc[qw][kt][v]);
          sc[qw][kt][v] = p;
          l_tile += p;
        }
      l_run[qw] += l_tile;     // each half-wave sums its own keys; the halves are added after the last tile
#pragma unroll
      for (int kt = kt0; kt < kt1; ++kt)
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            pk[qw][kt][s][e] = FA_PACK2(sc[qw][kt][8 * s + 2 * e], sc[qw][kt][8 * s + 2 * e + 1]);
    }
  };
  // The probabilities of the first sub-tiles are not read before the next iteration.  Left alone, the compiler
  // sinks their whole computation past the barrier into the next iteration's first block, where no MFMA runs
  // beside it; an empty asm that takes the values as operands keeps it where it is written.
  auto pin_sum = [&]() {
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw) asm volatile("" : "+v"(l_run[qw]));
  };
  auto pin_first_half = [&]() {
    pin_sum();
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw)
#pragma unroll
      for (int kt = 0; kt < KH; ++kt)
#pragma unroll
        for (int s = 0; s < 2; ++s) asm volatile("" : "+v"(pk[qw][kt][s]));
  };
  // MFMAs of a product dealt out between the VALU instructions of the softmax half that shares its region
  auto interleave = [&](auto valu_per_mfma) {
    __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);     // fragment reads run three MFMAs ahead: LDS latency
#pragma unroll
    for (int m = 0; m < FA_KTILES * FA_KSTEPS; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, FA_QW, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, decltype(valu_per_mfma)::v * FA_QW, 0);
    }
  };

  // Prologue of a run: its first K and V tiles and its second K tile into LDS, then the first tile's scores.
  auto prologue = [&](auto masked_c) __attribute__((always_inline)) {
    // every load of the prologue is in flight before the first of them is waited for
    load_k(t_lo);
    load_v(t_lo);
#if FA_D2L
    if (num_tiles > t_lo + 1) dma_k_tile(k_, t_lo + 1);
#else
    if (num_tiles > t_lo + 1) load_k_into(k_, t_lo + 1, rk1);
#endif
    __builtin_amdgcn_sched_barrier(0);
    scale_q();
    store_k(t_lo);
    store_v(t_lo);
#if !FA_D2L
    if (num_tiles > t_lo + 1) store_k_from(t_lo + 1, rk1);
#endif
    tiles_landed();
    __syncthreads();
    if (active(t_lo, masked_c)) scores(t_lo, s0);
    __syncthreads();      // the first iteration overwrites the K buffer just read
  };

  // A lane's four consecutive d of one query are 8 bytes of a row of O, and the 64 lanes of a store hold 32
  // different rows: written like that, a wavefront's 32 x FA_D tile takes 2 FA_D stores of 64 pieces in 32 cache lines
  // each.  With `stage_c` every wavefront turns its tile round in a piece of LDS of its own and writes whole rows: a
  // store covers 1 KiB that is contiguous in O.  The other wavefronts may still be reading the last V tile, nothing else.
  auto write_out = [&](auto stage_c, int qt, long bh) __attribute__((always_inline)) {
    constexpr bool STAGE = decltype(stage_c)::v != 0;
    // The lane's addresses are worked out here, from a copy of the thread id the compiler cannot see through: computed
    // once before the loop over the jobs they would be spilled across it, and reloaded here one after the other.
    int tid_e = tid;
    asm volatile("" : "+v"(tid_e));
    const int lane = tid_e & 63, wave = tid_e >> 6, l32 = lane & 31, lh = lane >> 5;
    const int q0 = qt * FA_BR + wave * (32 * FA_QW), myq = q0 + l32;
    char* stage = smem;
    if constexpr (STAGE) {
      if (FA_STAGE_OWN) {
        stage = smem + FA_LDS_TILES + wave * FA_STAGE_B;
      } else if (wave < FA_STAGE_NK) {
        stage = sK + wave * FA_STAGE_B;
      } else {
        const int j = wave - FA_STAGE_NK;
        stage = sV + ((num_tiles + voff + j / FA_STAGE_NV) % 3) * FA_VBUF + (j % FA_STAGE_NV) * FA_STAGE_B;
      }
    }
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw) {
      const float l_all = l_run[qw] + __shfl_xor(l_run[qw], 32, KCG_WAVE);
      const float inv_l = 1.0f / l_all;
#if FA_OUT_BF16
      unsigned short* o_ = O + bh * (long)FA_S * FA_D + (long)(myq + 32 * qw) * FA_D;
#else
      float* o_ = O + bh * (long)FA_S * FA_D + (long)(myq + 32 * qw) * FA_D;
#endif
#pragma unroll
      for (int i = 0; i < FA_DTILES; ++i)
#pragma unroll
        for (int v = 0; v < 16; v += 4) {
          const int d = i * 32 + 8 * (v / 4) + 4 * lh;     // four consecutive d: registers v .. v+3
#if FA_OUT_BF16
          kcg_u32x2 w;
          w[0] = FA_PACK2(oacc[qw][i][v] * inv_l, oacc[qw][i][v + 1] * inv_l);
          w[1] = FA_PACK2(oacc[qw][i][v + 2] * inv_l, oacc[qw][i][v + 3] * inv_l);
          if constexpr (STAGE) *(kcg_u32x2*)(stage + l32 * FA_SROWB + d * 2) = w;
          else if (!FA_RAGGED || myq + 32 * qw < FA_S) *(kcg_u32x2*)(o_ + d) = w;
#else
          kcg_f32x4 w = {oacc[qw][i][v] * inv_l, oacc[qw][i][v + 1] * inv_l, oacc[qw][i][v + 2] * inv_l,
                         oacc[qw][i][v + 3] * inv_l};
          if (!FA_RAGGED || myq + 32 * qw < FA_S) *(kcg_f32x4*)(o_ + d) = w;
#endif
        }
      if constexpr (STAGE) {
        // the wavefront reads back what its own lanes wrote: LDS accesses of one wavefront complete in order
        constexpr int CPR = FA_D / 8;                        // 16-byte chunks per row
        char* orow = (char*)(O + bh * (long)FA_S * FA_D + (long)(q0 + 32 * qw) * FA_D);
#pragma unroll
        for (int k = 0; k < 32 * CPR / 64; ++k) {
          const int c = k * 64 + lane, row = c / CPR, ch = c % CPR;
          if (!FA_RAGGED || q0 + 32 * qw + row < FA_S)
            *(kcg_u32x4*)(orow + (long)row * (FA_D * 2) + ch * 16) = *(const kcg_u32x4*)(stage + row * FA_SROWB + ch * 16);
        }
      }
    }
  };

  // The exponentials of a tile are split to even out the VALU work between the two products:
  // sub-tiles [0, KH) next to the score product of the following tile, sub-tiles [KH, FA_KTILES)
  // one iteration later next to the tile's own weighted sum (whose first steps only need the
  // first sub-tiles' probabilities).
  // `first_c`, `last_c`: tile t is known to be the job's first / last.  With `carry`, the first iteration's weighted sum
  // is the last tile of the job before (its probabilities are where a tile t-1 of this job would have left them), and
  // that job's result is written and the accumulators cleared before this job's first probabilities are summed.  The
  // last iteration of a job that has a successor takes that job's queries and computes its first scores.
  auto iteration = [&](int t, kcg_f32x16 (&cur)[FA_QW][FA_KTILES], kcg_f32x16 (&nxt)[FA_QW][FA_KTILES], auto masked_c,
                       auto first_c, auto last_c) __attribute__((always_inline)) {
    constexpr bool FIRST = decltype(first_c)::v != 0, LAST = decltype(last_c)::v != 0;
    load_k(t + 2);
    load_v(t + 1);
    if constexpr (LAST) {
      if (has_next) load_q(nq_, nqt);      // the fragments of this job's queries have been used for the last time
    }
    __builtin_amdgcn_sched_barrier(0);      // keep the global loads a whole tile ahead of the LDS stores that need them
    float m_rel[FA_QW];
    const bool pv = FIRST ? carry_active : (t > t_lo && active(t - 1, masked_c)), sm = active(t, masked_c);
    if (pv) {
      exponentials(nxt, KcgInt<KH>{}, KcgInt<FA_KTILES>{});     // rest of tile t-1, whose scores are still in `nxt`
      weighted_sum(t - 1);
    }
    if (sm) row_max(t, cur, m_rel, masked_c);
    interleave(KcgInt<5>{});
    __builtin_amdgcn_sched_barrier(0);
    if (sm) rescale(t, m_rel, cur);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (FIRST) {
      if (carry) {
        write_out(KcgInt<FA_STAGE_O && FA_STAGE_OWN>{}, prev_qt, prev_bh);
        clear_sums();
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if constexpr (LAST) {
      if (has_next) {
        // from here on m_run and the score registers in `nxt` belong to the next job; its first tile concerns every wavefront
        scale_q();
#pragma unroll
        for (int qw = 0; qw < FA_QW; ++qw) m_run[qw] = 0.0f;
        scores(t + 1, nxt);
      }
    } else {
      if (t + 1 < num_tiles && active(t + 1, masked_c)) {
        // the registers of `nxt` are free from here on: scores(t+1) initialises and fills them
        scores(t + 1, nxt);
      }
    }
    if (sm) {
      exponentials(cur, KcgInt<0>{}, KcgInt<KH>{});
      pin_first_half();
    }
    interleave(KcgInt<5>{});
    __builtin_amdgcn_sched_barrier(0);
    if (t + 2 < num_tiles || has_next) store_k(t + 2);
    if (t + 1 < num_tiles || has_next) store_v(t + 1);
    tiles_landed();
    __syncthreads();
  };
#if FA_FAST
  // Steady-state form of the iteration (both products and the softmax all present) as a chain of
  // steps fenced against each other.  A step issues the LDS reads of the NEXT step's two A operands into the
  // fragment pair not in use, runs this step's MFMAs from the pair read one step ago (each fragment serves
  // both query blocks), and carries a share of the softmax's VALU work, so LDS latency and VALU issue both
  // sit under MFMA time.
  FA_FRAG fr[FA_AHEAD + 1][2];             // fragment pairs: the one in use and those on their way
  constexpr int HG = FA_DTILES / 2;           // steps per key group of the second product: two d tiles each
  kcg_lds_ptr fast_v_tile = sV3;      // set at the start of every steady-state iteration: the V tile of its weighted sum
  auto read_v = [&](int t, auto a_c, FA_FRAG (&f)[2]) {      // V^T fragments of step a: key group a/HG, d tiles 2(a%HG)..+1
    constexpr int g = decltype(a_c)::v / HG, i0 = 2 * (decltype(a_c)::v % HG);
#pragma unroll
    for (int i = 0; i < 2; ++i) f[i] = read_vt(fast_v_tile, g * 16 * FA_VROWB + (i0 + i) * 64);
  };
  auto mfma_v = [&](auto a_c, FA_FRAG (&f)[2]) {
    constexpr int g = decltype(a_c)::v / HG, i0 = 2 * (decltype(a_c)::v % HG);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int qw = 0; qw < FA_QW; ++qw)
        oacc[qw][i0 + i] = FA_MFMA(
            f[i], __builtin_bit_cast(FA_FRAG, pk[qw][g / 2][g % 2]), oacc[qw][i0 + i], 0, 0, 0);
  };
  auto read_k = [&](int t, auto j_c, FA_FRAG (&f)[2]) {      // K fragments of k-step j, both 32-key sub-tiles
    const char* cK = sK + (t & 1) * (FA_BC * FA_KROWB) + l32 * FA_KROWB + (FA_D2L ? (lh ^ (l32 & 15)) : lh) * 16;
#if FA_D2L
    const kcg_lds_ptr cJ = (kcg_lds_ptr)(((unsigned)(size_t)(kcg_lds_ptr)cK) ^ (unsigned)(decltype(j_c)::v * 32));
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) f[kt] = *(const __attribute__((address_space(3))) FA_FRAG*)(cJ + kt * 32 * FA_KROWB);
#else
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) f[kt] = *(const FA_FRAG*)(cK + kt * 32 * FA_KROWB + decltype(j_c)::v * 32);
#endif
  };
  auto mfma_k = [&](auto j_c, FA_FRAG (&f)[2], kcg_f32x16 (&sc)[FA_QW][FA_KTILES]) {
    constexpr int j = decltype(j_c)::v;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int qw = 0; qw < FA_QW; ++qw)
        sc[qw][kt] = FA_MFMA(f[kt], fq[qw][j], sc[qw][kt], 0, 0, 0);
  };
  // the score registers of sub-tile kt start at -m_run
  auto init_scores = [&](kcg_f32x16 (&sc)[FA_QW][FA_KTILES], int kt) {
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw) {
      const float negm = -m_run[qw];
#pragma unroll
      for (int v = 0; v < 16; ++v) sc[qw][kt][v] = negm;
      asm volatile("" : "+v"(sc[qw][kt]));     // here, not sunk to the first MFMA
    }
  };
  // Exponentials number [i0, i1) of sub-tile kt, counted value-major over the query blocks (number = value *
  // FA_QW + block); a bf16 pair is packed as soon as its second value exists.
  auto exp_range = [&](kcg_f32x16 (&sc)[FA_QW][FA_KTILES], auto kt_c, auto i0_c, auto i1_c) {
    constexpr int kt = decltype(kt_c)::v;
#pragma unroll
    for (int n = decltype(i0_c)::v; n < decltype(i1_c)::v; ++n) {
      const int v = n / FA_QW, qw = n % FA_QW;
      const float p = __builtin_amdgcn_exp2f(sc[qw][kt][v]);
      sc[qw][kt][v] = p;
      l_run[qw] += p;
      if (v & 1) pk[qw][kt][v / 8][(v % 8) / 2] = FA_PACK2(sc[qw][kt][v - 1], p);
    }
  };
  auto mix = [&](auto valu_c) {     // order inside a step: the two reads first, VALU dealt between the MFMAs
    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
#pragma unroll
    for (int m = 0; m < 2 * FA_QW; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, decltype(valu_c)::v, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  constexpr int NE = 16 * FA_QW;      // exponentials per sub-tile and wavefront
  constexpr int NA = 4 * HG;          // steps of the second product
  constexpr int NAX = 3 * HG;         // of which these carry the exponentials of sub-tile 1 of tile t-1: key group 2 starts at
                                      // step 2 HG and needs the first half of them, key group 3 at step 3 HG needs all
  constexpr int NB = FA_KSTEPS;       // steps of the score product
  constexpr int NBX = NB - 1;         // of which the last carries the LDS stores, the others exponentials of tile t
  // the fragment reads of step n of iteration t: steps [0, NA) belong to the second product, [NA, NA + NB) to the first
  auto read_step = [&](int t, auto n_c) {
    constexpr int n = decltype(n_c)::v;
    if constexpr (n < NA) read_v(t - 1, KcgInt<n>{}, fr[n % (FA_AHEAD + 1)]);
    else if constexpr (n < NA + NB) read_k(t + 1, KcgInt<n - NA>{}, fr[n % (FA_AHEAD + 1)]);
  };
  auto fast_iteration = [&](int t, kcg_f32x16 (&cur)[FA_QW][FA_KTILES], kcg_f32x16 (&nxt)[FA_QW][FA_KTILES]) __attribute__((always_inline)) {
    load_k(t + 2);
    load_v(t + 1);
    __builtin_amdgcn_sched_barrier(0);
    // lead-in: first V fragments on their way while the row maxima of tile t are taken
    fast_v_tile = v_tile_base((t - 1 + voff + 3) % 3);
    kcg_static_for<0, FA_AHEAD>([&](auto n_c) { read_step(t, n_c); });
    float m_rel[FA_QW], m_other[FA_QW];
    row_max_local(t, cur, m_rel, KcgInt<0>{});
#pragma unroll
    for (int qw = 0; qw < FA_QW; ++qw) m_other[qw] = __shfl_xor(m_rel[qw], 32, KCG_WAVE);
    __builtin_amdgcn_sched_barrier(0);
    // O^T += V(t-1)^T P(t-1)^T
    kcg_static_for<0, NA>([&](auto a_c) {
      constexpr int a = decltype(a_c)::v;
      read_step(t, KcgInt<a + FA_AHEAD>{});
      mfma_v(a_c, fr[a % (FA_AHEAD + 1)]);
      if constexpr (a < NAX) {
        exp_range(nxt, KcgInt<1>{}, KcgInt<(NE * a + NAX - 1) / NAX>{}, KcgInt<(NE * (a + 1) + NAX - 1) / NAX>{});
      } else {
        // the registers of `nxt` are free now; the rare move of the reference point below initialises them again
        if constexpr (a == NAX && NA - NAX >= 2) init_scores(nxt, 0);
        if constexpr (a == NA - 1) {
          if constexpr (NA - NAX < 2) init_scores(nxt, 0);
          init_scores(nxt, 1);
#pragma unroll
          for (int qw = 0; qw < FA_QW; ++qw) m_rel[qw] = fmaxf(m_rel[qw], m_other[qw]);
        }
      }
      mix(KcgInt<4>{});
    });
    if (rescale(t, m_rel, cur)) {
      init_scores(nxt, 0);
      init_scores(nxt, 1);
    }
    __builtin_amdgcn_sched_barrier(0);
    // S(t+1)^T = K(t+1) Q^T - m_run, one k-step per step; exponentials of sub-tile 0 of tile t ride along
    kcg_static_for<0, NB>([&](auto j_c) {
      constexpr int j = decltype(j_c)::v;
      read_step(t, KcgInt<NA + j + FA_AHEAD>{});
      mfma_k(j_c, fr[(NA + j) % (FA_AHEAD + 1)], nxt);
      if constexpr (j < NBX) {
        exp_range(cur, KcgInt<0>{}, KcgInt<(NE * j + NBX - 1) / NBX>{}, KcgInt<(NE * (j + 1) + NBX - 1) / NBX>{});
        if constexpr (j == NBX - 1) pin_first_half();
        else pin_sum();
        mix(KcgInt<4>{});
      } else {
        if (t + 2 < num_tiles || has_next) store_k(t + 2);
        store_v(t + 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    });
    tiles_landed();
    __syncthreads();
  };
#endif
  // One run over the key tiles [t_lo, num_tiles), from empty softmax state to the unnormalised result in oacc.
  // The steady state runs in a loop of its own: with both forms of the iteration inside one loop the register
  // allocator no longer fits the kernel into its budget.  s0 holds the scores of the tiles at even distance from t_lo.
  auto run = [&](auto masked_c, auto fast_c, auto even_c) __attribute__((always_inline)) {
    if (!carry) {
      clear_sums();
#pragma unroll
      for (int qw = 0; qw < FA_QW; ++qw) m_run[qw] = 0.0f;
      prologue(masked_c);
    }
    if constexpr (decltype(even_c)::v != 0) {
      // An even number of tiles (at least two), so which of s0 and s1 holds what is fixed at every point of the code;
      // with that left to the run time, the copies between the two sets cost more registers than there are.
      // The first tile has no weighted sum of this job before it and the last no scores of this job after it; all
      // tiles between them run in the steady-state form where there is one (no tile of such a job is masked or skipped).
      iteration(t_lo, s0, s1, masked_c, KcgInt<1>{}, KcgInt<0>{});
#if FA_FAST && FA_CAUSAL
      if constexpr (decltype(fast_c)::v != 0) {
        // The tiles that cross the diagonal are the job's last FA_BR / FA_BC (an even number); the u tiles before them
        // (u even as well) concern every wavefront in full.  Of those, tile 0 has run, tiles 1 .. u-2 run in the
        // steady-state form, tile u-1 in the general form (the tile after it is masked).
        constexpr int DG = FA_BR / FA_BC;
        const int u = num_tiles - DG;
        if (u > 0) {
          for (int t = 1; t + 2 < u; t += 2) {
            fast_iteration(t, s1, s0);
            fast_iteration(t + 1, s0, s1);
          }
          iteration(u - 1, s1, s0, masked_c, KcgInt<0>{}, KcgInt<0>{});
          iteration(u, s0, s1, masked_c, KcgInt<0>{}, KcgInt<0>{});
        }
        kcg_static_for<1, DG - 1>([&](auto i_c) {
          constexpr int i = decltype(i_c)::v;
          if constexpr (i % 2) iteration(u + i, s1, s0, masked_c, KcgInt<0>{}, KcgInt<0>{});
          else iteration(u + i, s0, s1, masked_c, KcgInt<0>{}, KcgInt<0>{});
        });
      } else
#endif
      for (int t = t_lo + 1; t + 1 < num_tiles; t += 2) {
#if FA_FAST
        if constexpr (decltype(fast_c)::v != 0) {
          fast_iteration(t, s1, s0);
          fast_iteration(t + 1, s0, s1);
        } else
#endif
        {
          iteration(t, s1, s0, masked_c, KcgInt<0>{}, KcgInt<0>{});
          iteration(t + 1, s0, s1, masked_c, KcgInt<0>{}, KcgInt<0>{});
        }
      }
      iteration(num_tiles - 1, s1, s0, masked_c, KcgInt<0>{}, KcgInt<1>{});
      if (!has_next && active(num_tiles - 1, masked_c)) {
        exponentials(s1, KcgInt<KH>{}, KcgInt<FA_KTILES>{});
        weighted_sum(num_tiles - 1);
      }
    } else {
      int t = t_lo;
      for (; t + 1 < num_tiles; t += 2) {
        iteration(t, s0, s1, masked_c, KcgInt<0>{}, KcgInt<0>{});
        iteration(t + 1, s1, s0, masked_c, KcgInt<0>{}, KcgInt<0>{});
      }
      if (t < num_tiles) iteration(t, s0, s1, masked_c, KcgInt<0>{}, KcgInt<0>{});
      if (active(num_tiles - 1, masked_c)) {
        if ((num_tiles - 1 - t_lo) & 1) exponentials(s1, KcgInt<KH>{}, KcgInt<FA_KTILES>{});
        else exponentials(s0, KcgInt<KH>{}, KcgInt<FA_KTILES>{});
        weighted_sum(num_tiles - 1);
      }
    }
  };

  // ---- O[q, d] = O^T[d, q] / l : lane = query column, registers = d rows ----
  run(KcgInt<FA_CAUSAL>{}, KcgInt<FA_FAST>{}, KcgInt<EVEN>{});
  if (has_next) {
    // the next job's first iteration finishes this one
    carry = true;
    carry_active = active(num_tiles - 1, KcgInt<FA_CAUSAL>{});
    prev_qt = qt;
    prev_bh = bh;
    voff = (voff + num_tiles) % 3;
  } else {
    write_out(KcgInt<FA_STAGE_O>{}, qt, bh);
    carry = false;
    __syncthreads();      // the next job's prologue refills the LDS buffers
  }
  }
}
#undef FA_FRAG
#undef FA_MFMA
#undef FA_PACK2
#ifdef FA_F16_DEFAULTED
#undef FA_F16
#undef FA_F16_DEFAULTED
#endif
#undef FA_WAVES
#undef FA_NT
#undef FA_KROWB
#undef FA_SROWB
#ifdef FA_D2L_DEFAULTED
#undef FA_D2L
#undef FA_D2L_DEFAULTED
#endif
#undef FA_VROWB
#undef FA_VPAD
#undef FA_KTILES
#undef FA_DTILES
#undef FA_KSTEPS
#undef FA_KCHUNKS
#undef FA_KPER
#undef FA_VBUF
#undef FA_FAST
#undef FA_RAGGED
#undef FA_FAST_CAUSAL
#undef FA_PAIR
#undef FA_STAGE_O
#undef FA_STAGE_B
#undef FA_STAGE_OWN
#undef FA_LDS_TILES
#undef FA_PERSIST
#undef FA_STAGE_NK
#undef FA_STAGE_NV
#undef FA_AHEAD
#undef FA_QW
