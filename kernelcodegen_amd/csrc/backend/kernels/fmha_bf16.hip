// ---- fused attention forward, bf16 operands, fp32 softmax and accumulation ----
// O[b,h] = softmax(scale * Q[b,h] K[b,h]^T  (+ causal mask)) V[b,h]
// Q, K, V, O: [B, H, S, D] row-major.  Parameters:
//   FA_NAME, FA_B, FA_H, FA_S, FA_D      FA_D a multiple of 32
//   FA_BR     query rows per workgroup = 32 * number of wavefronts
//   FA_BC     keys per LDS tile, a multiple of 32
//   FA_CAUSAL 1: keys j <= i only       FA_C  scale * log2(e) as an fp32 literal
//   FA_OUT_BF16
//   FA_OCC    workgroups per CU the register allocation has to leave room for
//
// Every wavefront owns 32 query rows and computes the TRANSPOSED score tile
//   S^T[key, query] = K . Q^T      (A operand = K rows from LDS, B operand = Q rows kept in registers)
// so that one lane holds ONE query column: its 16 accumulator registers per
// 32-key tile are 16 keys of that query, and the row maximum / row sum of the
// online softmax need only in-lane work plus one exchange between the two
// half-waves.  The probabilities stay in registers and become the B operand of
//   O^T[d, query] += V^T . P^T     (A operand = V^T from LDS)
// The accumulator layout (lane l, register v -> row 8*(v/4) + 4*(l/32) + v%4)
// fixes which 8 keys a half-wave contributes to one 16-deep MFMA step:
//   key(step s, half h, position p) = 16*s + 8*(p/4) + 4*h + p%4   (inside a 32-key tile)
// V is therefore stored in LDS transposed and key-permuted, sVt[d][chunk][p]
// with chunk = (tile*2 + s)*2 + h, so that the A operand of that step is one
// 16-byte read.  The transposition happens in registers on the way in (8 keys x
// 8 d per lane, byte permutes), like the column-major operand of the GEMM.
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
#ifndef KCG_INT_TAG
#define KCG_INT_TAG
template <int N> struct KcgInt { static constexpr int v = N; };
#endif
#define FA_WAVES (FA_BR / 32)
#define FA_NT (64 * FA_WAVES)
#define FA_KROWB (FA_D * 2 + 16)          // bytes per K row in LDS
#define FA_VROWB (FA_BC * 2 + 16)         // bytes per d row of V^T in LDS
#define FA_KTILES (FA_BC / 32)            // 32-key tiles per LDS tile
#define FA_DTILES (FA_D / 32)
#define FA_KSTEPS (FA_D / 16)             // MFMA steps of the score product
#define FA_KCHUNKS (FA_BC * (FA_D / 8))   // 16-byte chunks of a K tile
#define FA_KPER ((FA_KCHUNKS + FA_NT - 1) / FA_NT)
#define FA_VBLOCKS ((FA_BC / 8) * (FA_D / 8))   // 8(key) x 8(d) blocks of a V tile
// a lane transposes FA_VKR key rows of one block: 8 when there is at least one block per lane, else 4 or 2
#define FA_VKR (FA_VBLOCKS >= FA_NT ? 8 : (FA_VBLOCKS * 2 >= FA_NT ? 4 : 2))
#define FA_VUNITS (FA_VBLOCKS * (8 / FA_VKR))
#define FA_VPER ((FA_VUNITS + FA_NT - 1) / FA_NT)

#if (FA_D % 32) || (FA_BC % 32) || (FA_BR % 32) || (FA_S % FA_BC) || (FA_S % FA_BR)
#error "fmha: D, BC, BR must be multiples of 32 and S a multiple of BC and BR"
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
  __shared__ __attribute__((aligned(16))) char smem[2 * FA_BC * FA_KROWB + 3 * FA_D * FA_VROWB];
  char* sK = smem;                                   // [2][FA_BC][FA_KROWB]
  char* sV = smem + 2 * FA_BC * FA_KROWB;            // [3][FA_D][FA_VROWB]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int lh = lane >> 5;

  // Workgroup id -> (query tile, batch*head).  Consecutive ids go round-robin to
  // the 8 XCDs: with the id's low 3 bits selecting the head, every query tile of
  // one head runs on one XCD and shares that head's K and V in its L2.
  constexpr int NQ = FA_S / FA_BR;
  constexpr int BH = FA_B * FA_H;
  // Under a causal mask query tile i needs i+1 key-tile groups: a workgroup takes the pair
  // (NQ-1-p, p), so that all workgroups do the same amount of work.
  constexpr bool PAIR = FA_CAUSAL && NQ % 2 == 0;
  constexpr int NSLOT = PAIR ? NQ / 2 : NQ;
  int slot, bhi;
  if (BH % 8 == 0) {
    const int r = blockIdx.x >> 3;
    slot = r % NSLOT;
    bhi = (r / NSLOT) * 8 + (blockIdx.x & 7);
  } else {
    slot = blockIdx.x % NSLOT;
    bhi = blockIdx.x / NSLOT;
  }
  const long bh = bhi;
  const unsigned short* q_ = Q + bh * (long)FA_S * FA_D;
  const unsigned short* k_ = K + bh * (long)FA_S * FA_D;
  const unsigned short* v_ = V + bh * (long)FA_S * FA_D;
  for (int pass = 0; pass < (PAIR ? 2 : 1); ++pass) {
  // query tile of this pass; under a causal mask the ones with the most keys go first
  const int qt = !FA_CAUSAL ? slot : (PAIR ? (pass == 0 ? NQ - 1 - slot : slot) : NQ - 1 - slot);
  const int q0 = qt * FA_BR + wave * 32;             // first query of this wavefront
  const int myq = q0 + l32;                          // the query this lane's columns belong to

  // Q fragments: B operand of S^T = K Q^T, lane = (query l32, d group lh)
  kcg_bf16x8 fq[FA_KSTEPS];
#pragma unroll
  for (int ks = 0; ks < FA_KSTEPS; ++ks)
    fq[ks] = *(const kcg_bf16x8*)(q_ + (long)myq * FA_D + ks * 16 + lh * 8);

  kcg_f32x16 oacc[FA_DTILES];
#pragma unroll
  for (int i = 0; i < FA_DTILES; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) oacc[i][v] = 0.0f;
  float m_run = -__builtin_inff();   // reference point of the exponentials, a raw score; same in both half-waves
  float l_run = 0.0f;        // running sum of exp2(score - m_run) over this half-wave's keys

#if FA_CAUSAL
  const int num_tiles = (qt * FA_BR + FA_BR + FA_BC - 1) / FA_BC;   // tiles that contain a key <= last query
#else
  const int num_tiles = FA_S / FA_BC;
#endif

  kcg_u32x4 rk[FA_KPER];
  kcg_u32x4 rv[FA_VPER][FA_VKR];

  auto load_k = [&](int t) {
    const int j0 = t * FA_BC;
#pragma unroll
    for (int i = 0; i < FA_KPER; ++i) {
      const int c = i * FA_NT + tid;
      if (FA_KCHUNKS % FA_NT == 0 || c < FA_KCHUNKS) {
        const int row = c / (FA_D / 8), ch = c % (FA_D / 8);
        rk[i] = *(const kcg_u32x4*)(k_ + (long)(j0 + row) * FA_D + ch * 8);
      }
    }
  };
  auto load_v = [&](int t) {
    const int j0 = t * FA_BC;
#pragma unroll
    for (int i = 0; i < FA_VPER; ++i) {
      const int u = i * FA_NT + tid;
      if (FA_VUNITS % FA_NT == 0 || u < FA_VUNITS) {
        const int part = u % (8 / FA_VKR), blk = u / (8 / FA_VKR);
        const int db = blk % (FA_D / 8), chunk = blk / (FA_D / 8);     // chunk = (tile*2 + s)*2 + h
        const int h = chunk & 1, s = (chunk >> 1) & 1, tile = chunk >> 2;
#pragma unroll
        for (int pp = 0; pp < FA_VKR; ++pp) {
          const int p = part * FA_VKR + pp;                           // position inside the 16-byte chunk
          const int key = tile * 32 + 16 * s + 8 * (p / 4) + 4 * h + (p % 4);
          rv[i][pp] = *(const kcg_u32x4*)(v_ + (long)(j0 + key) * FA_D + db * 8);
        }
      }
    }
  };
  auto store_k = [&](int t) {          // tile t into K buffer t%2
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
  auto store_v = [&](int t) {          // tile t into V buffer t%3, transposed and key-permuted
    char* dv = sV + (t % 3) * (FA_D * FA_VROWB);
#pragma unroll
    for (int i = 0; i < FA_VPER; ++i) {
      const int u = i * FA_NT + tid;
      if (FA_VUNITS % FA_NT == 0 || u < FA_VUNITS) {
        const int part = u % (8 / FA_VKR), blk = u / (8 / FA_VKR);
        const int db = blk % (FA_D / 8), chunk = blk / (FA_D / 8);
#pragma unroll
        for (int c = 0; c < 8; ++c) {       // d = db*8 + c: halves c%2 of dword c/2 of each of the key rows
          unsigned o[FA_VKR / 2];
#pragma unroll
          for (int e = 0; e < FA_VKR / 2; ++e) {
            const unsigned lo = rv[i][2 * e][c / 2], hi = rv[i][2 * e + 1][c / 2];
            o[e] = (c & 1) ? __builtin_amdgcn_perm(hi, lo, 0x07060302u) : __builtin_amdgcn_perm(hi, lo, 0x05040100u);
          }
          char* d = dv + (db * 8 + c) * FA_VROWB + chunk * 16 + part * (2 * FA_VKR);
          if (FA_VKR == 8) {
            kcg_u32x4 w = {o[0], o[FA_VKR / 2 > 1 ? 1 : 0], o[FA_VKR / 2 > 2 ? 2 : 0], o[FA_VKR / 2 > 3 ? 3 : 0]};
            *(kcg_u32x4*)d = w;
          } else if (FA_VKR == 4) {
            kcg_u32x2 w = {o[0], o[FA_VKR / 2 > 1 ? 1 : 0]};
            *(kcg_u32x2*)d = w;
          } else {
            *(unsigned*)d = o[0];
          }
        }
      }
    }
  };

  kcg_f32x16 s0[FA_KTILES], s1[FA_KTILES];   // raw scores of the tile in softmax and of the tile after it
  kcg_u32x4 pk[FA_KTILES][2];                // probabilities of one tile as bf16 pairs: B operands of the second product
  // Tile t concerns this wavefront unless every one of its keys lies after every query of the wavefront.
  auto active = [&](int t) { return !FA_CAUSAL || t * FA_BC <= q0 + 31; };

  // S^T = K(t) Q^T into `sc`: FA_KTILES tiles of 32 keys x 32 queries
  auto scores = [&](int t, kcg_f32x16 (&sc)[FA_KTILES]) {
    const char* cK = sK + (t & 1) * (FA_BC * FA_KROWB) + l32 * FA_KROWB + lh * 16;
#pragma unroll
    for (int kt = 0; kt < FA_KTILES; ++kt)
#pragma unroll
      for (int v = 0; v < 16; ++v) sc[kt][v] = 0.0f;
#pragma unroll
    for (int ks = 0; ks < FA_KSTEPS; ++ks)
#pragma unroll
      for (int kt = 0; kt < FA_KTILES; ++kt) {
        const kcg_bf16x8 fk = *(const kcg_bf16x8*)(cK + kt * 32 * FA_KROWB + ks * 32);
        sc[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fk, fq[ks], sc[kt], 0, 0, 0);
      }
  };
  // O^T += V(t)^T P^T with the probabilities in pk
  auto weighted_sum = [&](int t) {
    const char* cV = sV + (t % 3) * (FA_D * FA_VROWB) + l32 * FA_VROWB + lh * 16;
#pragma unroll
    for (int kt = 0; kt < FA_KTILES; ++kt)
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const kcg_bf16x8 fp = __builtin_bit_cast(kcg_bf16x8, pk[kt][s]);
        const int chunk_pair = (kt * 2 + s) * 2;    // this lane reads chunk_pair + lh (lh is folded into cV)
#pragma unroll
        for (int i = 0; i < FA_DTILES; ++i) {
          const kcg_bf16x8 fv = *(const kcg_bf16x8*)(cV + i * 32 * FA_VROWB + chunk_pair * 16);
          oacc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fv, fp, oacc[i], 0, 0, 0);
        }
      }
  };
  // First half of the online softmax of tile t (scores in `sc`): mask, row maximum.  Returns the
  // candidate reference point.
  auto row_max = [&](int t, kcg_f32x16 (&sc)[FA_KTILES]) {
#if FA_CAUSAL
    const int j0 = t * FA_BC;
    if (j0 + FA_BC - 1 > q0) {   // wave-uniform: only tiles that cross the diagonal need the mask
#pragma unroll
      for (int kt = 0; kt < FA_KTILES; ++kt)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int key = j0 + kt * 32 + 8 * (v / 4) + 4 * lh + (v % 4);
          if (key > myq) sc[kt][v] = -__builtin_inff();
        }
    }
#endif
    float m_tile = -__builtin_inff();   // maximum of the raw scores (the scale is positive)
#pragma unroll
    for (int kt = 0; kt < FA_KTILES; ++kt)
#pragma unroll
      for (int v = 0; v < 16; ++v) m_tile = fmaxf(m_tile, sc[kt][v]);
    m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, KCG_WAVE));
    return fmaxf(m_run, m_tile);
  };
  // The reference point m_run only has to keep exp2 in range, not to be the exact maximum: it
  // moves (and the accumulators are rescaled) only when some column's maximum has grown by more
  // than 2^8, which after the first tiles is rare.  m_run starts at -inf, so the first tile always
  // moves it; the first tile holds key 0 <= every query, so m_run is finite from then on.
  auto rescale = [&](float m_new) {
    if (__builtin_amdgcn_ballot_w64((m_new - m_run) * FA_C > 8.0f) != 0) {
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * FA_C);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int i = 0; i < FA_DTILES; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[i][v] *= alpha;
    }
  };
  // Second half, for the 32-key sub-tiles [kt0, kt1): exponentials, row sum, packing to bf16 into pk.
  auto exponentials = [&](kcg_f32x16 (&sc)[FA_KTILES], auto kt0_c, auto kt1_c) {
    constexpr int kt0 = decltype(kt0_c)::v, kt1 = decltype(kt1_c)::v;
    const float mc = m_run * FA_C;
    float l_tile = 0.0f;
#pragma unroll
    for (int kt = kt0; kt < kt1; ++kt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[kt][v], FA_C, -mc));
        sc[kt][v] = p;
        l_tile += p;
      }
    l_run += l_tile;     // each half-wave sums its own keys; the halves are added after the last tile
#pragma unroll
    for (int kt = kt0; kt < kt1; ++kt)
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int e = 0; e < 4; ++e) pk[kt][s][e] = kcg_pack_bf16x2(sc[kt][8 * s + 2 * e], sc[kt][8 * s + 2 * e + 1]);
  };
  // MFMAs of a product dealt out between the VALU instructions of the softmax half that shares its region
  auto interleave = [&](auto valu_per_mfma) {
    __builtin_amdgcn_sched_group_barrier(0x100, 3, 0);     // fragment reads run three MFMAs ahead: LDS latency
#pragma unroll
    for (int m = 0; m < FA_KTILES * FA_KSTEPS; ++m) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, decltype(valu_per_mfma)::v, 0);
    }
  };

  // Prologue: K(0), V(0), K(1) into LDS, then S(0).
  load_k(0);
  load_v(0);
  store_k(0);
  store_v(0);
  if (num_tiles > 1) {
    load_k(1);
    store_k(1);
  }
  __syncthreads();
  if (active(0)) scores(0, s0);
  __syncthreads();      // iteration 0 overwrites K buffer 0

  // The exponentials of a tile are split to even out the VALU work between the two products:
  // sub-tiles [0, KH) next to the score product of the following tile, sub-tiles [KH, FA_KTILES)
  // one iteration later next to the tile's own weighted sum (whose first steps only need the
  // first sub-tiles' probabilities).
  constexpr int KH = (FA_KTILES + 1) / 2;
  auto iteration = [&](int t, kcg_f32x16 (&cur)[FA_KTILES], kcg_f32x16 (&nxt)[FA_KTILES]) {
    if (t + 2 < num_tiles) load_k(t + 2);
    if (t + 1 < num_tiles) load_v(t + 1);
    __builtin_amdgcn_sched_barrier(0);      // keep the global loads a whole tile ahead of the LDS stores that need them
    float m_new = m_run;
    const bool pv = t > 0 && active(t - 1), sm = active(t);
    if (pv) {
      exponentials(nxt, KcgInt<KH>{}, KcgInt<FA_KTILES>{});     // rest of tile t-1, whose scores are still in `nxt`
      weighted_sum(t - 1);
    }
    if (sm) m_new = row_max(t, cur);
    interleave(KcgInt<5>{});
    __builtin_amdgcn_sched_barrier(0);
    if (sm) rescale(m_new);
    __builtin_amdgcn_sched_barrier(0);
    if (t + 1 < num_tiles && active(t + 1)) {
      // the registers of `nxt` are free from here on: scores(t+1) zeroes and fills them
      scores(t + 1, nxt);
    }
    if (sm) exponentials(cur, KcgInt<0>{}, KcgInt<KH>{});
    interleave(KcgInt<5>{});
    __builtin_amdgcn_sched_barrier(0);
    if (t + 2 < num_tiles) store_k(t + 2);
    if (t + 1 < num_tiles) store_v(t + 1);
    __syncthreads();
  };
  int t = 0;
  for (; t + 1 < num_tiles; t += 2) {
    iteration(t, s0, s1);
    iteration(t + 1, s1, s0);
  }
  if (t < num_tiles) iteration(t, s0, s1);
  if (active(num_tiles - 1)) {
    if ((num_tiles - 1) & 1) exponentials(s1, KcgInt<KH>{}, KcgInt<FA_KTILES>{});
    else exponentials(s0, KcgInt<KH>{}, KcgInt<FA_KTILES>{});
    weighted_sum(num_tiles - 1);
  }

  // ---- O[q, d] = O^T[d, q] / l : lane = query column, registers = d rows ----
  l_run += __shfl_xor(l_run, 32, KCG_WAVE);
  const float inv_l = 1.0f / l_run;
#if FA_OUT_BF16
  unsigned short* o_ = O + bh * (long)FA_S * FA_D + (long)myq * FA_D;
#else
  float* o_ = O + bh * (long)FA_S * FA_D + (long)myq * FA_D;
#endif
#pragma unroll
  for (int i = 0; i < FA_DTILES; ++i)
#pragma unroll
    for (int v = 0; v < 16; v += 4) {
      const int d = i * 32 + 8 * (v / 4) + 4 * lh;     // four consecutive d: registers v .. v+3
#if FA_OUT_BF16
      kcg_u32x2 w;
      w[0] = kcg_pack_bf16x2(oacc[i][v] * inv_l, oacc[i][v + 1] * inv_l);
      w[1] = kcg_pack_bf16x2(oacc[i][v + 2] * inv_l, oacc[i][v + 3] * inv_l);
      *(kcg_u32x2*)(o_ + d) = w;
#else
      kcg_f32x4 w = {oacc[i][v] * inv_l, oacc[i][v + 1] * inv_l, oacc[i][v + 2] * inv_l, oacc[i][v + 3] * inv_l};
      *(kcg_f32x4*)(o_ + d) = w;
#endif
    }
  __syncthreads();      // the next pass refills the LDS buffers
  }
}
#undef FA_WAVES
#undef FA_NT
#undef FA_KROWB
#undef FA_VROWB
#undef FA_KTILES
#undef FA_DTILES
#undef FA_KSTEPS
#undef FA_KCHUNKS
#undef FA_KPER
#undef FA_VBLOCKS
#undef FA_VKR
#undef FA_VUNITS
#undef FA_VPER
