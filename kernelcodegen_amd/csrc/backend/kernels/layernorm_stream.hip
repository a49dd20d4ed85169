// ---- LayerNorm for groups too long to keep in registers ---------------------
// One workgroup of LS_BLOCK threads per group; three passes over the group
// (sum, centred sum of squares, normalise), each a coalesced stride loop.  The
// second and third pass re-read x, which for groups up to a few MiB is served by
// the L2 / Infinity Cache.
// Parameters: LS_NAME, LS_ROWS, LS_N, LS_NG, LS_NB, LS_EPS, LS_BLOCK, LS_VW (4 or 1), LS_GELU,
// LS_F16 (1: IEEE half, 2: bfloat16 in memory; the arithmetic is fp32 either way).
#ifndef LS_F16
#define LS_F16 0
#define LS_F16_DEFAULTED
#endif
#if LS_F16 == 2
#define LS_IO __bf16
#elif LS_F16
#define LS_IO _Float16
#else
#define LS_IO float
#endif
extern "C" __global__ __launch_bounds__(LS_BLOCK)
void LS_NAME(const LS_IO* __restrict__ X, const LS_IO* __restrict__ G,
             const LS_IO* __restrict__ Bt, LS_IO* __restrict__ Y) {
  typedef float vec_t __attribute__((ext_vector_type(LS_VW)));
  typedef LS_IO io_vec_t __attribute__((ext_vector_type(LS_VW)));
  auto widen = [](io_vec_t in) {
    vec_t r;
#pragma unroll
    for (int j = 0; j < LS_VW; ++j) r[j] = (float)in[j];
    return r;
  };
  __shared__ float red[LS_BLOCK / KCG_WAVE];
  const int tid = threadIdx.x;
  const LS_IO* __restrict__ x = X + (long)blockIdx.x * LS_N;
  LS_IO* __restrict__ y = Y + (long)blockIdx.x * LS_N;

  auto block_sum = [&](float v) -> float {
    v = kcg_wave_sum(v);
    __syncthreads();                       // protects `red` from the previous use
    if ((tid % KCG_WAVE) == 0) red[tid / KCG_WAVE] = v;
    __syncthreads();
    float t = 0.0f;
#pragma unroll
    for (int w = 0; w < LS_BLOCK / KCG_WAVE; ++w) t += red[w];
    return t;
  };

  float s = 0.0f;
  for (long i = (long)tid * LS_VW; i < LS_N; i += (long)LS_BLOCK * LS_VW) {
    const vec_t v = widen(*(const io_vec_t*)(x + i));
#pragma unroll
    for (int j = 0; j < LS_VW; ++j) s += v[j];
  }
  const float mean = block_sum(s) / (float)LS_N;

  float q = 0.0f;
  for (long i = (long)tid * LS_VW; i < LS_N; i += (long)LS_BLOCK * LS_VW) {
    const vec_t v = widen(*(const io_vec_t*)(x + i));
#pragma unroll
    for (int j = 0; j < LS_VW; ++j) { const float d = v[j] - mean; q += d * d; }
  }
  const float den = sqrtf(block_sum(q) / (float)LS_N + LS_EPS);

  for (long i = (long)tid * LS_VW; i < LS_N; i += (long)LS_BLOCK * LS_VW) {
    const vec_t v = widen(*(const io_vec_t*)(x + i));
    const vec_t g = widen(*(const io_vec_t*)(G + (i % LS_NG)));
    const vec_t b = widen(*(const io_vec_t*)(Bt + (i % LS_NB)));
    io_vec_t o;
#pragma unroll
    for (int j = 0; j < LS_VW; ++j) {
      float t = g[j] * ((v[j] - mean) / den) + b[j];
#if LS_GELU
      t = kcg_gelu(t);
#endif
      o[j] = (LS_IO)t;
    }
    *(io_vec_t*)(y + i) = o;
  }
}
#undef LS_IO
#ifdef LS_F16_DEFAULTED
#undef LS_F16
#undef LS_F16_DEFAULTED
#endif
