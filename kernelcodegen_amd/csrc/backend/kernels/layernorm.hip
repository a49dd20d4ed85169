// ---- LayerNorm (+ optional fused GELU), fp32, one pass over HBM -------------
// Parameters (defined by the emitter in front of this text):
//   LN_NAME      kernel symbol
//   LN_ROWS      number of normalised groups (product of dims before axis)
//   LN_N         elements per group          LN_NG / LN_NB  gamma / beta length
//   LN_EPS       epsilon as an fp32 literal
//   LN_TPR       threads that share one row (power of two, 64..1024)
//   LN_RPB       rows per block; block size = LN_TPR * LN_RPB
//   LN_VW        vector width of the global accesses (4 or 1)
//   LN_VPT       vectors held per thread = ceil(LN_N / (LN_TPR * LN_VW))
//   LN_GELU      1: apply GELU to the normalised value before the store
//
// The whole row lives in registers between the load and the store, so X is
// read once and Y written once: 2 * N * 4 bytes per row.  The arithmetic keeps
// the reference nest's formulation (centre first, biased variance of the
// centred values, divide by sqrt(var + eps)); only the summation order differs.
extern "C" __global__ __launch_bounds__(LN_TPR * LN_RPB)
void LN_NAME(const float* __restrict__ X, const float* __restrict__ G,
             const float* __restrict__ Bt, float* __restrict__ Y) {
  typedef float vec_t __attribute__((ext_vector_type(LN_VW)));
  const int tid = threadIdx.x;
  const int tr = tid % LN_TPR;               // position inside the row team
  const int rb = tid / LN_TPR;               // row inside the block
  const long row = (long)blockIdx.x * LN_RPB + rb;
  const bool live = row < LN_ROWS;
  const float* __restrict__ x = X + (live ? row : 0) * (long)LN_N;
  float* __restrict__ y = Y + (live ? row : 0) * (long)LN_N;

  vec_t v[LN_VPT];
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < LN_VPT; ++i) {
    const int idx = (i * LN_TPR + tr) * LN_VW;
    if (live && idx < LN_N) {
      v[i] = __builtin_nontemporal_load((const vec_t*)(x + idx));
    } else {
#pragma unroll
      for (int j = 0; j < LN_VW; ++j) v[i][j] = 0.0f;
    }
#pragma unroll
    for (int j = 0; j < LN_VW; ++j) s += v[i][j];
  }

#if LN_TPR > KCG_WAVE
  __shared__ float red[2][LN_RPB][LN_TPR / KCG_WAVE];
  const int wv = tr / KCG_WAVE;
#endif

  s = kcg_wave_sum(s);
#if LN_TPR > KCG_WAVE
  if ((tr % KCG_WAVE) == 0) red[0][rb][wv] = s;
  __syncthreads();
  s = 0.0f;
#pragma unroll
  for (int w = 0; w < LN_TPR / KCG_WAVE; ++w) s += red[0][rb][w];
#endif
  const float mean = s / (float)LN_N;

  float q = 0.0f;
#pragma unroll
  for (int i = 0; i < LN_VPT; ++i) {
    const int idx = (i * LN_TPR + tr) * LN_VW;
#pragma unroll
    for (int j = 0; j < LN_VW; ++j) {
      const float d = (idx + j < LN_N) ? v[i][j] - mean : 0.0f;
      v[i][j] = d;
      q += d * d;
    }
  }
  q = kcg_wave_sum(q);
#if LN_TPR > KCG_WAVE
  if ((tr % KCG_WAVE) == 0) red[1][rb][wv] = q;
  __syncthreads();
  q = 0.0f;
#pragma unroll
  for (int w = 0; w < LN_TPR / KCG_WAVE; ++w) q += red[1][rb][w];
#endif
  const float den = sqrtf(q / (float)LN_N + LN_EPS);

#pragma unroll
  for (int i = 0; i < LN_VPT; ++i) {
    const int idx = (i * LN_TPR + tr) * LN_VW;
    if (live && idx < LN_N) {
      const vec_t g = *(const vec_t*)(G + (idx % LN_NG));
      const vec_t b = *(const vec_t*)(Bt + (idx % LN_NB));
      vec_t o;
#pragma unroll
      for (int j = 0; j < LN_VW; ++j) {
        float t = g[j] * (v[i][j] / den) + b[j];
#if LN_GELU
        t = kcg_gelu(t);
#endif
        o[j] = t;
      }
      __builtin_nontemporal_store(o, (vec_t*)(y + idx));
    }
  }
}
