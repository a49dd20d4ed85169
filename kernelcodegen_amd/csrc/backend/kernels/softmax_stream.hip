// ---- softmax over the last axis for rows too long to keep in registers ----
// y[r, :] = exp(x[r, :] - max) / sum exp(x[r, :] - max).  One workgroup of SS_BLOCK threads per row, two passes over
// the row: the first keeps, per thread, a running maximum and the sum of exp(x - that maximum), rescaled whenever the
// maximum moves, and merges the threads' pairs (wavefront shuffles, then LDS); the second reads the row again (for rows
// of a few MiB from the L2 / last-level cache) and writes the quotients.  In place each element is read and then
// written by the same thread in the second pass.
// Parameters: SS_NAME, SS_ROWS, SS_N, SS_BLOCK, SS_VW (4 or 1), SS_INPLACE, SS_F16 (1: IEEE half, 2: bfloat16 in memory; fp32 arithmetic).
#ifndef SS_F16
#define SS_F16 0
#define SS_F16_DEFAULTED
#endif
#if SS_F16 == 2
#define SS_IO __bf16
#elif SS_F16
#define SS_IO _Float16
#else
#define SS_IO float
#endif
extern "C" __global__ __launch_bounds__(SS_BLOCK)
#if SS_INPLACE
void SS_NAME(SS_IO* __restrict__ Y) {
  const SS_IO* X = Y;
#else
void SS_NAME(const SS_IO* __restrict__ X, SS_IO* __restrict__ Y) {
#endif
  typedef SS_IO io_vec_t __attribute__((ext_vector_type(SS_VW)));
  __shared__ float red_m[SS_BLOCK / KCG_WAVE], red_s[SS_BLOCK / KCG_WAVE];
  const int tid = threadIdx.x;
  const SS_IO* x = X + (long)blockIdx.x * SS_N;
  SS_IO* y = Y + (long)blockIdx.x * SS_N;
  constexpr float LOG2E = 1.4426950408889634f;

  // (m, s): maximum so far and sum of exp(x - m) over what has been seen; m = -inf, s = 0 before the first element
  float m = -__builtin_inff(), s = 0.0f;
  for (long i = (long)tid * SS_VW; i < SS_N; i += (long)SS_BLOCK * SS_VW) {
    const io_vec_t in = *(const io_vec_t*)(x + i);
    float mv = (float)in[0];
#pragma unroll
    for (int j = 1; j < SS_VW; ++j) mv = fmaxf(mv, (float)in[j]);
    if (mv > m) {                         // the reference point moves: rescale what has been summed
      s *= __builtin_amdgcn_exp2f((m - mv) * LOG2E);      // exp(-inf) = 0 the first time
      m = mv;
    }
    // while every element seen so far is -inf there is no reference point yet and nothing to add (each such element
    // counts as exp(-inf) = 0, as in exp(x) / sum exp(x); -inf - -inf would put a NaN into the sum)
    if (m > -__builtin_inff() || m != m) {
#pragma unroll
      for (int j = 0; j < SS_VW; ++j) s += __builtin_amdgcn_exp2f(((float)in[j] - m) * LOG2E);
    }
  }
  // merge of two pairs: the larger maximum wins, the other sum is rescaled to it (a thread that saw nothing, or only
  // -inf, has m = -inf, s = 0 and contributes nothing; two such threads give exp2(nan) * 0, avoided by the test on s,
  // which lets a sum that is NaN, from a NaN in the row, through: the whole row is then NaN, as in the plain quotient)
  auto merge = [&](float m2, float s2) {
    const float mm = fmaxf(m, m2);
    const float a = s == 0.0f ? 0.0f : s * __builtin_amdgcn_exp2f((m - mm) * LOG2E);
    const float b = s2 == 0.0f ? 0.0f : s2 * __builtin_amdgcn_exp2f((m2 - mm) * LOG2E);
    m = mm;
    s = a + b;
  };
#pragma unroll
  for (int off = KCG_WAVE / 2; off > 0; off >>= 1) merge(__shfl_xor(m, off, KCG_WAVE), __shfl_xor(s, off, KCG_WAVE));
  if ((tid % KCG_WAVE) == 0) { red_m[tid / KCG_WAVE] = m; red_s[tid / KCG_WAVE] = s; }
  __syncthreads();
  m = red_m[0]; s = red_s[0];
#pragma unroll
  for (int w = 1; w < SS_BLOCK / KCG_WAVE; ++w) merge(red_m[w], red_s[w]);
  const float rs = 1.0f / s;

  for (long i = (long)tid * SS_VW; i < SS_N; i += (long)SS_BLOCK * SS_VW) {
    const io_vec_t in = *(const io_vec_t*)(x + i);
    io_vec_t o;
#pragma unroll
    for (int j = 0; j < SS_VW; ++j) o[j] = (SS_IO)(__builtin_amdgcn_exp2f(((float)in[j] - m) * LOG2E) * rs);
    __builtin_nontemporal_store(o, (io_vec_t*)(y + i));
  }
}
#undef SS_IO
#ifdef SS_F16_DEFAULTED
#undef SS_F16
#undef SS_F16_DEFAULTED
#endif
