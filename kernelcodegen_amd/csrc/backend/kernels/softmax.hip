// ---- softmax over the last axis, fp32, one pass over HBM ----
// y[r, :] = exp(x[r, :]) / sum_k exp(x[r, k]), computed as exp(x - max) / sum exp(x - max): the same
// quotient, finite for every finite input.  The row lives in registers between the load and the store,
// so X is read once and Y written once.  Parameters:
//   SM_NAME      kernel symbol
//   SM_ROWS      number of rows (product of the leading dimensions)      SM_N   row length
//   SM_TPR       threads that share one row (power of two, 64..1024)
//   SM_RPB       rows per workgroup; block size = SM_TPR * SM_RPB
//   SM_VW        vector width of the global accesses (4 or 1)
//   SM_VPT       vectors held per thread = ceil(SM_N / (SM_TPR * SM_VW))
//   SM_INPLACE   1: the kernel takes one pointer and overwrites the input
//   SM_STREAM    1: the input is read with the non-temporal hint (it is read once); 0: plain loads
//   SM_F16       1: X and Y are IEEE half in memory, 2: bfloat16 (the arithmetic stays fp32); 0: fp32
#ifndef SM_F16
#define SM_F16 0
#define SM_F16_DEFAULTED
#endif
#if SM_F16 == 2
#define SM_IO __bf16
#elif SM_F16
#define SM_IO _Float16
#else
#define SM_IO float
#endif
extern "C" __global__ __launch_bounds__(SM_TPR * SM_RPB)
#if SM_INPLACE
void SM_NAME(SM_IO* __restrict__ Y) {
  const SM_IO* X = Y;
#else
void SM_NAME(const SM_IO* __restrict__ X, SM_IO* __restrict__ Y) {
#endif
  typedef float vec_t __attribute__((ext_vector_type(SM_VW)));
  typedef SM_IO io_vec_t __attribute__((ext_vector_type(SM_VW)));
  const int tid = threadIdx.x;
  const int tr = tid % SM_TPR;               // position inside the row team
  const int rb = tid / SM_TPR;               // row inside the workgroup
  const long row = (long)blockIdx.x * SM_RPB + rb;
  const bool live = row < SM_ROWS;
#if SM_TPR > KCG_WAVE
  __shared__ float red[2][SM_RPB][SM_TPR / KCG_WAVE];
  const int wv = tr / KCG_WAVE;
#endif
  const SM_IO* x = X + (live ? row : 0) * (long)SM_N;
  vec_t v[SM_VPT];
#pragma unroll
  for (int i = 0; i < SM_VPT; ++i) {
    const int idx = (i * SM_TPR + tr) * SM_VW;
    if (live && idx < SM_N) {
      const io_vec_t in = kcg_stream_load<SM_STREAM != 0>((const io_vec_t*)(x + idx));
#pragma unroll
      for (int j = 0; j < SM_VW; ++j) v[i][j] = (float)in[j];
    } else {
#pragma unroll
      for (int j = 0; j < SM_VW; ++j) v[i][j] = -__builtin_inff();     // exp gives 0: no effect on maximum or sum
    }
  }
  float m = -__builtin_inff();
#pragma unroll
  for (int i = 0; i < SM_VPT; ++i)
#pragma unroll
    for (int j = 0; j < SM_VW; ++j) m = fmaxf(m, v[i][j]);
  m = kcg_wave_max(m);
#if SM_TPR > KCG_WAVE
  if ((tr % KCG_WAVE) == 0) red[0][rb][wv] = m;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < SM_TPR / KCG_WAVE; ++w) m = fmaxf(m, red[0][rb][w]);
#endif
  if (!live) m = 0.0f;      // a row past the end holds only -inf: keep its arithmetic finite
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < SM_VPT; ++i)
#pragma unroll
    for (int j = 0; j < SM_VW; ++j) {
      const float e = __builtin_amdgcn_exp2f((v[i][j] - m) * 1.4426950408889634f);
      v[i][j] = e;
      s += e;
    }
  s = kcg_wave_sum(s);
#if SM_TPR > KCG_WAVE
  if ((tr % KCG_WAVE) == 0) red[1][rb][wv] = s;
  __syncthreads();
  s = 0.0f;
#pragma unroll
  for (int w = 0; w < SM_TPR / KCG_WAVE; ++w) s += red[1][rb][w];
#endif
  const float rs = 1.0f / s;
  SM_IO* y = Y + (live ? row : 0) * (long)SM_N;
#pragma unroll
  for (int i = 0; i < SM_VPT; ++i) {
    const int idx = (i * SM_TPR + tr) * SM_VW;
    if (live && idx < SM_N) {
      io_vec_t o;
#pragma unroll
      for (int j = 0; j < SM_VW; ++j) o[j] = (SM_IO)(v[i][j] * rs);
      __builtin_nontemporal_store(o, (io_vec_t*)(y + idx));
    }
  }
}
#undef SM_IO
#ifdef SM_F16_DEFAULTED
#undef SM_F16
#undef SM_F16_DEFAULTED
#endif
