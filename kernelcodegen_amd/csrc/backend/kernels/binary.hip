// ---- Binary operation with broadcasting, fp32, one pass over HBM ------------
// Z[i..] = X[i..] op Y[i..] where either operand may have extent 1 (or be
// missing) along any dimension of the result.  Parameters:
//   BN_NAME    kernel symbol          BN_RANK   rank of the result (1..6)
//   BN_DIMS    result extents, comma separated, outermost first
//   BN_SA / BN_SB   element strides of X / Y per result dimension (0 = broadcast)
//   BN_OP      0 Add, 1 Sub, 2 Mul, 3 Div, 4 Pow, 5 Equal, 6 Greater (ordered comparisons; the result is one
//              byte per element, 0 or 1: the device form of the IR's i1)
//   BN_VW      elements per lane along the innermost dimension (4 or 1)
//   BN_BLOCK   threads per block      BN_INPLACE 1: Z is X (X is not broadcast)
//   BN_STREAM  bit 0 / bit 1: X / Y is read with the non-temporal hint (an operand that is read once)
//   BN_F16     1: the operands (and an arithmetic result) are IEEE half in memory; the operation itself is done in
//              fp32 and rounded once, which for + - * / is the correctly rounded half result
// A lane owns BN_VW consecutive elements of the innermost dimension; an operand
// that is contiguous there is read with one 128-bit load, a broadcast one with
// a scalar load.
#define KCG_BN_CAT2(a, b) a##b
#define KCG_BN_CAT(a, b) KCG_BN_CAT2(a, b)
#define BN_APPLY KCG_BN_CAT(BN_NAME, _apply)

#ifndef BN_F16
#define BN_F16 0
#define BN_F16_DEFAULTED
#endif
#if BN_F16
#define BN_IN_T _Float16
#else
#define BN_IN_T float
#endif
#if BN_OP >= 5
typedef unsigned char KCG_BN_CAT(BN_NAME, _out_t);
#else
typedef BN_IN_T KCG_BN_CAT(BN_NAME, _out_t);
#endif
#define BN_OUT_T KCG_BN_CAT(BN_NAME, _out_t)

__device__ __forceinline__ BN_OUT_T BN_APPLY(float x, float y) {
#if BN_OP == 0
  return (BN_OUT_T)(x + y);
#elif BN_OP == 1
  return (BN_OUT_T)(x - y);
#elif BN_OP == 2
  return (BN_OUT_T)(x * y);
#elif BN_OP == 3
  return (BN_OUT_T)(x / y);
#elif BN_OP == 4
  return (BN_OUT_T)__powf(x, y);
#elif BN_OP == 5
  return x == y ? 1 : 0;
#elif BN_OP == 6
  return x > y ? 1 : 0;
#else
#error "unknown BN_OP"
#endif
}

#ifndef BN_STREAM
#define BN_STREAM 0
#define BN_STREAM_DEFAULTED
#endif
extern "C" __global__ __launch_bounds__(BN_BLOCK)
#if BN_INPLACE
void BN_NAME(BN_IN_T* __restrict__ X, const BN_IN_T* __restrict__ Y) {
  BN_IN_T* __restrict__ Z = X;
#else
void BN_NAME(const BN_IN_T* __restrict__ X, const BN_IN_T* __restrict__ Y, BN_OUT_T* __restrict__ Z) {
#endif
  typedef BN_IN_T vec_t __attribute__((ext_vector_type(BN_VW)));
  typedef BN_OUT_T out_vec_t __attribute__((ext_vector_type(BN_VW)));
  constexpr long dims[BN_RANK] = {BN_DIMS};
  constexpr long sa[BN_RANK] = {BN_SA};
  constexpr long sb[BN_RANK] = {BN_SB};
  long total = 1;
#pragma unroll
  for (int d = 0; d < BN_RANK; ++d) total *= dims[d];
  const long idx = ((long)blockIdx.x * BN_BLOCK + threadIdx.x) * BN_VW;   // flat index of the lane's first element
  if (idx >= total) return;
  long rest = idx, offA = 0, offB = 0;
#pragma unroll
  for (int d = BN_RANK - 1; d >= 0; --d) {
    const long i = rest % dims[d];
    rest /= dims[d];
    offA += i * sa[d];
    offB += i * sb[d];
  }
  vec_t x, y;
  out_vec_t z;
  if (sa[BN_RANK - 1] == 1) {
    x = kcg_stream_load<(BN_STREAM & 1) != 0>((const vec_t*)(X + offA));
  } else {
    const BN_IN_T s = X[offA];
#pragma unroll
    for (int j = 0; j < BN_VW; ++j) x[j] = s;
  }
  if (sb[BN_RANK - 1] == 1) {
    y = kcg_stream_load<(BN_STREAM & 2) != 0>((const vec_t*)(Y + offB));
  } else {
    const BN_IN_T s = Y[offB];
#pragma unroll
    for (int j = 0; j < BN_VW; ++j) y[j] = s;
  }
#pragma unroll
  for (int j = 0; j < BN_VW; ++j) z[j] = BN_APPLY((float)x[j], (float)y[j]);
  __builtin_nontemporal_store(z, (out_vec_t*)(Z + idx));
}
#undef BN_APPLY
#undef BN_OUT_T
#undef BN_IN_T
#ifdef BN_F16_DEFAULTED
#undef BN_F16
#undef BN_F16_DEFAULTED
#endif
#ifdef BN_STREAM_DEFAULTED
#undef BN_STREAM
#undef BN_STREAM_DEFAULTED
#endif
