// ---- Elementwise map over a flat tensor, one pass over HBM ------------------
// Parameters:
//   EW_NAME    kernel symbol          EW_N      number of elements
//   EW_OP      0 Tanh, 1 Sqrt, 2 Log, 3 Relu, 4 Gelu, 5 Cast (value conversion)
//   EW_VW      vector width (4 or 1)  EW_BLOCK  threads per block
//   EW_UNROLL  vectors per thread     EW_INPLACE 1: the kernel has one pointer
//   EW_IN_T / EW_OUT_T element types (float, int, ...)
//   EW_STREAM    1: the input is read with the non-temporal hint (it is read once); 0: plain loads
// Thread t of block b handles vectors (b*EW_UNROLL + u)*EW_BLOCK + t, so every
// wavefront issues fully coalesced 128-bit accesses, EW_UNROLL of them in
// flight per lane.
#define KCG_EW_CAT2(a, b) a##b
#define KCG_EW_CAT(a, b) KCG_EW_CAT2(a, b)
#define EW_APPLY KCG_EW_CAT(EW_NAME, _apply)

__device__ __forceinline__ EW_OUT_T EW_APPLY(EW_IN_T x) {
#if EW_OP == 0
  return kcg_fast_tanh(x);
#elif EW_OP == 1
  return __builtin_sqrtf(x);
#elif EW_OP == 2
  return __logf(x);
#elif EW_OP == 3
  return fmaxf(0.0f, x);
#elif EW_OP == 4
  return kcg_gelu(x);
#elif EW_OP == 5
  return static_cast<EW_OUT_T>(x);
#else
#error "unknown EW_OP"
#endif
}

extern "C" __global__ __launch_bounds__(EW_BLOCK)
#if EW_INPLACE
void EW_NAME(EW_IN_T* __restrict__ X) {
  EW_OUT_T* __restrict__ Y = (EW_OUT_T*)X;
#else
void EW_NAME(const EW_IN_T* __restrict__ X, EW_OUT_T* __restrict__ Y) {
#endif
  typedef EW_IN_T in_vec __attribute__((ext_vector_type(EW_VW)));
  typedef EW_OUT_T out_vec __attribute__((ext_vector_type(EW_VW)));
  const long base = (long)blockIdx.x * EW_UNROLL * EW_BLOCK + threadIdx.x;
  in_vec v[EW_UNROLL];
#pragma unroll
  for (int u = 0; u < EW_UNROLL; ++u) {
    const long idx = (base + (long)u * EW_BLOCK) * EW_VW;
    if (idx < (long)EW_N) v[u] = kcg_stream_load<EW_STREAM != 0>((const in_vec*)(X + idx));
  }
#pragma unroll
  for (int u = 0; u < EW_UNROLL; ++u) {
    const long idx = (base + (long)u * EW_BLOCK) * EW_VW;
    if (idx < (long)EW_N) {
      out_vec o;
#pragma unroll
      for (int j = 0; j < EW_VW; ++j) o[j] = EW_APPLY(v[u][j]);
      __builtin_nontemporal_store(o, (out_vec*)(Y + idx));
    }
  }
}
#undef EW_APPLY
