// ---- shared prelude of every emitted gfx950 translation unit ---------------
// Wavefronts are 64 lanes wide.  Types are spelled with clang vector
// extensions so the file needs no header beyond the HIP runtime built-ins.
#ifndef __HIPCC_RTC__
#include <hip/hip_runtime.h>  // offline hipcc builds; hipRTC has the built-ins already
#endif

typedef float kcg_f32x4 __attribute__((ext_vector_type(4)));
typedef float kcg_f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 kcg_bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned int kcg_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int kcg_u32x2 __attribute__((ext_vector_type(2)));
typedef int kcg_i32x8 __attribute__((ext_vector_type(8)));
typedef int kcg_i32x4 __attribute__((ext_vector_type(4)));

#define KCG_WAVE 64

// Load of data that is read once, for the single-pass kernels (elementwise, softmax, LayerNorm); NT selects the
// non-temporal hint (the kernels' STREAM parameter, on by default).  Measured on 16384 x 4096 fp32 with three
// rotating buffer sets (operands in HBM): GELU 6.55 against 6.2 TB/s, softmax 6.15 against 5.8, LayerNorm + GELU
// 6.15 against 5.95 with the hint; on one buffer set (operands left in the last-level cache by the previous
// launch, as between a producer and its consumer) the hint costs about 10 %.  The broadcast binary kernel gains
// nothing from it and uses plain loads.
template <bool NT, class T> __device__ __forceinline__ T kcg_stream_load(const T* p) {
  if (NT) return __builtin_nontemporal_load(p);
  return *p;
}

// Butterfly reductions over the 64 lanes of a wavefront; every lane ends up
// holding the result.
__device__ __forceinline__ float kcg_wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, KCG_WAVE);
  return v;
}
__device__ __forceinline__ float kcg_wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, KCG_WAVE));
  return v;
}

// tanh(u) = 1 - 2 / (exp(2u) + 1) on the hardware exp2 and reciprocal.
// Absolute error stays below 4e-7 over the whole real line.
__device__ __forceinline__ float kcg_fast_tanh(float u) {
  float e = __builtin_amdgcn_exp2f(u * 2.885390081777927f);  // exp(2u)
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f);
}

// GELU, tanh form with the Frontend's truncated constants 0.797884 and 0.044715:
//   0.5 x (1 + tanh(u)) = x - x / (exp(2u) + 1),   u = 0.797884 (x + 0.044715 x^3)
// with exp(2u) = exp2(x (A + B x^2)), A = 2 log2(e) 0.797884, B = A 0.044715: five VALU
// instructions, one exp2 and one reciprocal per element.  Saturates cleanly: exp2 -> inf gives
// x, exp2 -> 0 gives x - x = 0.
__device__ __forceinline__ float kcg_gelu(float x) {
  const float a = x * __builtin_fmaf(x * x, 0.10294316f, 2.3022065f);
  const float r = __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(a) + 1.0f);
  return __builtin_fmaf(-x, r, x);
}

// Round-to-nearest-even fp32 -> bf16 bit pattern; a NaN stays a (quiet) NaN instead of being carried
// over into the exponent by the rounding increment.
__device__ __forceinline__ unsigned int kcg_f32_to_bf16_bits(float f) {
  unsigned int u = __builtin_bit_cast(unsigned int, f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;
  u += 0x7FFFu + ((u >> 16) & 1u);
  return u >> 16;
}
// Two fp32 -> one dword of two bf16 (lo in bits 0..15), round-to-nearest-even:
// the vector conversion is one v_cvt_pk_bf16_f32 on gfx950.
typedef __bf16 kcg_bf16x2 __attribute__((ext_vector_type(2)));
typedef float kcg_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned int kcg_pack_bf16x2(float lo, float hi) {
  kcg_f32x2 v = {lo, hi};
  return __builtin_bit_cast(unsigned int, __builtin_convertvector(v, kcg_bf16x2));
}

// The same for IEEE half.
typedef _Float16 kcg_f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned int kcg_pack_f16x2(float lo, float hi) {
  kcg_f32x2 v = {lo, hi};
  return __builtin_bit_cast(unsigned int, __builtin_convertvector(v, kcg_f16x2));
}

// Workgroup id -> output tile.  Consecutive workgroup ids are dealt round-robin
// to the 8 XCDs, each with its own L2; the first step renumbers them so that
// one XCD receives a contiguous run of tiles.  The second step walks that run
// in column-major strips of `group_m` tile rows so that the A and B panels a
// strip touches stay L2-resident.
__device__ __forceinline__ void kcg_tile_coords(int pid, int tiles_m, int tiles_n, int group_m,
                                                int& tile_m, int& tile_n) {
  const int nb = tiles_m * tiles_n;
  if ((nb & 7) == 0) pid = (pid & 7) * (nb >> 3) + (pid >> 3);
  const int per_group = group_m * tiles_n;
  const int g = pid / per_group;
  const int first_m = g * group_m;
  const int rows = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
  const int in_g = pid - g * per_group;
  tile_m = first_m + in_g % rows;
  tile_n = in_g / rows;
}
