// ---- gather along one axis ----
// out[o, i, r] = in[o, idx[i], r]   o < GA_OUTER, i < GA_NIDX, r < GA_ROW bytes
// The input is [GA_OUTER][GA_AXIS][row], the indices are GA_NIDX 64-bit integers (the device form of the
// IR's `index` element type), the output [GA_OUTER][GA_NIDX][row].  A row is GA_ROW bytes and is moved in
// units of GA_VB bytes (16, 8, 4 or 2: the largest that divides the row), one unit per lane, so lanes of a
// wavefront read consecutive units of one or a few rows.
// An index outside [0, GA_AXIS) is clamped to the nearest valid row: the kernel never reads outside the input.
// Parameters: GA_NAME, GA_OUTER, GA_AXIS, GA_NIDX, GA_ROW, GA_VB, GA_BLOCK, GA_UNROLL (units per lane).
#if GA_VB == 16
typedef kcg_u32x4 kcg_ga_unit;
#elif GA_VB == 8
typedef kcg_u32x2 kcg_ga_unit;
#elif GA_VB == 4
typedef unsigned kcg_ga_unit;
#elif GA_VB == 2
typedef unsigned short kcg_ga_unit;
#else
#error "gather: GA_VB must be 16, 8, 4 or 2"
#endif
#if GA_ROW % GA_VB
#error "gather: the unit must divide the row"
#endif
#define GA_RV (GA_ROW / GA_VB)                       // units per row
#define GA_TOTAL ((long)GA_OUTER * GA_NIDX * GA_RV)  // units of the output

extern "C" __global__ __launch_bounds__(GA_BLOCK)
void GA_NAME(const kcg_ga_unit* __restrict__ in, const long long* __restrict__ idx, kcg_ga_unit* __restrict__ out) {
  // A lane moves GA_UNROLL units GA_BLOCK apart: all its index loads are issued first, then all its row loads,
  // so that the two dependent latencies are paid once per lane and not once per unit.
  const long base = (long)blockIdx.x * (GA_BLOCK * GA_UNROLL) + threadIdx.x;
  long src[GA_UNROLL];
#pragma unroll
  for (int k = 0; k < GA_UNROLL; ++k) {
    const long u = base + (long)k * GA_BLOCK;
    src[k] = -1;
    if (u < GA_TOTAL) {
      const long c = u % GA_RV;
      const long i = (u / GA_RV) % GA_NIDX;
      const long o = u / ((long)GA_RV * GA_NIDX);
      long long j = idx[i];
      j = j < 0 ? 0 : (j >= GA_AXIS ? GA_AXIS - 1 : j);
      src[k] = (o * GA_AXIS + j) * GA_RV + c;
    }
  }
  kcg_ga_unit v[GA_UNROLL];
#pragma unroll
  for (int k = 0; k < GA_UNROLL; ++k)
    if (src[k] >= 0) v[k] = in[src[k]];       // table rows may repeat: cached loads, streaming stores
#pragma unroll
  for (int k = 0; k < GA_UNROLL; ++k)
    if (src[k] >= 0) __builtin_nontemporal_store(v[k], out + base + (long)k * GA_BLOCK);
}
#undef GA_UNROLL
#undef GA_RV
#undef GA_TOTAL
