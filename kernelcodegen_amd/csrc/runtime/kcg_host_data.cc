// Seeded synthetic operands and narrow-float codecs on the host (declared in include/kcg_hip.h).
// Used by KernelCodeGenerator::evaluate(), by the host adaptor it generates and by the benchmark, so that
// all three fill a buffer of a given (seed, stream) with the same bits.
#include "kcg_hip.h"

#include <cmath>
#include <cstdint>
#include <cstring>

namespace {

inline uint64_t mix(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

inline uint32_t bitsOf(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
inline float floatOf(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

// ---- bf16 ------------------------------------------------------------------
inline uint16_t toBf16(float f) {
  uint32_t u = bitsOf(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);   // NaN stays a quiet NaN
  return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}
inline float fromBf16(uint16_t h) { return floatOf((uint32_t)h << 16); }

// ---- IEEE half --------------------------------------------------------------
inline uint16_t toF16(float f) {
  const uint32_t u = bitsOf(f);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const uint32_t mag = u & 0x7FFFFFFFu;
  if (mag > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);
  if (mag >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);    // rounds to 65520 or more: infinity
  if (mag < 0x33000001u) return sign;                           // at most 2^-25: rounds to zero
  int e = (int)(mag >> 23) - 127;
  uint32_t m = (mag & 0x7FFFFFu) | 0x800000u;                   // 1.m, 24 bits
  int shift = 13;                                               // to a 10-bit fraction
  if (e < -14) { shift += -14 - e; e = -15; }                   // subnormal half
  const uint32_t kept = m >> shift, rest = m & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
  uint32_t r = kept + ((rest > halfway || (rest == halfway && (kept & 1u))) ? 1u : 0u);
  // r carries the hidden bit (normal) or not (subnormal); adding it to the exponent field handles the carry
  const uint32_t bits = e == -15 ? r : (((uint32_t)(e + 15) << 10) + (r - 0x400u));
  return (uint16_t)(sign | bits);
}
inline float fromF16(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const int e = (h >> 10) & 0x1F;
  const uint32_t m = h & 0x3FFu;
  if (e == 0x1F) return floatOf(sign | 0x7F800000u | (m << 13));
  if (e == 0) {
    const float v = std::ldexp((float)m, -24);
    return sign ? -v : v;
  }
  return floatOf(sign | ((uint32_t)(e + 112) << 23) | (m << 13));
}

// ---- OCP e4m3fn: bias 7, no infinities, 0x7F / 0xFF are NaN, largest finite value 448 --------------------
struct E4m3Table {
  float value[128];       // magnitudes of the codes 0..0x7E; 0x7F is NaN
  E4m3Table() {
    for (int c = 0; c < 128; ++c) {
      const int e = c >> 3, m = c & 7;
      value[c] = e == 0 ? std::ldexp((float)m, -9) : std::ldexp(1.0f + (float)m / 8.0f, e - 7);
    }
  }
};
const E4m3Table& e4m3() {
  static const E4m3Table t;
  return t;
}
inline float fromE4m3(uint8_t b) {
  if ((b & 0x7Fu) == 0x7Fu) return floatOf(0x7FC00000u | ((uint32_t)(b & 0x80u) << 24));
  const float v = e4m3().value[b & 0x7Fu];
  return (b & 0x80u) ? -v : v;
}
inline uint8_t toE4m3(float f) {
  const uint8_t sign = (uint8_t)((bitsOf(f) >> 24) & 0x80u);
  const float a = std::fabs(f);
  if (a != a) return (uint8_t)(sign | 0x7Fu);
  const float* v = e4m3().value;
  if (a >= v[0x7E]) return (uint8_t)(sign | 0x7Eu);
  // the largest code whose value does not exceed a, by bisection over the monotone table
  int lo = 0, hi = 0x7E;
  while (hi - lo > 1) {
    const int mid = (lo + hi) / 2;
    if (v[mid] <= a) lo = mid; else hi = mid;
  }
  const float below = a - v[lo], above = v[hi] - a;      // both exact: neighbours differ by one unit of a's binade
  int code = lo;
  if (above < below || (above == below && (lo & 1))) code = hi;
  return (uint8_t)(sign | (uint8_t)code);
}

template <typename F>
void generate(size_t count, int dist, uint64_t seed, uint64_t stream, float p0, float p1, F&& put) {
  const uint64_t base = seed + (stream << 40);
  if (dist == KCG_DIST_UNIFORM) {
    for (size_t i = 0; i < count; ++i) {
      const float u = (float)(mix(base + i) >> 40) * (1.0f / 16777216.0f);
      put(i, p0 + (p1 - p0) * u);
    }
    return;
  }
  const double twoPi = 6.283185307179586476925286766559;
  for (size_t i = 0; i < count; i += 2) {
    const double u1 = ((double)(mix(base + i) >> 11) + 1.0) * (1.0 / 9007199254740992.0);   // (0,1]
    const double u2 = (double)(mix(base + i + 1) >> 11) * (1.0 / 9007199254740992.0);       // [0,1)
    const double radius = std::sqrt(-2.0 * std::log(u1));
    put(i, (float)((double)p0 + (double)p1 * radius * std::cos(twoPi * u2)));
    if (i + 1 < count) put(i + 1, (float)((double)p0 + (double)p1 * radius * std::sin(twoPi * u2)));
  }
}

inline void store(void* dst, size_t i, int dtype, float v) {
  switch (dtype) {
    case KCG_DT_F32: ((float*)dst)[i] = v; break;
    case KCG_DT_BF16: ((uint16_t*)dst)[i] = toBf16(v); break;
    case KCG_DT_F8E4M3: ((uint8_t*)dst)[i] = toE4m3(v); break;
    case KCG_DT_F16: ((uint16_t*)dst)[i] = toF16(v); break;
    case KCG_DT_F64: ((double*)dst)[i] = (double)v; break;
    case KCG_DT_I32: ((int32_t*)dst)[i] = (int32_t)v; break;
    case KCG_DT_I64: ((int64_t*)dst)[i] = (int64_t)v; break;
    case KCG_DT_I16: ((int16_t*)dst)[i] = (int16_t)v; break;
    case KCG_DT_I8: ((int8_t*)dst)[i] = (int8_t)v; break;
  }
}

}  // namespace

extern "C" {

size_t kcg_dtype_size(int dtype) {
  switch (dtype) {
    case KCG_DT_F32: case KCG_DT_I32: return 4;
    case KCG_DT_BF16: case KCG_DT_F16: case KCG_DT_I16: return 2;
    case KCG_DT_F8E4M3: case KCG_DT_I8: return 1;
    case KCG_DT_F64: case KCG_DT_I64: return 8;
    default: return 0;
  }
}

int kcg_host_fill(void* dst, size_t count, int dtype, int dist, uint64_t seed, uint64_t stream,
                  float p0, float p1, float scale) {
  if ((!dst && count) || kcg_dtype_size(dtype) == 0 || (dist != KCG_DIST_UNIFORM && dist != KCG_DIST_NORMAL))
    return KCG_ERR_INVALID_ARGUMENT;
  if (scale == 1.0f) generate(count, dist, seed, stream, p0, p1, [&](size_t i, float v) { store(dst, i, dtype, v); });
  else generate(count, dist, seed, stream, p0, p1, [&](size_t i, float v) { store(dst, i, dtype, v * scale); });
  return KCG_OK;
}

int kcg_host_to_f32(const void* src, float* dst, size_t count, int dtype) {
  if ((count && (!src || !dst)) || kcg_dtype_size(dtype) == 0) return KCG_ERR_INVALID_ARGUMENT;
  for (size_t i = 0; i < count; ++i) {
    switch (dtype) {
      case KCG_DT_F32: dst[i] = ((const float*)src)[i]; break;
      case KCG_DT_BF16: dst[i] = fromBf16(((const uint16_t*)src)[i]); break;
      case KCG_DT_F8E4M3: dst[i] = fromE4m3(((const uint8_t*)src)[i]); break;
      case KCG_DT_F16: dst[i] = fromF16(((const uint16_t*)src)[i]); break;
      case KCG_DT_F64: dst[i] = (float)((const double*)src)[i]; break;
      case KCG_DT_I32: dst[i] = (float)((const int32_t*)src)[i]; break;
      case KCG_DT_I64: dst[i] = (float)((const int64_t*)src)[i]; break;
      case KCG_DT_I16: dst[i] = (float)((const int16_t*)src)[i]; break;
      case KCG_DT_I8: dst[i] = (float)((const int8_t*)src)[i]; break;
    }
  }
  return KCG_OK;
}

int kcg_host_from_f32(const float* src, void* dst, size_t count, int dtype, float scale) {
  if ((count && (!src || !dst)) || kcg_dtype_size(dtype) == 0) return KCG_ERR_INVALID_ARGUMENT;
  for (size_t i = 0; i < count; ++i) store(dst, i, dtype, scale == 1.0f ? src[i] : src[i] * scale);
  return KCG_OK;
}

}  // extern "C"
