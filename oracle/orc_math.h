// TEST INFRASTRUCTURE — CPU oracle for the Seedless decode path.  Nothing outside tests/,
// __graft_entry__.smoke() and bench.py's cpu_baseline leg may use this directory.
//
// orc_math.h: the scalar arithmetic every stage of the oracle is built from.  All functions use
// only IEEE-754 binary32 +,-,*,/,sqrt, fmaf and integer operations, so a GPU implementation of
// the same expressions (compiled without contraction) produces identical bits.  The reference
// calls Metal's precise::exp / precise::log / fast::exp at these points
// (SeedlessFusedVerify.swift:198, 654, 931-935; SeedlessMetalForward.swift:4966-4967); their
// last-bit behaviour is not portable, so this build fixes its own.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstring>
#if defined(__F16C__)
#include <immintrin.h>
#endif

namespace orc {

static inline uint32_t f2u(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

// ---- IEEE half <-> float, round to nearest even ------------------------------------------------
static inline uint16_t f2h_soft(float f) {
  uint32_t x = f2u(f);
  uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7fffffffu;
  if (x >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | ((x > 0x7f800000u) ? 0x200u : 0u));
  if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);            // rounds to >= 65520 -> inf
  if (x < 0x38800000u) {                                              // subnormal half or zero
    if (x < 0x33000000u) return (uint16_t)sign;                       // < 2^-25 -> 0
    uint32_t e = x >> 23;                                             // 102..112
    uint32_t mant = (x & 0x7fffffu) | 0x800000u;
    uint32_t shift = 126u - e;                                        // 14..24
    uint32_t r = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (r & 1u))) r++;
    return (uint16_t)(sign | r);
  }
  uint32_t r = x - 0x38000000u;                                       // rebias exponent
  uint32_t rem = r & 0x1fffu;
  r >>= 13;
  if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++;
  return (uint16_t)(sign | r);
}
static inline float h2f_soft(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 31u, m = h & 0x3ffu;
  if (e == 31u) return u2f(sign | 0x7f800000u | (m << 13));
  if (e == 0u) {
    if (m == 0u) return u2f(sign);
    float v = (float)m * 5.9604644775390625e-8f;                      // m * 2^-24, exact
    return sign ? -v : v;
  }
  return u2f(sign | ((e + 112u) << 23) | (m << 13));
}
#if defined(__F16C__)
static inline uint16_t f2h(float f) { return (uint16_t)_cvtss_sh(f, 0); }
static inline float h2f(uint16_t h) { return _cvtsh_ss(h); }
#else
static inline uint16_t f2h(float f) { return f2h_soft(f); }
static inline float h2f(uint16_t h) { return h2f_soft(h); }
#endif
// Round a float to the nearest half and return it as a float.
static inline float f16r(float x) { return h2f(f2h(x)); }

// ---- exp -----------------------------------------------------------------------------------------
// n = rint(x*log2 e); r = x - n*ln2 (two-constant Cody-Waite); degree-6 polynomial; scale by 2^n
// in two exact steps.  x > 88.72 -> +inf, x < -86 -> 0 (no subnormal results).
static inline float exp_c(float x) {
  if (x > 88.72f) return INFINITY;
  if (!(x >= -86.0f)) return 0.0f;                                    // also maps NaN to 0
  float n = std::rint(x * 1.44269504f);
  float r = std::fmaf(n, -0.693359375f, x);
  r = std::fmaf(n, 2.12194440e-4f, r);
  float p = 1.9875691500e-4f;
  p = std::fmaf(p, r, 1.3981999507e-3f);
  p = std::fmaf(p, r, 8.3334519073e-3f);
  p = std::fmaf(p, r, 4.1665795894e-2f);
  p = std::fmaf(p, r, 1.6666665459e-1f);
  p = std::fmaf(p, r, 5.0000001201e-1f);
  float y = std::fmaf(p, r * r, r) + 1.0f;
  int ni = (int)n;
  int a = ni >> 1, b = ni - a;
  return (y * u2f((uint32_t)(a + 127) << 23)) * u2f((uint32_t)(b + 127) << 23);
}

// ---- log, for normal positive x ----------------------------------------------------------------
// x = m*2^e with m in (sqrt(1/2), sqrt(2)]; s = (m-1)/(m+1); log m = s*(2 + 2/3 s^2 + ... + 2/9 s^8).
static inline float log_c(float x) {
  uint32_t u = f2u(x);
  int e = (int)((u >> 23) & 255u) - 127;
  float m = u2f((u & 0x7fffffu) | 0x3f800000u);
  if (m > 1.41421356f) { m = m * 0.5f; e += 1; }
  float f = m - 1.0f;
  float s = f / (2.0f + f);
  float z = s * s;
  float p = 0.2222222222f;
  p = std::fmaf(p, z, 0.2857142857f);
  p = std::fmaf(p, z, 0.4f);
  p = std::fmaf(p, z, 0.6666666667f);
  p = std::fmaf(p, z, 2.0f);
  return std::fmaf((float)e, 0.69314718f, s * p);
}

// ---- sigmoid family --------------------------------------------------------------------------------
// fp32 "stable" sigmoid: y = 1/(1+exp|x|); x<0 ? y : 1-y  (SeedlessFusedVerify.swift:652-654).
static inline float sigmoid32(float x) {
  float y = 1.0f / (1.0f + exp_c(std::fabs(x)));
  return (x < 0.0f) ? y : (1.0f - y);
}
// The same expression evaluated in half precision, every operation rounded to half
// (SeedlessMetalForward.swift:987-989).  x must already be a half value.
static inline float sigmoid16(float x) {
  float e = f16r(exp_c(std::fabs(x)));
  float d = f16r(1.0f + e);
  float y = f16r(1.0f / d);
  return (x < 0.0f) ? y : f16r(1.0f - y);
}
// softplus(x) = max(x,0) + log(1 + exp(-|x|))  (SeedlessFusedVerify.swift:932-934).
static inline float softplus_c(float x) {
  return std::fmax(x, 0.0f) + log_c(1.0f + exp_c(-std::fabs(x)));
}

// ---- counter-based generator ---------------------------------------------------------------------
// 64-bit mix of (seed, index) -> 23-bit uniform in (0,1) -> standard normal by Wichura's AS241
// PPND7 rational approximation.
static inline uint64_t hash64(uint64_t seed, uint64_t idx) {
  uint64_t z = (idx + 1ull) * 0x9E3779B97F4A7C15ull ^ (seed * 0xD1B54A32D192ED03ull + 0x8CB92BA72F3D8DD7ull);
  z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ull;
  z ^= z >> 27; z *= 0x94D049BB133111EBull;
  z ^= z >> 31;
  return z;
}
static inline float uniform01(uint64_t seed, uint64_t idx) {
  uint32_t k = (uint32_t)(hash64(seed, idx) >> 41);                   // 23 bits
  return (float)(2u * k + 1u) * 5.9604644775390625e-8f;               // (2k+1) * 2^-24, exact
}
static inline float ppnd7(float p) {
  float q = p - 0.5f;
  if (std::fabs(q) <= 0.425f) {
    float r = 0.180625f - q * q;
    float num = ((5.9109374720e+01f * r + 1.5929113202e+02f) * r + 5.0434271938e+01f) * r + 3.3871327179e+00f;
    float den = ((6.7187563600e+01f * r + 7.8757757664e+01f) * r + 1.7895169469e+01f) * r + 1.0f;
    return q * num / den;
  }
  float r = (q < 0.0f) ? p : (1.0f - p);
  r = std::sqrt(-log_c(r));
  float v;
  if (r <= 5.0f) {
    r = r - 1.6f;
    float num = ((1.7023821103e-01f * r + 1.3067284816e+00f) * r + 2.7568153900e+00f) * r + 1.4234372777e+00f;
    float den = (1.2021132975e-01f * r + 7.3700164250e-01f) * r + 1.0f;
    v = num / den;
  } else {
    r = r - 5.0f;
    float num = ((1.7337203997e-02f * r + 4.2868294337e-01f) * r + 3.0812263860e+00f) * r + 6.6579051150e+00f;
    float den = (1.2258202635e-02f * r + 2.4197894225e-01f) * r + 1.0f;
    v = num / den;
  }
  return (q < 0.0f) ? -v : v;
}
static inline float normal01(uint64_t seed, uint64_t idx) { return ppnd7(uniform01(seed, idx)); }

// Balanced binary tree over n = 2^j values, adjacent pairs first: ((v0+v1)+(v2+v3))+...
static inline float tree_sum(float* v, int n) {
  for (int s = 1; s < n; s <<= 1)
    for (int i = 0; i < n; i += 2 * s) v[i] = v[i] + v[i + s];
  return v[0];
}

}  // namespace orc
