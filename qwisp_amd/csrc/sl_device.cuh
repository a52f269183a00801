// Device-side scalar arithmetic and wave64 helpers for the Seedless kernels (gfx950).
//
// Every function here is built from IEEE binary32 +,-,*,/,sqrt, fmaf and integer operations only
// and the translation unit is compiled with -ffp-contract=off, so results do not depend on how
// a kernel is tiled.  Reductions: lanes are combined by an xor-butterfly (adjacent lanes first), which
// is a balanced binary tree whose value is the same on every lane; a lane partial is an fmaf chain over
// elements the lane owns or a sub-tree of the same balanced tree, as stated where it is formed.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#define SL_DEV __device__ __forceinline__

namespace sl {

// Rounding to half is always a separate step applied to an already-rounded fp32 value.  The empty
// asm keeps the compiler from folding the producing fp32 multiply/add into a mixed-precision
// instruction that rounds the exact result to half once (v_fma_mixlo_f16), which differs from
// fp32-then-half rounding in about 6e-5 of cases.
SL_DEV float opaque(float x) { asm("" : "+v"(x)); return x; }
SL_DEV float f16r(float x) { return __half2float(__float2half_rn(opaque(x))); }
SL_DEV float h2f(uint16_t h) { return __half2float(__ushort_as_half(h)); }
SL_DEV uint16_t f2h(float x) { return __half_as_ushort(__float2half_rn(opaque(x))); }

// exp: n = rint(x*log2 e), two-constant Cody-Waite reduction, degree-6 polynomial, 2^n applied in
// two exact steps.  x > 88.72 -> +inf, x < -86 (or NaN) -> 0.
SL_DEV float exp_c(float x) {
  if (x > 88.72f) return __int_as_float(0x7f800000);
  if (!(x >= -86.0f)) return 0.0f;
  float n = rintf(x * 1.44269504f);
  float r = fmaf(n, -0.693359375f, x);
  r = fmaf(n, 2.12194440e-4f, r);
  float p = 1.9875691500e-4f;
  p = fmaf(p, r, 1.3981999507e-3f);
  p = fmaf(p, r, 8.3334519073e-3f);
  p = fmaf(p, r, 4.1665795894e-2f);
  p = fmaf(p, r, 1.6666665459e-1f);
  p = fmaf(p, r, 5.0000001201e-1f);
  float y = fmaf(p, r * r, r) + 1.0f;
  int ni = (int)n;
  int a = ni >> 1, b = ni - a;
  return (y * __int_as_float((a + 127) << 23)) * __int_as_float((b + 127) << 23);
}

// log for normal positive x: x = m*2^e, m in (sqrt(1/2), sqrt(2)], s = (m-1)/(m+1), odd series to s^9.
SL_DEV float log_c(float x) {
  uint32_t u = (uint32_t)__float_as_int(x);
  int e = (int)((u >> 23) & 255u) - 127;
  float m = __int_as_float((int)((u & 0x7fffffu) | 0x3f800000u));
  if (m > 1.41421356f) { m = m * 0.5f; e += 1; }
  float f = m - 1.0f;
  float s = f / (2.0f + f);
  float z = s * s;
  float p = 0.2222222222f;
  p = fmaf(p, z, 0.2857142857f);
  p = fmaf(p, z, 0.4f);
  p = fmaf(p, z, 0.6666666667f);
  p = fmaf(p, z, 2.0f);
  return fmaf((float)e, 0.69314718f, s * p);
}

SL_DEV float sigmoid32(float x) {
  float y = 1.0f / (1.0f + exp_c(fabsf(x)));
  return (x < 0.0f) ? y : (1.0f - y);
}
// Half-precision sigmoid: every operation rounded to half; x must be a half value.
SL_DEV float sigmoid16(float x) {
  float e = f16r(exp_c(fabsf(x)));
  float d = f16r(1.0f + e);
  float y = f16r(1.0f / d);
  return (x < 0.0f) ? y : f16r(1.0f - y);
}
SL_DEV float softplus_c(float x) { return fmaxf(x, 0.0f) + log_c(1.0f + exp_c(-fabsf(x))); }
SL_DEV float swiglu16(float g, float u) { return f16r(f16r(g * sigmoid16(g)) * u); }

// ---- wave64 reductions ------------------------------------------------------------------------------
// The value of every reduction is that of the xor-butterfly (partners at distance 1, 2, 4, ... combined in
// that order), which is a balanced binary tree over adjacent lanes.  After step k all 2^k lanes of a group
// hold the same value, so a lane may take its partner group's value from ANY lane of that group and, the
// operation being commutative, gets the same bits.  That lets the first four steps run as DPP operand
// modifiers (quad permutes, half-row mirror, row mirror: no LDS round trip) and the last two as reads of one
// lane per 16-lane row.
template <int CTRL>
SL_DEV float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
template <int CTRL>
SL_DEV uint32_t dpp_u(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
}
constexpr int DPP_XOR1 = 0xB1;          // quad_perm [1,0,3,2]
constexpr int DPP_XOR2 = 0x4E;          // quad_perm [2,3,0,1]
constexpr int DPP_HALF_MIRROR = 0x141;  // lane i <-> 7-i within 8
constexpr int DPP_MIRROR = 0x140;       // lane i <-> 15-i within 16
constexpr int DPP_SHR1 = 0x111;         // lane i takes lane i-1 within its 16-lane row
SL_DEV float row_lane_f(float v, int lane) { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane)); }
// Values of lanes base..base+7 as scalars.  The empty asm keeps all eight in scalar registers at one point, so the
// extractions are issued back to back ahead of their uses: a scalar written by the vector unit takes tens of cycles
// to become readable, and extraction and use strictly alternating on one register pay that for every element.
SL_DEV void lanes8(float v, int base, float (&out)[8]) {
  int t[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) t[i] = __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), base + i);
  asm volatile("" : "+s"(t[0]), "+s"(t[1]), "+s"(t[2]), "+s"(t[3]), "+s"(t[4]), "+s"(t[5]), "+s"(t[6]), "+s"(t[7]));
#pragma unroll
  for (int i = 0; i < 8; ++i) out[i] = __builtin_bit_cast(float, t[i]);
}

#ifndef SL_SWAP_REDUCE
#define SL_SWAP_REDUCE 1
#endif
// {row0, row1, row2, row3} -> {row0+row1, row0+row1, row2+row3, row2+row3} (rows of 16 lanes), and lower + upper half.
SL_DEV float swap16_sum(float v) {
  const unsigned u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
SL_DEV float swap32_sum(float v) {
  const unsigned u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
template <int WIDTH>
SL_DEV float tree_sum(float v) {
  static_assert(WIDTH == 4 || WIDTH == 8 || WIDTH == 16 || WIDTH == 32 || WIDTH == 64, "group sizes used by the kernels");
  v = v + dpp_f<DPP_XOR1>(v);
  v = v + dpp_f<DPP_XOR2>(v);
  if constexpr (WIDTH == 4) return v;
  v = v + dpp_f<DPP_HALF_MIRROR>(v);
  if constexpr (WIDTH == 8) return v;
  v = v + dpp_f<DPP_MIRROR>(v);
  if constexpr (WIDTH == 16) return v;
#if SL_SWAP_REDUCE
  // rows 0|1 and 2|3, then halves: v_permlane16_swap / v_permlane32_swap of a value with its own copy hand every
  // lane its partner group's value (no trip through scalar registers); a + b == b + a bit for bit
  v = swap16_sum(v);
  if constexpr (WIDTH == 32) return v;
  return swap32_sum(v);
#else
  const float r0 = row_lane_f(v, 0), r1 = row_lane_f(v, 16), r2 = row_lane_f(v, 32), r3 = row_lane_f(v, 48);
  const float lo = r0 + r1, hi = r2 + r3;
  if constexpr (WIDTH == 32) return (__lane_id() < 32) ? lo : hi;
  return lo + hi;
#endif
}
// Four sums over the 64 lanes reduced together.  After the first two levels of tree_sum (lane pairs, then quads)
// the four lanes of a quad hold the same value, so one register can carry all four: lane l the value of row
// rho(l) = l % 4 in the lower quad of every eight lanes and 3 - l % 4 in the upper one.  The partners of the remaining
// levels (mirror within 8, mirror within 16, the other row of 16, the other half) then hold the same row, and every
// addition has the operands it has in tree_sum<64>: the same bits with 19 instead of 40 instructions.  Returns the
// sum of row rho(lane); lanes 0..3 hold rows 0..3.
SL_DEV int quad_row(int lane) { return (lane & 4) ? 3 - (lane & 3) : (lane & 3); }
SL_DEV float tree_sum4(float q0, float q1, float q2, float q3, int lane) {
  q0 = tree_sum<4>(q0); q1 = tree_sum<4>(q1); q2 = tree_sum<4>(q2); q3 = tree_sum<4>(q3);
  const int rho = quad_row(lane);
  float f = rho == 0 ? q0 : (rho == 1 ? q1 : (rho == 2 ? q2 : q3));
  f = f + dpp_f<DPP_HALF_MIRROR>(f);
  f = f + dpp_f<DPP_MIRROR>(f);
  return swap32_sum(swap16_sum(f));
}
// The value of lane j of the caller's quad, j = 0..3 (after tree_sum4: rows 0..3, in the lower quad of every eight lanes).
SL_DEV void quad_values(float f, float (&out)[4]) {
  out[0] = dpp_f<0x00>(f); out[1] = dpp_f<0x55>(f); out[2] = dpp_f<0xAA>(f); out[3] = dpp_f<0xFF>(f);
}
template <int WIDTH>
SL_DEV float tree_max(float v) {
  static_assert(WIDTH == 64, "group sizes used by the kernels");
  v = fmaxf(v, dpp_f<DPP_XOR1>(v));
  v = fmaxf(v, dpp_f<DPP_XOR2>(v));
  v = fmaxf(v, dpp_f<DPP_HALF_MIRROR>(v));
  v = fmaxf(v, dpp_f<DPP_MIRROR>(v));
#if SL_SWAP_REDUCE
  {
    const unsigned u = __float_as_uint(v);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    const unsigned w = __float_as_uint(v);
    const auto q = __builtin_amdgcn_permlane32_swap(w, w, false, false);
    return fmaxf(__uint_as_float(q[0]), __uint_as_float(q[1]));
  }
#else
  const float r0 = row_lane_f(v, 0), r1 = row_lane_f(v, 16), r2 = row_lane_f(v, 32), r3 = row_lane_f(v, 48);
  return fmaxf(fmaxf(r0, r1), fmaxf(r2, r3));
#endif
}
// Largest of an unsigned value over the 64 lanes, in every lane (the tree of tree_max: no trip through scalar registers).
SL_DEV uint32_t wave_max_u32(uint32_t v) {
  v = max(v, dpp_u<DPP_XOR1>(v));
  v = max(v, dpp_u<DPP_XOR2>(v));
  v = max(v, dpp_u<DPP_HALF_MIRROR>(v));
  v = max(v, dpp_u<DPP_MIRROR>(v));
  const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
  v = max(r[0], r[1]);
  const auto q = __builtin_amdgcn_permlane32_swap(v, v, false, false);
  return max(q[0], q[1]);
}
// Value of the previous lane (lanes 0, 16, 32, 48 get 0): for left-to-right chains inside a 16-lane row.
SL_DEV float prev_lane(float v) { return dpp_f<DPP_SHR1>(v); }

// Workgroup barrier for data exchanged through LDS: waits for the wave's LDS operations only.  __syncthreads() also
// waits for every vector-memory load in flight, which would drain weight rows requested ahead of their use.
SL_DEV void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// ---- 16-byte vector access -------------------------------------------------------------------------
SL_DEV uint4 ld16(const void* p) { return *reinterpret_cast<const uint4*>(p); }
SL_DEV void st16(void* p, uint4 v) { *reinterpret_cast<uint4*>(p) = v; }
SL_DEV float lo_h(uint32_t u) { return h2f((uint16_t)(u & 0xffffu)); }
SL_DEV float hi_h(uint32_t u) { return h2f((uint16_t)(u >> 16)); }
// 8 halves (one uint4) -> 8 floats
SL_DEV void unpack8(uint4 v, float* f) {
  f[0] = lo_h(v.x); f[1] = hi_h(v.x); f[2] = lo_h(v.y); f[3] = hi_h(v.y);
  f[4] = lo_h(v.z); f[5] = hi_h(v.z); f[6] = lo_h(v.w); f[7] = hi_h(v.w);
}
SL_DEV uint32_t pack2(float a, float b) { return (uint32_t)f2h(a) | ((uint32_t)f2h(b) << 16); }
SL_DEV uint4 pack8(const float* f) {
  return make_uint4(pack2(f[0], f[1]), pack2(f[2], f[3]), pack2(f[4], f[5]), pack2(f[6], f[7]));
}

// A pointer read from device memory (a table of per-sequence buffers) is device memory itself: saying so lets the
// compiler use global instead of generic ("flat") accesses through it.
template <class T>
SL_DEV T* as_global(T* p) { return (T*)(T __attribute__((address_space(1)))*)(unsigned long long)p; }

// ---- 4-bit dot: a share of 32 activations against 4 packed words ------------------------------------------
// A share is 32 consecutive elements of a row: 4 packed words (one 16-byte load), half a quantisation group, so one
// scale s and one bias b.  Its term is T = fmaf(s, A + B, b * sx), A the fmaf chain over the share's even-indexed
// elements in order, B the chain over the odd-indexed ones, sx the balanced tree over the 16 pair sums.
//
// The activations arrive as 16 packed half pairs {x[2i], x[2i+1]}.  Masking a word with 0x000F000F leaves two halves
// whose bit patterns are the nibbles 0 and 4: as (subnormal) half values they equal q * 2^-24 exactly; masking with
// 0x00F000F0 leaves the nibbles 1 and 5 four bits up, q * 2^-20.  After one shift by 8 the same two masks give the
// nibbles 2 | 6 and 3 | 7: five integer operations per word, no integer-to-float conversion, and the masked halves go
// straight into v_fma_mix_f32.  Every product and partial sum of chain A is thereby the true one times 2^-24, of
// chain B times 2^-20 (powers of two: same roundings), so A + B is formed as fmaf(B', 2^-4, A') and the 2^24 is
// returned with the scale.
typedef _Float16 h2_t __attribute__((ext_vector_type(2)));
SL_DEV h2_t as_h2(uint32_t u) { return __builtin_bit_cast(h2_t, u); }
// The four masked forms of a word: mk[0] nibbles 0 | 4, mk[1] nibbles 1 | 5 (x16), mk[2] nibbles 2 | 6, mk[3] nibbles 3 | 7 (x16).
SL_DEV void word_masks(uint32_t w, h2_t* mk /*4*/) {
  const uint32_t w8 = w >> 8;
  mk[0] = as_h2(w & 0x000F000Fu); mk[1] = as_h2(w & 0x00F000F0u);
  mk[2] = as_h2(w8 & 0x000F000Fu); mk[3] = as_h2(w8 & 0x00F000F0u);
}
// One word's eight multiply-adds: elements 0, 2, 4, 6 onto chain A, elements 1, 3, 5, 7 onto chain B.
SL_DEV void word_chains(const h2_t* mk /*4*/, const uint32_t* xp /*4 packed pairs*/, float& A, float& B) {
  const h2_t x0 = as_h2(xp[0]), x1 = as_h2(xp[1]), x2 = as_h2(xp[2]), x3 = as_h2(xp[3]);
  A = fmaf((float)x0.x, (float)mk[0].x, A);
  B = fmaf((float)x0.y, (float)mk[1].x, B);
  A = fmaf((float)x1.x, (float)mk[2].x, A);
  B = fmaf((float)x1.y, (float)mk[3].x, B);
  A = fmaf((float)x2.x, (float)mk[0].y, A);
  B = fmaf((float)x2.y, (float)mk[1].y, B);
  A = fmaf((float)x3.x, (float)mk[2].y, A);
  B = fmaf((float)x3.y, (float)mk[3].y, B);
}
// T of a share whose 16 masked forms the caller prepared (reused over several activation rows).
SL_DEV float share_term_masked(const h2_t* mk /*16*/, uint32_t sb, const uint32_t* xp /*16 packed pairs*/, float sx) {
  float A = 0.0f, B = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) word_chains(mk + 4 * j, xp + 4 * j, A, B);
  const float s = lo_h(sb) * 16777216.0f, b = hi_h(sb);
  return fmaf(s, fmaf(B, 0.0625f, A), b * sx);
}
SL_DEV float share_term(uint4 w, uint32_t sb, const uint32_t* xp /*16 packed pairs*/, float sx) {
  const uint32_t ws[4] = {w.x, w.y, w.z, w.w};
  float A = 0.0f, B = 0.0f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    h2_t mk[4];
    word_masks(ws[j], mk);
    word_chains(mk, xp + 4 * j, A, B);
  }
  const float s = lo_h(sb) * 16777216.0f, b = hi_h(sb);
  return fmaf(s, fmaf(B, 0.0625f, A), b * sx);
}
// 8-bit affine row dot, group 64 (the router gate and shared-expert gate of the released checkpoint; reference
// kernel qmm8, SeedlessMetalForward.swift:372-428).  Lane l owns the 32 contiguous values 32l..32l+31 = 8 words,
// half a group.  Per 8 values: t = fmaf(s, chain of fmaf(x, q), b * sx) with sx the sequential fp32 sum of the
// eight x; the lane's partial is (t0+t1)+(t2+t3).
SL_DEV float q8_lane(const uint32_t* w8 /*8 words*/, uint32_t sb, const float* x /*32*/) {
  const float s = lo_h(sb), b = hi_h(sb);
  float t[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float dq = 0.0f, sx = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float q = (float)((w8[2 * j + (i >> 2)] >> (8 * (i & 3))) & 255u);
      dq = fmaf(x[8 * j + i], q, dq);
      sx = sx + x[8 * j + i];
    }
    t[j] = fmaf(s, dq, b * sx);
  }
  return (t[0] + t[1]) + (t[2] + t[3]);
}
// 32 half-valued floats -> 16 packed pairs (exact)
SL_DEV void pack_x(const float* x, uint32_t* xp) {
#pragma unroll
  for (int i = 0; i < 16; ++i) xp[i] = pack2(x[2 * i], x[2 * i + 1]);
}
// Sum of a share's 32 activations: balanced tree over the 16 pair sums x[2i] + x[2i+1], adjacent pairs first.
SL_DEV float share_sum(const float* x /*32*/) {
  float p[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) p[i] = x[2 * i] + x[2 * i + 1];
#pragma unroll
  for (int st = 1; st < 16; st <<= 1)
#pragma unroll
    for (int i = 0; i < 16; i += 2 * st) p[i] = p[i] + p[i + st];
  return p[0];
}
// The same from the packed pairs.
SL_DEV float share_sum_packed(const uint32_t* xp /*16*/) {
  float p[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) p[i] = lo_h(xp[i]) + hi_h(xp[i]);
#pragma unroll
  for (int st = 1; st < 16; st <<= 1)
#pragma unroll
    for (int i = 0; i < 16; i += 2 * st) p[i] = p[i] + p[i + st];
  return p[0];
}
// Sum of squares of 32 consecutive elements as the sub-tree of the canonical order: pair terms fmaf(x1, x1, x0*x0),
// then a balanced tree over the 16 of them.  (A sum of squares over D elements is the balanced binary tree over its
// D/2 pair terms, adjacent ones first; lanes that own aligned runs of 32 elements continue it with tree_sum.)
SL_DEV float share_sumsq(const float* x /*32*/) {
  float p[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) p[i] = fmaf(x[2 * i + 1], x[2 * i + 1], x[2 * i] * x[2 * i]);
#pragma unroll
  for (int st = 1; st < 16; st <<= 1)
#pragma unroll
    for (int i = 0; i < 16; i += 2 * st) p[i] = p[i] + p[i + st];
  return p[0];
}

// ---- counter-based generator (the same rule a host implementation can state) -----------------------
SL_DEV uint64_t hash64(uint64_t seed, uint64_t idx) {
  uint64_t z = (idx + 1ull) * 0x9E3779B97F4A7C15ull ^ (seed * 0xD1B54A32D192ED03ull + 0x8CB92BA72F3D8DD7ull);
  z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ull;
  z ^= z >> 27; z *= 0x94D049BB133111EBull;
  z ^= z >> 31;
  return z;
}
SL_DEV float uniform01(uint64_t seed, uint64_t idx) {
  uint32_t k = (uint32_t)(hash64(seed, idx) >> 41);
  return (float)(2u * k + 1u) * 5.9604644775390625e-8f;
}
// Wichura AS241 PPND7, single precision.
SL_DEV float ppnd7(float p) {
  float q = p - 0.5f;
  if (fabsf(q) <= 0.425f) {
    float r = 0.180625f - q * q;
    float num = ((5.9109374720e+01f * r + 1.5929113202e+02f) * r + 5.0434271938e+01f) * r + 3.3871327179e+00f;
    float den = ((6.7187563600e+01f * r + 7.8757757664e+01f) * r + 1.7895169469e+01f) * r + 1.0f;
    return q * num / den;
  }
  float r = (q < 0.0f) ? p : (1.0f - p);
  r = sqrtf(-log_c(r));
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
SL_DEV float normal01(uint64_t seed, uint64_t idx) { return ppnd7(uniform01(seed, idx)); }

}  // namespace sl
