// Matrix-core GEMM with 4-bit dequantisation for rows of a prefill chunk ("hybrid" prefill; the reference runs
// these projections on the matrix units as well and documents them as not bit-identical to its GEMV path,
// SeedlessFusedVerify.swift:4240-4247).
//
//   Y[m, n] = half( sum_k X[m, k] * half(s * q + b) ),  X fp16 [M, K], W MLX-affine 4-bit group 64 [N, K],
//   the weight formed in half arithmetic (one fused multiply-add), fp32 accumulation in v_mfma_f32_32x32x8_f16.
//
// A wave owns a 32x32 tile of Y (32 rows of X against 32 weight rows): it walks K in chunks of 64 (one
// quantisation group), dequantises its 4 weights per MFMA step in registers and feeds them as the B operand;
// the X chunk [M, 64] is staged in LDS by the whole workgroup (double-buffered, one barrier per chunk) and
// read as the A operand.  A row's result depends only on that row of X and on W, and K is walked in a fixed
// order, so the result is independent of M and of the chunking of a prompt.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sl_kernels.cuh"

namespace sl {

typedef _Float16 mf_h4 __attribute__((ext_vector_type(4)));
typedef float mf_f16v __attribute__((ext_vector_type(16)));
typedef _Float16 mf_h2 __attribute__((ext_vector_type(2)));

// Dequantisation of a lane's 4 weights of an MFMA step in packed half arithmetic.  `wsh` holds two nibble pairs
// (bits 0-7 and 16-23).  or-ing a nibble into the mantissa of 1024.0 gives 1024 + q exactly, subtracting 1024
// gives q exactly, and half(q * s + b) is one fused multiply-add per pair.  The four results belong to the
// nibbles {a, a+4, a+1, a+5} of the word (a = 0 or 2), which is the order the X chunk is staged in.
SL_DEV mf_h4 dequant4(uint32_t wsh, mf_h2 s2, mf_h2 b2) {
  const mf_h2 k1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
  const mf_h2 q0 = __builtin_bit_cast(mf_h2, (wsh & 0x000F000Fu) | 0x64006400u) - k1024;
  const mf_h2 q1 = __builtin_bit_cast(mf_h2, ((wsh >> 4) & 0x000F000Fu) | 0x64006400u) - k1024;
  const mf_h2 w0 = __builtin_elementwise_fma(q0, s2, b2), w1 = __builtin_elementwise_fma(q1, s2, b2);
  mf_h4 r;
  r[0] = w0[0]; r[1] = w0[1]; r[2] = w1[0]; r[3] = w1[1];
  return r;
}
// The 8 halves of a staged 16-byte piece (k = 8j .. 8j+7) in the order {0,4,1,5, 2,6,3,7}: positions 0-3 are read
// by the lanes of the lower half-wave, 4-7 by the upper, matching dequant4.
SL_DEV uint4 permute8(uint4 v) {
  return make_uint4((v.x & 0xffffu) | (v.z << 16), (v.x >> 16) | (v.z & 0xffff0000u),
                    (v.y & 0xffffu) | (v.w << 16), (v.y >> 16) | (v.w & 0xffff0000u));
}

struct QmmArgs {
  const uint16_t* x;     // [M, x_stride] fp16
  int x_stride;
  const uint32_t* W;     // [N, K/8] packed
  const uint32_t* SB;    // [N, K/64] {scale, bias}
  int M, N, K;           // N % 32 == 0, K % 64 == 0, M <= 128
  uint16_t* y;           // [M, y_stride] fp16
  int y_stride;
};

constexpr int QMM_XS = 72;   // halves per staged X row: 64 + 8 pad (rows 144 bytes apart spread over the LDS banks)

// WM = number of 32-row tiles of X, spread over the waves of a workgroup: wave = (strip of the workgroup, row
// tile), 4 / WM strips per workgroup.  Every wave holds one 32x32 accumulator; the waves of a strip read the same
// weights (from cache) and dequantise them again, which costs less than the latency of a lone wave per SIMD.
template <int WM>
__global__ __launch_bounds__(256) void k_qmm4_mfma(QmmArgs a) {
  __shared__ __align__(16) uint16_t xs[2][WM * 32 * QMM_XS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, hh = lane >> 5;
  const int mt = wave % WM;
  const int n0 = (blockIdx.x * (4 / WM) + wave / WM) * 32;
  const bool live = n0 < a.N && mt * 32 < a.M;          // a workgroup's last waves may have no strip or no rows
  const size_t wrow = (size_t)(n0 < a.N ? n0 + col : 0);
  const int chunks = a.K / 64;
  mf_f16v acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;

  // X chunks travel global -> registers -> LDS one iteration apart, so that no iteration waits for a load it
  // has just issued: 32*WM rows x 128 bytes, one 16-byte piece per thread and pass; rows beyond M are zero
  uint4 xr[WM];
  auto fetch = [&](int c) {
#pragma unroll
    for (int p = 0; p < WM; ++p) {
      const int row = p * 32 + (tid >> 3);
      xr[p] = make_uint4(0, 0, 0, 0);
      if (row < a.M) xr[p] = ld16(a.x + (size_t)row * a.x_stride + c * 64 + (tid & 7) * 8);
    }
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int p = 0; p < WM; ++p) st16(&xs[buf][(p * 32 + (tid >> 3)) * QMM_XS + (tid & 7) * 8], permute8(xr[p]));
  };
  fetch(0);
  put(0);
  if (chunks > 1) fetch(1);
  // the weights of chunk c+1 are requested before chunk c is consumed
  uint4 nw0 = make_uint4(0, 0, 0, 0), nw1 = make_uint4(0, 0, 0, 0);
  uint32_t nsb = 0;
  if (live) { nw0 = ld16(a.W + wrow * (a.K / 8)); nw1 = ld16(a.W + wrow * (a.K / 8) + 4); nsb = a.SB[wrow * (a.K / 64)]; }
  for (int c = 0; c < chunks; ++c) {
    const int buf = c & 1;
    const uint4 w0 = nw0, w1 = nw1;
    const uint32_t sb = nsb;
    if (live && c + 1 < chunks) {
      nw0 = ld16(a.W + wrow * (a.K / 8) + (c + 1) * 8);
      nw1 = ld16(a.W + wrow * (a.K / 8) + (c + 1) * 8 + 4);
      nsb = a.SB[wrow * (a.K / 64) + c + 1];
    }
    __syncthreads();                                     // chunk c is staged; chunk c-1 is no longer read
    if (c + 1 < chunks) { put(buf ^ 1); if (c + 2 < chunks) fetch(c + 2); }
    if (!live) continue;
    const mf_h2 s2 = __builtin_bit_cast(mf_h2, (sb & 0xffffu) * 0x10001u), b2 = __builtin_bit_cast(mf_h2, (sb >> 16) * 0x10001u);
    const uint32_t words[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
    for (int st = 0; st < 8; ++st) {
      // this lane's 4 weights of the step: nibbles {a, a+4, a+1, a+5} of word st with a = 2*hh
      const mf_h4 bw = dequant4(words[st] >> (8 * hh), s2, b2);
      const mf_h4 ax = *reinterpret_cast<const mf_h4*>(&xs[buf][(mt * 32 + col) * QMM_XS + 8 * st + 4 * hh]);
      acc = __builtin_amdgcn_mfma_f32_32x32x8f16(ax, bw, acc, 0, 0, 0);
    }
  }
  if (!live) return;
  // D layout of the 32x32 tile: register r of lane (col, hh) holds row 8*(r/4) + 4*hh + r%4, column col
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int m = mt * 32 + 8 * (r >> 2) + 4 * hh + (r & 3);
    if (m < a.M) a.y[(size_t)m * a.y_stride + n0 + col] = f2h(acc[r]);
  }
}

// -------------------------------------------------------------------------------------------------
// Routed experts of a prefill chunk, grouped by expert (reference: steelMoEGather,
// SeedlessFusedVerify.swift:4174): the (row, slot) pairs that chose expert e are gathered, multiplied with that
// expert's matrix once, and scattered back by pair.  Workgroup = (strip block, expert); experts nobody chose exit.
// -------------------------------------------------------------------------------------------------
constexpr int GROUP_CAP = 512;          // pairs per expert: an expert is chosen at most once per row, M <= 512

struct QmmGroupArgs {
  const uint16_t* x;     // source rows, fp16
  int x_stride;
  int x_by_pair;         // 0: source row = token row (pair >> 3); 1: source row = pair index (m * 8 + slot)
  const uint32_t* W;     // [E * NE, K/8]: expert e owns rows e*NE .. e*NE + NE - 1
  const uint32_t* SB;    // [E * NE, K/64]
  int NE, K;
  const uint16_t* lists; // [E, GROUP_CAP] pair indices
  const int32_t* counts; // [E]
  uint16_t* y;           // [pairs, y_stride]
  int y_stride;
};

__global__ __launch_bounds__(256) void k_qmm4_mfma_grouped(QmmGroupArgs a) {
  // One 32-row tile per pass and one accumulator per wave (most experts have fewer than 32 rows in a chunk; an
  // expert with more takes several passes over its weights, which then come from cache).
  __shared__ __align__(16) uint16_t xs[2][32 * QMM_XS];
  const int e = blockIdx.y;
  const int cnt_all = min(a.counts[e], GROUP_CAP);
  if (cnt_all == 0) return;                              // uniform for the workgroup
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, hh = lane >> 5;
  const int n0 = (blockIdx.x * 4 + wave) * 32;
  const bool live = n0 < a.NE;
  const size_t wrow = (size_t)e * a.NE + (live ? n0 + col : 0);
  const int chunks = a.K / 64;
  for (int r0 = 0; r0 < cnt_all; r0 += 32) {
    const int cnt = min(cnt_all - r0, 32);
    const uint16_t* list = a.lists + (size_t)e * GROUP_CAP + r0;
    // the row this thread stages
    int src = -1;
    if ((tid >> 3) < cnt) { const int pr = list[tid >> 3]; src = a.x_by_pair ? pr : (pr >> 3); }
    mf_f16v acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    uint4 xr = make_uint4(0, 0, 0, 0);
    auto fetch = [&](int c) {
      xr = make_uint4(0, 0, 0, 0);
      if (src >= 0) xr = ld16(a.x + (size_t)src * a.x_stride + c * 64 + (tid & 7) * 8);
    };
    auto put = [&](int buf) { st16(&xs[buf][(tid >> 3) * QMM_XS + (tid & 7) * 8], permute8(xr)); };
    __syncthreads();                                     // the pass before has finished reading the staging buffers
    fetch(0);
    put(0);
    if (chunks > 1) fetch(1);
    uint4 nw0 = make_uint4(0, 0, 0, 0), nw1 = make_uint4(0, 0, 0, 0);
    uint32_t nsb = 0;
    if (live) { nw0 = ld16(a.W + wrow * (a.K / 8)); nw1 = ld16(a.W + wrow * (a.K / 8) + 4); nsb = a.SB[wrow * (a.K / 64)]; }
    for (int c = 0; c < chunks; ++c) {
      const int buf = c & 1;
      const uint4 w0 = nw0, w1 = nw1;
      const uint32_t sb = nsb;
      if (live && c + 1 < chunks) {
        nw0 = ld16(a.W + wrow * (a.K / 8) + (c + 1) * 8);
        nw1 = ld16(a.W + wrow * (a.K / 8) + (c + 1) * 8 + 4);
        nsb = a.SB[wrow * (a.K / 64) + c + 1];
      }
      __syncthreads();
      if (c + 1 < chunks) { put(buf ^ 1); if (c + 2 < chunks) fetch(c + 2); }
      const mf_h2 s2 = __builtin_bit_cast(mf_h2, (sb & 0xffffu) * 0x10001u), b2 = __builtin_bit_cast(mf_h2, (sb >> 16) * 0x10001u);
      const uint32_t words[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
      for (int st = 0; st < 8; ++st) {
        const mf_h4 bw = dequant4(words[st] >> (8 * hh), s2, b2);
        const mf_h4 ax = *reinterpret_cast<const mf_h4*>(&xs[buf][col * QMM_XS + 8 * st + 4 * hh]);
        acc = __builtin_amdgcn_mfma_f32_32x32x8f16(ax, bw, acc, 0, 0, 0);
      }
    }
    if (live) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = 8 * (r >> 2) + 4 * hh + (r & 3);
        if (row < cnt) a.y[(size_t)list[row] * a.y_stride + n0 + col] = f2h(acc[r]);
      }
    }
  }
}

// Pairs (row, slot) listed per expert (M * 8 <= 4096 pairs over 1024 threads), places handed out by LDS counters.
// The order within a list varies from run to run; results do not depend on it (they are scattered back by pair).
__global__ __launch_bounds__(1024) void k_group_pairs(const int32_t* __restrict__ inds, int M, int E, uint16_t* __restrict__ lists,
                                                      int32_t* __restrict__ counts) {
  __shared__ int s_cnt[SL_MAX_EXPERTS];
  if (threadIdx.x < SL_MAX_EXPERTS) s_cnt[threadIdx.x] = 0;
  __syncthreads();
  for (int p = threadIdx.x; p < M * 8; p += 1024) {
    const int e = inds[p];
    if (e >= 0 && e < E) {
      const int pos = atomicAdd(&s_cnt[e], 1);
      if (pos < GROUP_CAP) lists[e * GROUP_CAP + pos] = (uint16_t)p;
    }
  }
  __syncthreads();
  if ((int)threadIdx.x < E) counts[threadIdx.x] = s_cnt[threadIdx.x];
}
// act = half(silu(g) * u) in half arithmetic, elementwise over [rows, 512] (same rule as the GEMV kernels).
__global__ __launch_bounds__(256) void k_swiglu_rows(const uint16_t* __restrict__ g, const uint16_t* __restrict__ u,
                                                     uint16_t* __restrict__ act, int total) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < total) act[i] = f2h(swiglu16(h2f(g[i]), h2f(u[i])));
}
// out[m, n] = half-precision combine of the 8 routed results in routing order + sigmoid(gate) * shared
// (combine_rows SeedlessFusedVerify.swift:462-470, shared_gate_combine_rows :1051-1109).
__global__ __launch_bounds__(256) void k_moe_combine_rows(const uint16_t* __restrict__ d, const uint16_t* __restrict__ scores,
                                                          const uint16_t* __restrict__ sgate, const uint16_t* __restrict__ sy,
                                                          uint16_t* __restrict__ out) {
  const int m = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x;
  float acc = 0.0f;
#pragma unroll
  for (int k = 0; k < 8; ++k) acc = f16r(acc + f16r(h2f(d[((size_t)m * 8 + k) * H + n]) * h2f(scores[m * 8 + k])));
  const float s = sigmoid16(h2f(sgate[m]));
  out[(size_t)m * H + n] = f2h(f16r(acc + f16r(s * h2f(sy[(size_t)m * H + n]))));
}

// Host-side launch: picks the row-tile count per block of up to 128 rows.
inline void launch_qmm4_mfma(const QmmArgs& all, hipStream_t stream) {
  const int strips = all.N / 32;
  const dim3 block(256);
  for (int r0 = 0; r0 < all.M; r0 += 128) {             // the kernel takes up to 128 rows: longer chunks go in blocks
    QmmArgs a = all;
    a.x = all.x + (size_t)r0 * all.x_stride;
    a.y = all.y + (size_t)r0 * all.y_stride;
    a.M = all.M - r0 < 128 ? all.M - r0 : 128;
    if (a.M <= 32) hipLaunchKernelGGL(k_qmm4_mfma<1>, dim3((unsigned)((strips + 3) / 4)), block, 0, stream, a);
    else if (a.M <= 64) hipLaunchKernelGGL(k_qmm4_mfma<2>, dim3((unsigned)((strips + 1) / 2)), block, 0, stream, a);
    else hipLaunchKernelGGL(k_qmm4_mfma<4>, dim3((unsigned)strips), block, 0, stream, a);
  }
}

}  // namespace sl
