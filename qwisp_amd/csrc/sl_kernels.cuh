// Decode kernels for the Seedless engine on gfx950 (wave64).  Row m of an M-row forward is
// blockIdx.y (or .z); every per-row computation is independent of M, which is what makes an
// M-row verify step equal M single-row steps bit for bit.
//
// Reduction order shared by all kernels (and by the CPU checker used in the tests):
//  * 4-bit dot, K = 2048*NBLK: lane l owns the share of 32 elements (words 4l..4l+3, one 16-byte load) of each
//    2048-element block, share term T = fmaf(s, A + B, b*sx) (share_term in sl_device.cuh), lane partial = sum of
//    its terms block after block, then a 64-lane butterfly.  K = 512: the same with 16 lanes per row, four rows per wave.
//  * dense fp16 dot over 2048: lane l owns elements 32l..32l+31, fmaf chain, butterfly.
//  * sum of squares over D = 128, 256 or 2048: pair terms fmaf(x1, x1, x0*x0), balanced tree over the D/2 of them.
#pragma once
#include "sl_device.cuh"
#include "../../include/seedless_hip.h"

namespace sl {

constexpr int H = SL_H;
constexpr float EPS = 1e-6f;
constexpr int PROJ_STRIDE = SL_GDN_IN_N;     // row stride of the projection scratch (>= 9216)
constexpr int SDPA_TILE = 64;
constexpr int KT_STRIDE = 264;               // halves per staged key row (256 + 8 pad)

// -------------------------------------------------------------------------------------------------
// Hidden-row prologue: x = half(h + r) (optional), optional rmsnorm with weight w.
// Reference: resid_add + rmsnorm fused as gdn_resid_postnorm_rows, SeedlessFusedVerify.swift:943-1001.
// -------------------------------------------------------------------------------------------------
SL_DEV void load32(const uint16_t* p, float* x) {
#pragma unroll
  for (int j = 0; j < 4; ++j) unpack8(ld16(p + 8 * j), x + 8 * j);
}
SL_DEV void store32(uint16_t* p, const float* x) {
#pragma unroll
  for (int j = 0; j < 4; ++j) st16(p + 8 * j, pack8(x + 8 * j));
}
SL_DEV float inv_rms_2048(const float* x) {
  const float ss = tree_sum<64>(share_sumsq(x));
  return 1.0f / sqrtf(ss / 2048.0f + EPS);
}
struct HiddenArgs {
  const uint16_t* h_in;    // [M, 2048]
  const uint16_t* r_in;    // [M, 2048] residual to add first, or null
  const uint16_t* lnw;     // [2048] norm weight, or null for "x is used as given"
  uint16_t* h_out;         // [M, 2048] receives half(h + r) (written once per row), or null
  uint16_t* xn_out;        // [M, 2048] receives the normed row (written once per row), or null
  float* xs_out;           // [M, 64] receives the sums of the row's 64 shares of 32 elements (share_sum), or null
};
// Every wave of the grid calls this; `writer` selects the single wave that stores the outputs.
SL_DEV void hidden_prologue(const HiddenArgs& a, int m, int lane, bool writer, float* x) {
  load32(a.h_in + (size_t)m * H + 32 * lane, x);
  if (a.r_in) {
    float r[32];
    load32(a.r_in + (size_t)m * H + 32 * lane, r);
#pragma unroll
    for (int i = 0; i < 32; ++i) x[i] = f16r(x[i] + r[i]);
  }
  if (writer && a.h_out) store32(a.h_out + (size_t)m * H + 32 * lane, x);
  if (a.lnw) {
    const float inv = inv_rms_2048(x);
    float w[32];
    load32(a.lnw + 32 * lane, w);
#pragma unroll
    for (int i = 0; i < 32; ++i) x[i] = f16r(w[i] * f16r(x[i] * inv));
  }
  if (writer && a.xn_out) store32(a.xn_out + (size_t)m * H + 32 * lane, x);
  if (writer && a.xs_out) a.xs_out[(size_t)m * 64 + lane] = share_sum(x);   // the dots of the row's consumers need these sums: formed once here
}

// -------------------------------------------------------------------------------------------------
// 4-bit dots.  W: packed words [rows, K/8]; SB: {scale, bias} half pairs [rows, K/64].
// Reference arithmetic: qmm4, SeedlessMetalForward.swift:238-310.
// -------------------------------------------------------------------------------------------------
template <int NBLK, int R>
SL_DEV void qdot_rows(const uint32_t* __restrict__ W, const uint32_t* __restrict__ SB, const size_t* rows, int lane,
                      const uint32_t* xp, const float* sx, float* out) {
  constexpr int WPR = NBLK * 256, GPR = NBLK * 32;
  uint4 wv[R][NBLK];
  uint32_t sb[R][NBLK];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int b = 0; b < NBLK; ++b) {
      wv[r][b] = ld16(W + rows[r] * WPR + b * 256 + 4 * lane);
      sb[r][b] = SB[rows[r] * GPR + b * 32 + (lane >> 1)];
    }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    float acc = share_term(wv[r][0], sb[r][0], xp, sx[0]);
#pragma unroll
    for (int b = 1; b < NBLK; ++b) acc = acc + share_term(wv[r][b], sb[r][b], xp + 16 * b, sx[b]);
    out[r] = tree_sum<64>(acc);
  }
}
// K = 512: 16 lanes per row; li = lane & 15 owns words 4li..4li+3.  Result valid on all 16 lanes.
SL_DEV float qdot512(const uint32_t* __restrict__ W, const uint32_t* __restrict__ SB, size_t row, int li,
                     const uint32_t* xp, float sx) {
  const uint4 wv = ld16(W + row * 64 + 4 * li);
  const uint32_t sb = SB[row * 8 + (li >> 1)];
  return tree_sum<16>(share_term(wv, sb, xp, sx));
}
// Dense fp16 row against the lane's 32 activations (router gate, shared-expert gate).
SL_DEV float dense_dot(const uint16_t* __restrict__ wrow, int lane, const float* x) {
  float w[32];
  load32(wrow + 32 * lane, w);
  float acc = 0.0f;
#pragma unroll
  for (int i = 0; i < 32; ++i) acc = fmaf(x[i], w[i], acc);
  return tree_sum<64>(acc);
}

// -------------------------------------------------------------------------------------------------
// embed_rows_q4 (SeedlessFusedVerify.swift:556-570): h = half(half(s*nib) + b).
// -------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_embed(const int32_t* __restrict__ tokens, const uint32_t* __restrict__ W,
                                               const uint32_t* __restrict__ SB, uint16_t* __restrict__ h) {
  const int m = blockIdx.y, j = blockIdx.x * 256 + threadIdx.x;
  const size_t tok = (size_t)tokens[m];
  const uint32_t w = W[tok * 256 + (j >> 3)];
  const uint32_t sb = SB[tok * 32 + (j >> 6)];
  const float nib = (float)((w >> (4 * (j & 7))) & 15u);
  h[(size_t)m * H + j] = f2h(f16r(lo_h(sb) * nib) + hi_h(sb));
}

// -------------------------------------------------------------------------------------------------
// Projection with the hidden prologue: y[m, n] = half(dot(x_m, W[n])), K = 2048.
// Used for the GDN in-proj (qkv|z|b|a concatenated, SeedlessFusedVerify.swift:690) and the
// attention q|k|v projection.  4 waves x R rows per workgroup.
// -------------------------------------------------------------------------------------------------
template <int R>
__global__ __launch_bounds__(256) void k_qmv_hidden(HiddenArgs ha, const uint32_t* __restrict__ W,
                                                    const uint32_t* __restrict__ SB, int N, uint16_t* __restrict__ y,
                                                    int y_stride) {
  const int m = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float x[32], sx[1];
  hidden_prologue(ha, m, lane, blockIdx.x == 0 && wave == 0, x);
  sx[0] = share_sum(x);
  uint32_t xp[16];
  pack_x(x, xp);
  const size_t row0 = ((size_t)blockIdx.x * 4 + wave) * R;
  if (row0 >= (size_t)N) return;
  size_t rows[R];
#pragma unroll
  for (int r = 0; r < R; ++r) rows[r] = row0 + r;
  float out[R];
  qdot_rows<1, R>(W, SB, rows, lane, xp, sx, out);
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) y[(size_t)m * y_stride + row0 + r] = f2h(out[r]);
  }
}

// Plain projection from an fp16 activation buffer, K = 2048*NBLK (attention o_proj: NBLK = 2).
template <int NBLK, int R>
__global__ __launch_bounds__(256) void k_qmv_plain(const uint16_t* __restrict__ xin, int x_stride,
                                                   const uint32_t* __restrict__ W, const uint32_t* __restrict__ SB,
                                                   int N, uint16_t* __restrict__ y, int y_stride) {
  const int m = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float sx[NBLK];
  uint32_t xp[16 * NBLK];
#pragma unroll
  for (int b = 0; b < NBLK; ++b) {
    float x[32];
    load32(xin + (size_t)m * x_stride + b * 2048 + 32 * lane, x);
    sx[b] = share_sum(x);
    pack_x(x, xp + 16 * b);
  }
  const size_t row0 = ((size_t)blockIdx.x * 4 + wave) * R;
  if (row0 >= (size_t)N) return;
  size_t rows[R];
#pragma unroll
  for (int r = 0; r < R; ++r) rows[r] = row0 + r;
  float out[R];
  qdot_rows<NBLK, R>(W, SB, rows, lane, xp, sx, out);
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) y[(size_t)m * y_stride + row0 + r] = f2h(out[r]);
  }
}

// -------------------------------------------------------------------------------------------------
// The same projections for a tile of MT activation rows at a time (verify rows, lane batches, exact prefill
// chunks): a wave fetches and masks its R weight rows once and runs every activation row of the tile against
// them, so the weight stream and the nibble unpacking are shared; per activation row the arithmetic is that of
// k_qmv_hidden / k_qmv_plain.  The tile's activation rows are prepared once per workgroup (residual, norm,
// packing: wave w takes rows w, w + waves, ...) and parked in LDS, 20 words per lane (16 packed pairs, the share's
// sum and three words of padding) so that a lane reads back its own 80 bytes with five 16-byte reads free of bank
// conflicts.
// HIDDEN: x comes from the hidden prologue (K = 2048; steps of up to four rows, where a wave preparing one row in
// every workgroup costs less than a launch that prepares the rows once); otherwise from the fp16 buffer xin
// (K = 2048*NBLK).  Grid (G, ceil(M / MT)), four waves (three workgroups share a compute unit).  G workgroups cover G*waves*R rows; rows beyond that (fewer than G) are taken one each by wave 0 of the
// first workgroups, so that G can be chosen to fill the machine exactly once (12352 rows: 768 workgroups of 16
// rows + 64 single rows, instead of 772 workgroups on 768 places).
// -------------------------------------------------------------------------------------------------
// ARGMAX (lm_head, R = 4, 4 waves): y is the logits matrix and every workgroup also leaves one (value, index)
// candidate per activation row, the first maximum of its 16 rounded logits, for k_argmax_final.
template <int NBLK, int R, int MT, bool HIDDEN, bool ARGMAX = false>
__global__ __launch_bounds__(256, 3) void k_qmv_tile(HiddenArgs ha, const uint16_t* __restrict__ xin, int x_stride,
                                                  const uint32_t* __restrict__ W, const uint32_t* __restrict__ SB,
                                                  int N, uint16_t* __restrict__ y, int y_stride, int M,
                                                  float* __restrict__ cand_v = nullptr, int32_t* __restrict__ cand_i = nullptr,
                                                  const float* __restrict__ xsums = nullptr) {
  static_assert(!HIDDEN || NBLK == 1, "the hidden row is one block of 2048");
  static_assert(!ARGMAX || R == 4, "candidates are formed over four rows per wave");
  constexpr int WPR = NBLK * 256, GPR = NBLK * 32;
  __shared__ uint4 xs[MT * NBLK * 64 * 5];
  __shared__ float s_v[ARGMAX ? MT * 8 : 1];
  __shared__ int s_i[ARGMAX ? MT * 8 : 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  const int m0 = blockIdx.y * MT, mc = min(MT, M - m0);
  const size_t row0 = ((size_t)blockIdx.x * waves + wave) * R;
  const bool live = row0 < (size_t)N;
  // weights first: their latency hides behind the preparation of the activation rows
  uint4 wv[R][NBLK];
  uint32_t sb[R][NBLK];
  if (live) {
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int b = 0; b < NBLK; ++b) {
        wv[r][b] = ld16(W + (row0 + r) * WPR + b * 256 + 4 * lane);
        sb[r][b] = SB[(row0 + r) * GPR + b * 32 + (lane >> 1)];
      }
  }
  const size_t xrow = (size_t)gridDim.x * waves * R + blockIdx.x;      // this workgroup's single row beyond the grid's cover
  const bool extra = !ARGMAX && wave == 0 && xrow < (size_t)N;
  for (int m = wave; m < mc; m += waves) {
#pragma unroll
    for (int b = 0; b < NBLK; ++b) {
      uint4* dst = xs + ((m * NBLK + b) * 64 + lane) * 5;
      if (!HIDDEN && xsums) {                              // the stored halves are the packed pairs; their sums came with the row
        const uint16_t* src = xin + (size_t)(m0 + m) * x_stride + b * 2048 + 32 * lane;
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[j] = ld16(src + 8 * j);
        dst[4] = make_uint4(__float_as_uint(xsums[(size_t)(m0 + m) * (64 * NBLK) + b * 64 + lane]), 0u, 0u, 0u);
        continue;
      }
      float x[32];
      if constexpr (HIDDEN) hidden_prologue(ha, m0 + m, lane, blockIdx.x == 0, x);
      else load32(xin + (size_t)(m0 + m) * x_stride + b * 2048 + 32 * lane, x);
      const float sx = share_sum(x);
      uint32_t xp[16];
      pack_x(x, xp);
#pragma unroll
      for (int j = 0; j < 4; ++j) dst[j] = make_uint4(xp[4 * j], xp[4 * j + 1], xp[4 * j + 2], xp[4 * j + 3]);
      dst[4] = make_uint4(__float_as_uint(sx), 0u, 0u, 0u);
    }
  }
  __syncthreads();
  if (!live) {
    if constexpr (ARGMAX) {
      if (lane == 0) for (int m = 0; m < mc; ++m) { s_v[m * 8 + wave] = -__int_as_float(0x7f800000); s_i[m * 8 + wave] = 0x7fffffff; }
      __syncthreads();
    }
    return;
  }
  h2_t mk[R][NBLK][16];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int b = 0; b < NBLK; ++b) {
      word_masks(wv[r][b].x, mk[r][b]); word_masks(wv[r][b].y, mk[r][b] + 4);
      word_masks(wv[r][b].z, mk[r][b] + 8); word_masks(wv[r][b].w, mk[r][b] + 12);
    }
  for (int m = 0; m < mc; ++m) {
    float acc[R];
#pragma unroll
    for (int b = 0; b < NBLK; ++b) {
      const uint4* src = xs + ((m * NBLK + b) * 64 + lane) * 5;
      uint32_t xp[16];
#pragma unroll
      for (int j = 0; j < 4; ++j) { const uint4 v = src[j]; xp[4 * j] = v.x; xp[4 * j + 1] = v.y; xp[4 * j + 2] = v.z; xp[4 * j + 3] = v.w; }
      const float sx = __uint_as_float(reinterpret_cast<const uint32_t*>(src + 4)[0]);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const float t = share_term_masked(mk[r][b], sb[r][b], xp, sx);
        acc[r] = (b == 0) ? t : acc[r] + t;
      }
    }
    float out[R];
    if constexpr (R == 4) {                              // the four sums in one register, then handed round the quad
      float o4[4];
      quad_values(tree_sum4(acc[0], acc[1], acc[2], acc[3], lane), o4);
#pragma unroll
      for (int r = 0; r < 4; ++r) out[r] = o4[r];
    } else {
#pragma unroll
      for (int r = 0; r < R; ++r) out[r] = tree_sum<64>(acc[r]);
    }
    if constexpr (ARGMAX) {
      if (lane == 0) {
        float bv = -__int_as_float(0x7f800000);
        int bi = 0x7fffffff;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float v = f16r(out[r]);
          if (v > bv) { bv = v; bi = (int)(row0 + r); }
        }
        s_v[m * 8 + wave] = bv; s_i[m * 8 + wave] = bi;
        *reinterpret_cast<uint2*>(y + (size_t)(m0 + m) * y_stride + row0) = make_uint2(pack2(out[0], out[1]), pack2(out[2], out[3]));
      }
    } else if (lane == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r) y[(size_t)(m0 + m) * y_stride + row0 + r] = f2h(out[r]);
    }
  }
  if (extra) {
    uint4 wx[NBLK];
    uint32_t sbx[NBLK];
#pragma unroll
    for (int b = 0; b < NBLK; ++b) { wx[b] = ld16(W + xrow * WPR + b * 256 + 4 * lane); sbx[b] = SB[xrow * GPR + b * 32 + (lane >> 1)]; }
    h2_t mx[NBLK][16];
#pragma unroll
    for (int b = 0; b < NBLK; ++b) {
      word_masks(wx[b].x, mx[b]); word_masks(wx[b].y, mx[b] + 4); word_masks(wx[b].z, mx[b] + 8); word_masks(wx[b].w, mx[b] + 12);
    }
    for (int m = 0; m < mc; ++m) {
      float acc = 0.0f;
#pragma unroll
      for (int b = 0; b < NBLK; ++b) {
        const uint4* src = xs + ((m * NBLK + b) * 64 + lane) * 5;
        uint32_t xp[16];
#pragma unroll
        for (int j = 0; j < 4; ++j) { const uint4 v = src[j]; xp[4 * j] = v.x; xp[4 * j + 1] = v.y; xp[4 * j + 2] = v.z; xp[4 * j + 3] = v.w; }
        const float sx = __uint_as_float(reinterpret_cast<const uint32_t*>(src + 4)[0]);
        const float t = share_term_masked(mx[b], sbx[b], xp, sx);
        acc = (b == 0) ? t : acc + t;
      }
      const float o = tree_sum<64>(acc);
      if (lane == 0) y[(size_t)(m0 + m) * y_stride + xrow] = f2h(o);
    }
  }
  if constexpr (ARGMAX) {
    __syncthreads();
    if ((int)threadIdx.x < mc) {
      const int m = threadIdx.x;
      float bv = s_v[m * 8];
      int bi = s_i[m * 8];
      for (int w = 1; w < waves; ++w) if (s_v[m * 8 + w] > bv) { bv = s_v[m * 8 + w]; bi = s_i[m * 8 + w]; }
      cand_v[(size_t)(m0 + m) * gridDim.x + blockIdx.x] = bv;
      cand_i[(size_t)(m0 + m) * gridDim.x + blockIdx.x] = bi;
    }
  }
}

// -------------------------------------------------------------------------------------------------
// Gated-DeltaNet core: causal conv(4)+SiLU+history shift, q/k head norms and scales, beta and
// decay, and the gated delta rule with the fp32 state in registers, M rows in sequence.
// References: conv_shift_fused_rows SeedlessFusedVerify.swift:634-663; gdn_prep_rows :839-938;
// gated_delta_step GatedDelta.swift:63-124.
// Grid: 32 value heads x 8 slices of 16 state rows; 4 waves, each wave 2 x 2 rows, a row = 32
// lanes x 4 contiguous dk.  State layout [hv][dv][dk] fp32, ping-pong selected by st[1].
// -------------------------------------------------------------------------------------------------
// One sequence ("lane") of a lane-batched step as one layer's kernels see it: row b of the batch belongs to
// lanes[b], which brings its own caches and its own step state (st[0] = position, st[1 + layer] = parity).
struct LaneRef {
  uint16_t* hist[2];         // Gated-DeltaNet layers
  float* state[2];
  uint16_t *kcache, *vcache; // attention layers
  int32_t* st;
  int max_seq, pad;
};

struct GdnArgs {
  const uint16_t* proj;      // [M, PROJ_STRIDE]: qkv 8192 | z 4096 | b 32 | a 32
  const float* conv_w;       // [8192, 4]
  const float* a_log;        // [32]
  const float* dt_bias;      // [32]
  uint16_t* hist[2];         // [3, 8192] each
  float* state[2];           // [32, 128, 128] each
  const int32_t* st;         // st[1] = parity: read side
  uint16_t* ycore;           // [M, 4096]
  int M;
  const LaneRef* lanes;      // lane batch: blockIdx.y = lane, one row each, caches and parity of that lane
  int layer;
};
SL_DEV float conv_tap(const uint16_t* proj, const uint16_t* hin, int row, int ch) {
  // row of the concatenation [hist(3) | qkv(M)]
  return (row < 3) ? h2f(hin[row * SL_CONV_DIM + ch]) : h2f(proj[(size_t)(row - 3) * PROJ_STRIDE + ch]);
}
SL_DEV float conv_silu(const uint16_t* proj, const float* conv_w, const uint16_t* hin, int t, int ch) {
  float acc = 0.0f;
#pragma unroll
  for (int k = 0; k < 4; ++k) acc = fmaf(conv_tap(proj, hin, t + k, ch), conv_w[ch * 4 + k], acc);
  return f16r(acc * sigmoid32(acc));
}
// The ping-pong sides of the conv history and the recurrent state, and the rows a workgroup works on: of the
// engine's own sequence, or (lane batch) of lane blockIdx.y.  Plain selects: the argument struct is never indexed
// with a run-time value nor written, so it stays in scalar registers.
struct GdnView {
  const uint16_t* hin; uint16_t* hout;
  const float* sin_; float* sout;
  const uint16_t* proj; uint16_t* ycore;
  int M;
};
SL_DEV GdnView gdn_view(const GdnArgs& a, int lane_row) {
  GdnView v;
  const uint16_t *h0 = a.hist[0], *h1 = a.hist[1];
  const float *s0 = a.state[0], *s1 = a.state[1];
  const int32_t* st = a.st;
  v.proj = a.proj; v.ycore = a.ycore; v.M = a.M;
  if (a.lanes) {
    const LaneRef& r = a.lanes[lane_row];
    h0 = as_global(r.hist[0]); h1 = as_global(r.hist[1]); s0 = as_global(r.state[0]); s1 = as_global(r.state[1]);
    st = as_global(r.st) + a.layer;
    v.proj += (size_t)lane_row * PROJ_STRIDE; v.ycore += (size_t)lane_row * 4096; v.M = 1;
  }
  const bool par = st[1] != 0;
  v.hin = par ? h1 : h0; v.hout = const_cast<uint16_t*>(par ? h0 : h1);
  v.sin_ = par ? s1 : s0; v.sout = const_cast<float*>(par ? s0 : s1);
  return v;
}
// NIT pairs of value rows per wave: a workgroup owns 8 * NIT value dims of one head (grid.x = 32 heads * 16 / NIT).
// Lane batches use NIT = 4 (half the workgroups, twice the state bytes in flight per workgroup); the arithmetic per
// value row is the same.
template <int NIT>
__global__ __launch_bounds__(256) void k_gdn_core(GdnArgs a) {
  constexpr int DVW = 8 * NIT, NB = 128 / DVW;          // value dims per workgroup, workgroups per head
  __shared__ float s_q[128], s_k[128], s_v[DVW], s_gb[2];
  const GdnView vw = gdn_view(a, blockIdx.y);
  const uint16_t* hin = vw.hin;
  uint16_t* hout = vw.hout;
  const float* sin_ = vw.sin_;
  float* sout = vw.sout;
  const uint16_t* proj = vw.proj;
  uint16_t* ycore = vw.ycore;
  const int M = vw.M;
  const int hv = blockIdx.x / NB, dvb = blockIdx.x % NB, hk = hv >> 1;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;

  float s[NIT][4];
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int dv = dvb * DVW + wave * 2 * NIT + it * 2 + half;
    const float4 v = *reinterpret_cast<const float4*>(sin_ + ((size_t)hv * 128 + dv) * 128 + 4 * l32);
    s[it][0] = v.x; s[it][1] = v.y; s[it][2] = v.z; s[it][3] = v.w;
  }
  const int qk_ch = (tid < 128) ? (hk * 128 + tid) : (2048 + hk * 128 + (tid - 128));
  const int v_ch = 4096 + hv * 128 + dvb * DVW + (tid & (DVW - 1));

  for (int t = 0; t < M; ++t) {
    const float c = conv_silu(proj, a.conv_w, hin, t, qk_ch);
    if (tid < 128) s_q[tid] = c; else s_k[tid - 128] = c;
    if (tid < DVW) s_v[tid] = conv_silu(proj, a.conv_w, hin, t, v_ch);
    __syncthreads();
    if (wave < 2) {
      // weightless rmsnorm over 128, then the key/query scale, both rounded to half
      float* buf = wave ? s_k : s_q;
      const float x0 = buf[2 * lane], x1 = buf[2 * lane + 1];
      float ss = fmaf(x1, x1, fmaf(x0, x0, 0.0f));
      ss = tree_sum<64>(ss);
      const float inv = 1.0f / sqrtf(ss / 128.0f + EPS);
      const float sc = wave ? f16r(0.08838834764831845f) : f16r(0.0078125f);
      const float y0 = f16r(sc * f16r(x0 * inv)), y1 = f16r(sc * f16r(x1 * inv));
      buf[2 * lane] = y0; buf[2 * lane + 1] = y1;
    } else if (tid == 128) {
      const float bP = h2f(proj[(size_t)t * PROJ_STRIDE + 12288 + hv]);
      const float aP = h2f(proj[(size_t)t * PROJ_STRIDE + 12320 + hv]);
      s_gb[0] = exp_c(-(exp_c(a.a_log[hv]) * softplus_c(aP + a.dt_bias[hv])));
      s_gb[1] = sigmoid16(bP);
    }
    __syncthreads();
    const float g = s_gb[0], beta = s_gb[1];
    const float4 k4 = *reinterpret_cast<const float4*>(&s_k[4 * l32]);
    const float4 q4 = *reinterpret_cast<const float4*>(&s_q[4 * l32]);
    const float kk[4] = {k4.x, k4.y, k4.z, k4.w}, qq[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int dvl = wave * 2 * NIT + it * 2 + half;
      float acc = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; ++i) { s[it][i] = s[it][i] * g; acc = fmaf(s[it][i], kk[i], acc); }
      const float kv = tree_sum<32>(acc);
      const float delta = (s_v[dvl] - kv) * beta;
      acc = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; ++i) { s[it][i] = fmaf(kk[i], delta, s[it][i]); acc = fmaf(s[it][i], qq[i], acc); }
      const float y = tree_sum<32>(acc);
      if (l32 == 0) ycore[(size_t)t * 4096 + hv * 128 + dvb * DVW + dvl] = f2h(y);
    }
    __syncthreads();
  }
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int dv = dvb * DVW + wave * 2 * NIT + it * 2 + half;
    *reinterpret_cast<float4*>(sout + ((size_t)hv * 128 + dv) * 128 + 4 * l32) = make_float4(s[it][0], s[it][1], s[it][2], s[it][3]);
  }
  // history shift: rows M..M+2 of [hist | qkv]; each channel written by exactly one workgroup
  if ((hv & 1) == 0 && dvb == 0) {
#pragma unroll
    for (int j = 0; j < 3; ++j) hout[j * SL_CONV_DIM + qk_ch] = f2h(conv_tap(proj, hin, M + j, qk_ch));
  }
  if (tid < DVW) {
#pragma unroll
    for (int j = 0; j < 3; ++j) hout[j * SL_CONV_DIM + v_ch] = f2h(conv_tap(proj, hin, M + j, v_ch));
  }
}

// -------------------------------------------------------------------------------------------------
// The same layer for M >= 2 rows in two kernels with the same arithmetic.  Everything that does not depend on the
// recurrent state (conv + silu, q/k norms, decay and beta) is formed for all rows at once (k_gdn_prep_rows);
// the recurrence itself then streams through the rows without a barrier (k_gdn_scan_rows), the next row's inputs
// being requested while the current row is worked on.
// -------------------------------------------------------------------------------------------------
struct GdnPrepArgs {
  GdnArgs g;                 // proj, conv_w, a_log, dt_bias, hist, st, M as above
  uint16_t *qn, *kn;         // [M, 2048] normed, scaled query / key (half values)
  uint16_t* vc;              // [M, 4096] conv + silu of the value channels
  float* gb;                 // [M, 64]: decay g of the 32 value heads, then beta
};
// One wave per (unit, block of PR rows): units 0..15 query heads, 16..31 key heads, 32..63 value heads,
// 64 decay / beta.  A wave walks its rows with the conv window in registers (a row's four taps are the three rows
// before it and itself: every row of the projection is loaded once, all loads of the block up front), which also
// keeps the number of waves of a 2048-row chunk at 8320 instead of one per row and unit.  The arithmetic per row is
// that of conv_silu.
// PR = 16 for long chunks; steps of fewer rows take PR = 4, so that a step of 17 rows is 325 waves and not 130 waves
// of up to 16 rows in sequence.
template <int PR>
__global__ __launch_bounds__(64) void k_gdn_prep_rows(GdnPrepArgs p) {
  const GdnArgs& a = p.g;
  const int u = blockIdx.x, t0 = blockIdx.y * PR, lane = threadIdx.x;
  const int rows = min(PR, a.M - t0);
  const uint16_t* hin = a.st[1] ? a.hist[1] : a.hist[0];
  if (u < 64) {
    const bool isq = u < 16, isk = u >= 16 && u < 32;
    const int ch = u < 32 ? (isk ? 2048 : 0) + (u & 15) * 128 + 2 * lane : 4096 + (u - 32) * 128 + 2 * lane;
    // rows t0 .. t0 + rows + 2 of the concatenation [hist(3) | qkv(M)], two neighbouring channels per lane
    uint32_t win[PR + 3];
#pragma unroll
    for (int j = 0; j < PR + 3; ++j) {
      const int row = min(t0 + j, t0 + rows + 2);
      win[j] = (row < 3) ? *reinterpret_cast<const uint32_t*>(hin + row * SL_CONV_DIM + ch)
                         : *reinterpret_cast<const uint32_t*>(a.proj + (size_t)(row - 3) * PROJ_STRIDE + ch);
    }
    float w0[4], w1[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) { w0[k] = a.conv_w[ch * 4 + k]; w1[k] = a.conv_w[(ch + 1) * 4 + k]; }
    const float sc = isk ? f16r(0.08838834764831845f) : f16r(0.0078125f);
#pragma unroll
    for (int j = 0; j < PR; ++j) {
      if (j >= rows) continue;                  // (uniform; a break would keep the loop from unrolling)
      const int t = t0 + j;
      float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
      for (int k = 0; k < 4; ++k) { a0 = fmaf(lo_h(win[j + k]), w0[k], a0); a1 = fmaf(hi_h(win[j + k]), w1[k], a1); }
      const float x0 = f16r(a0 * sigmoid32(a0)), x1 = f16r(a1 * sigmoid32(a1));
      if (isq || isk) {
        float ss = fmaf(x1, x1, fmaf(x0, x0, 0.0f));
        ss = tree_sum<64>(ss);
        const float inv = 1.0f / sqrtf(ss / 128.0f + EPS);
        const float y0 = f16r(sc * f16r(x0 * inv)), y1 = f16r(sc * f16r(x1 * inv));
        *reinterpret_cast<uint32_t*>((isk ? p.kn : p.qn) + (size_t)t * 2048 + (u & 15) * 128 + 2 * lane) = pack2(y0, y1);
      } else {
        *reinterpret_cast<uint32_t*>(p.vc + (size_t)t * 4096 + (u - 32) * 128 + 2 * lane) = pack2(x0, x1);
      }
    }
  } else {
    const int hv = lane & 31;
    for (int j = 0; j < rows; ++j) {
      const int t = t0 + j;
      if (lane < 32) {
        const float aP = h2f(a.proj[(size_t)t * PROJ_STRIDE + 12320 + hv]);
        p.gb[(size_t)t * 64 + hv] = exp_c(-(exp_c(a.a_log[hv]) * softplus_c(aP + a.dt_bias[hv])));
      } else {
        p.gb[(size_t)t * 64 + 32 + hv] = sigmoid16(h2f(a.proj[(size_t)t * PROJ_STRIDE + 12288 + hv]));
      }
    }
  }
}
// The recurrence over the rows: workgroup = (value head, block of 8 dv), arithmetic of k_gdn_core.  Also shifts the conv history.
__global__ __launch_bounds__(256) void k_gdn_scan_rows(GdnPrepArgs p) {
  const GdnArgs& a = p.g;
  const int hv = blockIdx.x >> 4, dvb = blockIdx.x & 15, hk = hv >> 1;   // 16 slices of 8 state rows per value head
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;
  const bool par = a.st[1] != 0;
  const uint16_t* hin = par ? a.hist[1] : a.hist[0];
  uint16_t* hout = par ? a.hist[0] : a.hist[1];
  const float* sin_ = par ? a.state[1] : a.state[0];
  float* sout = par ? a.state[0] : a.state[1];
  // a wave owns two state rows (one per half-wave): twice the waves of k_gdn_core, because here a wave's step is a
  // chain of dependent instructions and a SIMD with one wave idles between them
  const int dv = dvb * 8 + wave * 2 + half;
  float s[4];
  {
    const float4 v = *reinterpret_cast<const float4*>(sin_ + ((size_t)hv * 128 + dv) * 128 + 4 * l32);
    s[0] = v.x; s[1] = v.y; s[2] = v.z; s[3] = v.w;
  }
  struct Row { uint2 k, q; uint16_t v; float g, beta; };
  auto fetch = [&](int t) {
    Row r;
    r.k = *reinterpret_cast<const uint2*>(p.kn + (size_t)t * 2048 + hk * 128 + 4 * l32);
    r.q = *reinterpret_cast<const uint2*>(p.qn + (size_t)t * 2048 + hk * 128 + 4 * l32);
    r.v = p.vc[(size_t)t * 4096 + hv * 128 + dv];
    r.g = p.gb[(size_t)t * 64 + hv]; r.beta = p.gb[(size_t)t * 64 + 32 + hv];
    return r;
  };
  // the inputs of the next SCAN_AHEAD rows are in flight while a row is worked on (a row's step is far shorter than
  // a trip to memory); the ring is indexed with constants only, so it stays in registers
  constexpr int SCAN_AHEAD = 8;
  Row ring[SCAN_AHEAD];
#pragma unroll
  for (int j = 0; j < SCAN_AHEAD; ++j) if (j < a.M) ring[j] = fetch(j);
  for (int t0 = 0; t0 < a.M; t0 += SCAN_AHEAD) {
#pragma unroll
    for (int j = 0; j < SCAN_AHEAD; ++j) {
      const int t = t0 + j;
      if (t >= a.M) break;
      const Row cur = ring[j];
      if (t + SCAN_AHEAD < a.M) ring[j] = fetch(t + SCAN_AHEAD);
      const float kk[4] = {lo_h(cur.k.x), hi_h(cur.k.x), lo_h(cur.k.y), hi_h(cur.k.y)};
      const float qq[4] = {lo_h(cur.q.x), hi_h(cur.q.x), lo_h(cur.q.y), hi_h(cur.q.y)};
      float acc = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; ++i) { s[i] = s[i] * cur.g; acc = fmaf(s[i], kk[i], acc); }
      const float kv = tree_sum<32>(acc);
      const float delta = (h2f(cur.v) - kv) * cur.beta;
      acc = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; ++i) { s[i] = fmaf(kk[i], delta, s[i]); acc = fmaf(s[i], qq[i], acc); }
      const float y = tree_sum<32>(acc);
      if (l32 == 0) a.ycore[(size_t)t * 4096 + hv * 128 + dv] = f2h(y);
    }
  }
  *reinterpret_cast<float4*>(sout + ((size_t)hv * 128 + dv) * 128 + 4 * l32) = make_float4(s[0], s[1], s[2], s[3]);
  // history shift: rows M..M+2 of [hist | qkv]; each channel written by exactly one workgroup
  const int qk_ch = (tid < 128) ? (hk * 128 + tid) : (2048 + hk * 128 + (tid - 128));
  const int v_ch = 4096 + hv * 128 + dvb * 8 + (tid & 7);
  if ((hv & 1) == 0 && dvb == 0) {
#pragma unroll
    for (int j = 0; j < 3; ++j) hout[j * SL_CONV_DIM + qk_ch] = f2h(conv_tap(a.proj, hin, a.M + j, qk_ch));
  }
  if (tid < 8) {
#pragma unroll
    for (int j = 0; j < 3; ++j) hout[j * SL_CONV_DIM + v_ch] = f2h(conv_tap(a.proj, hin, a.M + j, v_ch));
  }
}

// -------------------------------------------------------------------------------------------------
// GDN out-proj with the gated rmsnorm as prologue: x = half(silu(z) * half(w * half(y*inv))) per value
// head (with an fp32 norm weight: half(silu(z) * (w * (y*inv)))), then the K = 4096 4-bit dot.  Reference: gdn_norm_gate_rows SeedlessFusedVerify.swift:768-812.
// -------------------------------------------------------------------------------------------------
template <int R>
__global__ __launch_bounds__(256) void k_qmv_gdn_out(const uint16_t* __restrict__ ycore, const uint16_t* __restrict__ proj,
                                                     const float* __restrict__ norm_w, int norm_f32, const uint32_t* __restrict__ W,
                                                     const uint32_t* __restrict__ SB, int N, uint16_t* __restrict__ y) {
  const int m = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float sx[2];
  uint32_t xp[32];
  float nw[32];                                  // norm weight as fp32 (exact for an fp16 checkpoint weight)
#pragma unroll
  for (int i = 0; i < 32; i += 4) {
    const float4 v = *reinterpret_cast<const float4*>(norm_w + 32 * (lane & 3) + i);
    nw[i] = v.x; nw[i + 1] = v.y; nw[i + 2] = v.z; nw[i + 3] = v.w;
  }
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    float xb[32];
    load32(ycore + (size_t)m * 4096 + b * 2048 + 32 * lane, xb);
    float leaf[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) leaf[j] = fmaf(xb[2 * j + 1], xb[2 * j + 1], fmaf(xb[2 * j], xb[2 * j], 0.0f));
#pragma unroll
    for (int st = 1; st < 16; st <<= 1)
#pragma unroll
      for (int j = 0; j < 16; j += 2 * st) leaf[j] = leaf[j] + leaf[j + st];
    const float ss = tree_sum<4>(leaf[0]);
    const float inv = 1.0f / sqrtf(ss / 128.0f + EPS);
    float z[32];
    load32(proj + (size_t)m * PROJ_STRIDE + 8192 + b * 2048 + 32 * lane, z);
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      const float nrm = norm_f32 ? nw[i] * (xb[i] * inv) : f16r(nw[i] * f16r(xb[i] * inv));
      xb[i] = f16r((z[i] * sigmoid32(z[i])) * nrm);
    }
    sx[b] = share_sum(xb);
    pack_x(xb, xp + 16 * b);
  }
  const size_t row0 = ((size_t)blockIdx.x * 4 + wave) * R;
  if (row0 >= (size_t)N) return;
  size_t rows[R];
#pragma unroll
  for (int r = 0; r < R; ++r) rows[r] = row0 + r;
  float out[R];
  qdot_rows<2, R>(W, SB, rows, lane, xp, sx, out);
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) y[(size_t)m * H + row0 + r] = f2h(out[r]);
  }
}

// -------------------------------------------------------------------------------------------------
// Gated rmsnorm rows on their own (hybrid prefill: the out-projection then runs on the matrix cores):
// gated[m, hv, :] = half(silu(z) * norm(y)) in place of y.  One wave per (value head, row); lane l owns the pair
// 2l, 2l+1, so the sum of squares is the same balanced tree as in the fused kernel above.
// -------------------------------------------------------------------------------------------------
// `ysum` (or null) receives the sums of the row's shares of 32 gated values ([M, 128], share_sum's tree) for the
// projection that follows: a share sits on sixteen neighbouring lanes.
__global__ __launch_bounds__(64) void k_gdn_gate_rows(uint16_t* __restrict__ ycore, const uint16_t* __restrict__ proj,
                                                      const float* __restrict__ norm_w, int norm_f32, float* __restrict__ ysum = nullptr) {
  const int hv = blockIdx.x, m = blockIdx.y, lane = threadIdx.x;
  uint16_t* yp = ycore + (size_t)m * 4096 + hv * 128 + 2 * lane;
  const uint32_t yw = *reinterpret_cast<const uint32_t*>(yp);
  const uint32_t zw = *reinterpret_cast<const uint32_t*>(proj + (size_t)m * PROJ_STRIDE + 8192 + hv * 128 + 2 * lane);
  const float y0 = lo_h(yw), y1 = hi_h(yw), z0 = lo_h(zw), z1 = hi_h(zw);
  const float ss = tree_sum<64>(fmaf(y1, y1, fmaf(y0, y0, 0.0f)));
  const float inv = 1.0f / sqrtf(ss / 128.0f + EPS);
  const float w0 = norm_w[2 * lane], w1 = norm_w[2 * lane + 1];
  const float n0 = norm_f32 ? w0 * (y0 * inv) : f16r(w0 * f16r(y0 * inv));
  const float n1 = norm_f32 ? w1 * (y1 * inv) : f16r(w1 * f16r(y1 * inv));
  const float o0 = f16r((z0 * sigmoid32(z0)) * n0), o1 = f16r((z1 * sigmoid32(z1)) * n1);
  *reinterpret_cast<uint32_t*>(yp) = pack2(o0, o1);
  if (ysum) {
    const float sw = tree_sum<16>(o0 + o1);
    if ((lane & 15) == 0) ysum[(size_t)m * 128 + hv * 4 + (lane >> 4)] = sw;
  }
}

// -------------------------------------------------------------------------------------------------
// A GDN layer's core for a few rows of one sequence (a verify step, M <= GDN_FEW_ROWS) in one launch: what
// k_gdn_prep_rows, k_gdn_scan_rows and k_gdn_gate_rows do in three, with the same arithmetic per row.  Grid 32: a
// workgroup of 16 waves owns one value head, so the gated norm over the head's 128 outputs stays inside it.  Every
// load from the projection rows is requested up front (a thread holds the conv window of its channel, M + 3 taps);
// conv outputs, normed queries / keys, decays and betas of all rows wait in LDS, and the recurrence then runs
// through the rows without a barrier.  Wave w holds state rows 8 w .. 8 w + 7 of the head, one per half-wave and pass.
// -------------------------------------------------------------------------------------------------
constexpr int GDN_FEW_ROWS = 8;
__global__ __launch_bounds__(1024) void k_gdn_few_rows(GdnArgs a, const float* __restrict__ norm_w, int norm_f32, float* __restrict__ ysum) {
  __shared__ float s_q[GDN_FEW_ROWS][128], s_k[GDN_FEW_ROWS][128], s_v[GDN_FEW_ROWS][128], s_y[GDN_FEW_ROWS][128];
  __shared__ float s_g[GDN_FEW_ROWS], s_b[GDN_FEW_ROWS];
  const int hv = blockIdx.x, hk = hv >> 1, M = a.M;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, half = lane >> 5, l32 = lane & 31;
  const bool par = a.st[1] != 0;
  const uint16_t* hin = par ? a.hist[1] : a.hist[0];
  uint16_t* hout = par ? a.hist[0] : a.hist[1];
  const float* sin_ = par ? a.state[1] : a.state[0];
  float* sout = par ? a.state[0] : a.state[1];
  float s[4][4];
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int dv = wave * 8 + it * 2 + half;
    const float4 v = *reinterpret_cast<const float4*>(sin_ + ((size_t)hv * 128 + dv) * 128 + 4 * l32);
    s[it][0] = v.x; s[it][1] = v.y; s[it][2] = v.z; s[it][3] = v.w;
  }
  // waves 0-1: query channels of the key head, 2-3: its key channels, 4-5: the value channels of this head;
  // wave 6, lane t: decay of row t; wave 7, lane t: beta of row t; waves 8..8+M-1: the z row of the gated norm
  const int ch = tid < 128 ? hk * 128 + tid : (tid < 256 ? 2048 + hk * 128 + (tid - 128) : 4096 + hv * 128 + (tid - 256));
  uint16_t win[GDN_FEW_ROWS + 3];
  float cw[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (tid < 384) {
#pragma unroll
    for (int j = 0; j < GDN_FEW_ROWS + 3; ++j) {
      const int row = min(j, M + 2);                     // rows of the concatenation [hist(3) | qkv(M)]
      win[j] = (row < 3) ? hin[row * SL_CONV_DIM + ch] : a.proj[(size_t)(row - 3) * PROJ_STRIDE + ch];
    }
    const float4 c4 = *reinterpret_cast<const float4*>(a.conv_w + ch * 4);
    cw[0] = c4.x; cw[1] = c4.y; cw[2] = c4.z; cw[3] = c4.w;
  }
  uint32_t zw = 0;
  float nw0 = 0.0f, nw1 = 0.0f;
  if (wave >= 8 && wave - 8 < M) {
    zw = *reinterpret_cast<const uint32_t*>(a.proj + (size_t)(wave - 8) * PROJ_STRIDE + 8192 + hv * 128 + 2 * lane);
    nw0 = norm_w[2 * lane]; nw1 = norm_w[2 * lane + 1];
  }
  if (tid < 384) {
    float* dst = tid < 128 ? &s_q[0][tid] : (tid < 256 ? &s_k[0][tid - 128] : &s_v[0][tid - 256]);
#pragma unroll
    for (int t = 0; t < GDN_FEW_ROWS; ++t) {
      if (t >= M) continue;
      float acc = 0.0f;
#pragma unroll
      for (int k = 0; k < 4; ++k) acc = fmaf(h2f(win[t + k]), cw[k], acc);
      dst[t * 128] = f16r(acc * sigmoid32(acc));
    }
  } else if (wave == 6 && lane < M) {
    const float aP = h2f(a.proj[(size_t)lane * PROJ_STRIDE + 12320 + hv]);
    s_g[lane] = exp_c(-(exp_c(a.a_log[hv]) * softplus_c(aP + a.dt_bias[hv])));
  } else if (wave == 7 && lane < M) {
    s_b[lane] = sigmoid16(h2f(a.proj[(size_t)lane * PROJ_STRIDE + 12288 + hv]));
  }
  __syncthreads();
  if (wave < 2 * M) {
    // weightless rmsnorm over 128, then the key / query scale, both rounded to half: wave = (row, query | key)
    float* buf = (wave & 1) ? s_k[wave >> 1] : s_q[wave >> 1];
    const float x0 = buf[2 * lane], x1 = buf[2 * lane + 1];
    float ss = fmaf(x1, x1, fmaf(x0, x0, 0.0f));
    ss = tree_sum<64>(ss);
    const float inv = 1.0f / sqrtf(ss / 128.0f + EPS);
    const float sc = (wave & 1) ? f16r(0.08838834764831845f) : f16r(0.0078125f);
    buf[2 * lane] = f16r(sc * f16r(x0 * inv)); buf[2 * lane + 1] = f16r(sc * f16r(x1 * inv));
  }
  __syncthreads();
  for (int t = 0; t < M; ++t) {
    const float g = s_g[t], beta = s_b[t];
    const float4 k4 = *reinterpret_cast<const float4*>(&s_k[t][4 * l32]);
    const float4 q4 = *reinterpret_cast<const float4*>(&s_q[t][4 * l32]);
    const float kk[4] = {k4.x, k4.y, k4.z, k4.w}, qq[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int dvl = wave * 8 + it * 2 + half;
      float acc = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; ++i) { s[it][i] = s[it][i] * g; acc = fmaf(s[it][i], kk[i], acc); }
      const float kv = tree_sum<32>(acc);
      const float delta = (s_v[t][dvl] - kv) * beta;
      acc = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; ++i) { s[it][i] = fmaf(kk[i], delta, s[it][i]); acc = fmaf(s[it][i], qq[i], acc); }
      const float y = tree_sum<32>(acc);
      if (l32 == 0) s_y[t][dvl] = f16r(y);
    }
  }
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int dv = wave * 8 + it * 2 + half;
    *reinterpret_cast<float4*>(sout + ((size_t)hv * 128 + dv) * 128 + 4 * l32) = make_float4(s[it][0], s[it][1], s[it][2], s[it][3]);
  }
  // history shift: rows M .. M + 2 of [hist | qkv]; query and key channels by the even heads, value channels by every head
  if (tid < 384 && (tid >= 256 || (hv & 1) == 0)) {
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      uint16_t tap = win[3];                             // (a run-time index into the window would move it to scratch memory)
#pragma unroll
      for (int r = 1; r <= GDN_FEW_ROWS; ++r) if (M == r) tap = win[r + j];
      hout[j * SL_CONV_DIM + ch] = tap;
    }
  }
  __syncthreads();
  if (wave >= 8 && wave - 8 < M) {
    // gated norm of row wave - 8 over the head's 128 outputs (the arithmetic of k_gdn_gate_rows), and the sums of
    // each share of 32 gated values for the out-projection's dots
    const int m = wave - 8;
    const float y0 = s_y[m][2 * lane], y1 = s_y[m][2 * lane + 1], z0 = lo_h(zw), z1 = hi_h(zw);
    const float ss = tree_sum<64>(fmaf(y1, y1, fmaf(y0, y0, 0.0f)));
    const float inv = 1.0f / sqrtf(ss / 128.0f + EPS);
    const float n0 = norm_f32 ? nw0 * (y0 * inv) : f16r(nw0 * f16r(y0 * inv));
    const float n1 = norm_f32 ? nw1 * (y1 * inv) : f16r(nw1 * f16r(y1 * inv));
    const float o0 = f16r((z0 * sigmoid32(z0)) * n0), o1 = f16r((z1 * sigmoid32(z1)) * n1);
    *reinterpret_cast<uint32_t*>(a.ycore + (size_t)m * 4096 + hv * 128 + 2 * lane) = pack2(o0, o1);
    const float sw = tree_sum<16>(o0 + o1);
    if ((lane & 15) == 0) ysum[(size_t)m * 128 + hv * 4 + (lane >> 4)] = sw;
  }
}

// -------------------------------------------------------------------------------------------------
// MoE stage A: residual + post-attention norm, then in one launch the shared expert's gate/up
// with SwiGLU (64 workgroups), the fp16 router gate rows and the shared-expert gate row.
// References: MoEBlock.swift:69-97; shared expert SeedlessFusedVerify.swift:1859-1871.
// -------------------------------------------------------------------------------------------------
struct MoeAArgs {
  HiddenArgs ha;
  const uint32_t *shg_w, *shg_sb, *shu_w, *shu_sb;   // shared gate_proj / up_proj [512, 2048]
  const uint16_t* router_w;                          // [E, 2048]
  const uint16_t* sgate_w;                           // [2048]
  const uint32_t *g8_w, *g8_sb;                      // 8-bit gates instead (null: fp16): [E+1, 512] words, [E+1, 32] {scale, bias}; row E = shared gate
  int E;
  int skip_shared;                                   // hybrid prefill: the shared expert's gate/up run on the matrix cores; grid.x = router blocks only
  const uint16_t* xn_in;                             // rows already normed by k_final_rows (M >= 2), or null: hidden prologue here
  uint16_t* sh_act;                                  // [M, 512]
  uint16_t* rlogits;                                 // [M, 256]
  uint16_t* sgate;                                   // [M]
};
constexpr int MOE_A_SHARED_BLOCKS = 64;
__global__ __launch_bounds__(256) void k_moe_a(MoeAArgs a) {
  const int m = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float x[32], sx[1];
  if (a.xn_in) load32(a.xn_in + (size_t)m * H + 32 * lane, x);
  else hidden_prologue(a.ha, m, lane, blockIdx.x == 0 && wave == 0, x);
  // skip_shared: the grid holds the router blocks only
  const int bx = a.skip_shared ? (int)blockIdx.x + MOE_A_SHARED_BLOCKS : (int)blockIdx.x;
  if (bx < MOE_A_SHARED_BLOCKS) {
    sx[0] = share_sum(x);
    uint32_t xp[16];
    pack_x(x, xp);
    const size_t i0 = ((size_t)bx * 4 + wave) * 2;
    const size_t rows[2] = {i0, i0 + 1};
    float g[2], u[2];
    qdot_rows<1, 2>(a.shg_w, a.shg_sb, rows, lane, xp, sx, g);
    qdot_rows<1, 2>(a.shu_w, a.shu_sb, rows, lane, xp, sx, u);
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < 2; ++r) a.sh_act[(size_t)m * 512 + i0 + r] = f2h(swiglu16(f16r(g[r]), f16r(u[r])));
    }
  } else {
    const int row0 = ((bx - MOE_A_SHARED_BLOCKS) * 4 + wave) * 4;
    for (int r = 0; r < 4; ++r) {
      const int row = row0 + r;
      if (row > a.E) continue;
      float v;
      if (a.g8_w) {
        const uint4 w0 = ld16(a.g8_w + (size_t)row * 512 + 8 * lane), w1 = ld16(a.g8_w + (size_t)row * 512 + 8 * lane + 4);
        const uint32_t w8[8] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
        v = tree_sum<64>(q8_lane(w8, a.g8_sb[(size_t)row * 32 + (lane >> 1)], x));
      } else {
        v = dense_dot(row < a.E ? a.router_w + (size_t)row * H : a.sgate_w, lane, x);
      }
      if (lane == 0) { if (row < a.E) a.rlogits[(size_t)m * 256 + row] = f2h(v); else a.sgate[m] = f2h(v); }
    }
  }
}

// -------------------------------------------------------------------------------------------------
// Router: softmax over the half logits, gates rounded to half, 8 x arg-max of the raw logits
// (ties to the lower index), half renormalisation.  One wave; lane l owns experts 4l..4l+3.
// Reference: route_top8_rows SeedlessFusedVerify.swift:191-213.
// -------------------------------------------------------------------------------------------------
// Order key of a router logit: larger logit first, lower expert index first on ties (+0 and -0 tie).
SL_DEV uint32_t route_order_key(uint32_t hbits, int e) {
  uint32_t u = hbits & 0xffffu;
  if ((u & 0x7fffu) == 0) u = 0;
  u = (u & 0x8000u) ? (~u & 0xffffu) : (u | 0x8000u);
  return (u << 8) | (uint32_t)(255 - e);
}
SL_DEV void route_wave(const uint16_t* __restrict__ logits, int E, int lane, int* inds /*LDS [8]*/, float* scores /*LDS [8]*/) {
  const float NEG = -__int_as_float(0x7f800000);
  float lg[4], ex[4];
  uint32_t key[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const bool in = 4 * lane + i < E;
    const uint32_t bits = in ? logits[4 * lane + i] : 0u;
    lg[i] = in ? h2f((uint16_t)bits) : NEG;
    key[i] = in ? route_order_key(bits, 4 * lane + i) : 0u;
  }
  const float mx = tree_max<64>(fmaxf(fmaxf(lg[0], lg[1]), fmaxf(lg[2], lg[3])));
#pragma unroll
  for (int i = 0; i < 4; ++i) ex[i] = (4 * lane + i < E) ? exp_c(lg[i] - mx) : 0.0f;
  const float Z = tree_sum<64>(((ex[0] + ex[1]) + ex[2]) + ex[3]);
  // eight times: the largest remaining key (one value to reduce; the index rides in its low byte), then remove it
  float sc[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    uint32_t m = max(max(key[0], key[1]), max(key[2], key[3]));
    m = max(m, dpp_u<DPP_XOR1>(m));
    m = max(m, dpp_u<DPP_XOR2>(m));
    m = max(m, dpp_u<DPP_HALF_MIRROR>(m));
    m = max(m, dpp_u<DPP_MIRROR>(m));
    const uint32_t top = max(max((uint32_t)__builtin_amdgcn_readlane((int)m, 0), (uint32_t)__builtin_amdgcn_readlane((int)m, 16)),
                             max((uint32_t)__builtin_amdgcn_readlane((int)m, 32), (uint32_t)__builtin_amdgcn_readlane((int)m, 48)));
#pragma unroll
    for (int i = 0; i < 4; ++i) key[i] = (key[i] == top) ? 0u : key[i];
    const int bi = min(255 - (int)(top & 255u), E - 1), sub = bi & 3;
    const float mine = (sub == 0) ? ex[0] : (sub == 1) ? ex[1] : (sub == 2) ? ex[2] : ex[3];
    const float e = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(mine), bi >> 2));
    sc[k] = f16r(e / Z);
    if (lane == 0) inds[k] = bi;
  }
  if (lane == 0) {
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; ++k) ss = f16r(ss + sc[k]);
#pragma unroll
    for (int k = 0; k < 8; ++k) scores[k] = f16r(sc[k] / ss);
  }
}

// Routing of M rows: one wave per row (softmax, top-8, renormalise; MoEBlock.swift:69-97).
__global__ __launch_bounds__(64) void k_route_rows(const uint16_t* __restrict__ rlogits, int E, int32_t* __restrict__ inds,
                                                   uint16_t* __restrict__ scores) {
  __shared__ int s_inds[8];
  __shared__ float s_sc[8];
  const int m = blockIdx.x, lane = threadIdx.x;
  route_wave(rlogits + (size_t)m * 256, E, lane, s_inds, s_sc);
  __syncthreads();
  if (lane < 8) { inds[m * 8 + lane] = s_inds[lane]; scores[m * 8 + lane] = f2h(s_sc[lane]); }
}

// MoE stage B: the 8 routed experts' gate/up with SwiGLU, after k_route_rows (ROUTE: every wave routes its row itself
// first, for steps of a few rows, and workgroup 0 of the row leaves the routing for stage C).  A wave owns four consecutive rows of
// one expert (gate and up); all eight weight loads are in flight before the first dot.  Grid (256, M).
// Reference: gqmm4_swiglu_rows SeedlessMetalForward.swift:1419-1460.
struct MoeBArgs {
  const uint16_t* xn;          // [M, 2048] post-normed rows
  const uint32_t *g_w, *g_sb, *u_w, *u_sb;   // [E*512, 2048]
  uint16_t* act;               // [M, 8, 512]
  const int32_t* inds;         // [M, 8]
  const float* xsum;           // [M, 64] share sums of the rows (HiddenArgs::xs_out), or null: formed here
  // a few rows (a verify step): no routing launch before this one; every wave routes its row itself from the logits
  // and workgroup 0 of the row leaves indices and scores for stage C
  const uint16_t* rlogits;     // [M, 256] (k_moe_b<true>; otherwise `inds` holds the routing)
  int E;
  int32_t* inds_out;           // [M, 8]
  uint16_t* scores_out;        // [M, 8]
};
constexpr int GROUP_CAP = 2048;         // pairs per expert: an expert is chosen at most once per row, M <= 2048
// Pairs (row, slot) listed per expert (M * 8 pairs walked by 1024 threads), places handed out by LDS counters.
// The order within a list varies from run to run; results do not depend on it (they are scattered back by pair).
// `order` (optional) receives the experts sorted by falling count, ties by index: kernels whose workgroups are
// dealt out by expert start the long ones first, which shortens the tail of the launch.
__global__ __launch_bounds__(1024) void k_group_pairs(const int32_t* __restrict__ inds, int M, int E, uint16_t* __restrict__ lists,
                                                      int32_t* __restrict__ counts, int32_t* __restrict__ order) {
  __shared__ __align__(16) int s_cnt[SL_MAX_EXPERTS];
  static_assert(SL_MAX_EXPERTS * 4 == 1024, "four lanes rank one expert");
  if (threadIdx.x < SL_MAX_EXPERTS) s_cnt[threadIdx.x] = 0;
  __syncthreads();
  // a thread's pairs (M <= GROUP_CAP: at most 16) are all requested before the first of them is counted: the walk
  // is one round trip to memory instead of one per pair
  static_assert(GROUP_CAP * 8 == 16 * 1024, "sixteen pairs per thread at most");
  int ev[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) { const int p = threadIdx.x + 1024 * i; ev[i] = p < M * 8 ? inds[p] : -1; }
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int p = threadIdx.x + 1024 * i, e = ev[i];
    if (e >= 0 && e < E) {
      const int pos = atomicAdd(&s_cnt[e], 1);
      if (pos < GROUP_CAP) lists[e * GROUP_CAP + pos] = (uint16_t)p;
    }
  }
  __syncthreads();
  // four lanes per expert: each ranks it against a quarter of the counts (16-byte reads), the quarters add up by shuffle
  const int e = threadIdx.x >> 2, part = threadIdx.x & 3;
  const int c = s_cnt[e];
  if (part == 0 && e < E) counts[e] = c;
  if (order) {
    int rank = 0;
    const int4* cq = reinterpret_cast<const int4*>(s_cnt) + part * (SL_MAX_EXPERTS / 16);
#pragma unroll 4
    for (int q = 0; q < SL_MAX_EXPERTS / 16; ++q) {
      const int4 v = cq[q];
      const int j = (part * (SL_MAX_EXPERTS / 16) + q) * 4;
      rank += (j < E && (v.x > c || (v.x == c && j < e))) ? 1 : 0;
      rank += (j + 1 < E && (v.y > c || (v.y == c && j + 1 < e))) ? 1 : 0;
      rank += (j + 2 < E && (v.z > c || (v.z == c && j + 2 < e))) ? 1 : 0;
      rank += (j + 3 < E && (v.w > c || (v.w == c && j + 3 < e))) ? 1 : 0;
    }
    rank += __shfl_xor(rank, 1);
    rank += __shfl_xor(rank, 2);
    if (part == 0 && e < E) order[rank] = e;
  }
}
// Stage B by expert (steps of many rows): grid (64, E), or (64, ceil(M / 64) + E) with the shared expert.  A workgroup holds eight gate/up row pairs of one expert
// (two pairs per wave, unpacked into masks once) and walks the expert's list of (row, slot) pairs in tiles of
// MOEB_MT activation rows parked in LDS as in k_qmv_tile, so the expert's weights are fetched and unpacked once
// per step instead of once per row that chose it.  Same arithmetic per (pair, weight row) as k_moe_b.
struct MoeBGroupArgs {
  const uint16_t* xn;          // [M, 2048]
  const uint32_t *g_w, *g_sb, *u_w, *u_sb;   // [E*512, 2048]
  uint16_t* act;               // [M, 8, 512]
  const uint16_t* lists;       // [E, GROUP_CAP] pair indices row*8 + slot
  const int32_t* counts;       // [E]
  const float* xsum;           // [M, 64] share sums of the rows (HiddenArgs::xs_out), or null: formed here
  const int32_t* order;        // [E] experts by falling count: the long lists start first
  // the shared expert as one more list (every row of the step, in segments of 64 rows that come first in the grid):
  const uint32_t *shg_w, *shg_sb, *shu_w, *shu_sb;   // its gate_proj / up_proj [512, 2048], or null: grid (64, E) only
  uint16_t* sh_act;            // [M, 512]
  int M;
};
constexpr int MOEB_MT = 8;          // pairs per tile: one per eight lanes of a wave in the tile's SwiGLU
__global__ __launch_bounds__(256, 3) void k_moe_b_grouped(MoeBGroupArgs a) {
  __shared__ uint4 xs[MOEB_MT * 64 * 5];
  __shared__ int s_pair[MOEB_MT];
  const int S = a.shg_w ? (a.M + 63) / 64 : 0;           // grid (64, S + E): the shared expert's segments, then the experts
  const bool shared = (int)blockIdx.y < S;
  const int e = shared ? 0 : a.order[blockIdx.y - S];
  const int row0 = shared ? 64 * blockIdx.y : 0;
  const int cnt = shared ? min(64, a.M - row0) : min(a.counts[e], GROUP_CAP);
  if (cnt == 0) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int i0 = (blockIdx.x * 4 + wave) * 2;
  const size_t base = (size_t)e * 512 + i0;
  const uint32_t* const gw = shared ? a.shg_w : a.g_w;
  const uint32_t* const gsb = shared ? a.shg_sb : a.g_sb;
  const uint32_t* const uw = shared ? a.shu_w : a.u_w;
  const uint32_t* const usb = shared ? a.shu_sb : a.u_sb;
  uint4 wv[4];
  uint32_t sb[4];
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    wv[r] = ld16(gw + (base + r) * 256 + 4 * lane); sb[r] = gsb[(base + r) * 32 + (lane >> 1)];
    wv[2 + r] = ld16(uw + (base + r) * 256 + 4 * lane); sb[2 + r] = usb[(base + r) * 32 + (lane >> 1)];
  }
  h2_t mk[4][16];
  for (int t0 = 0; t0 < cnt; t0 += MOEB_MT) {
    const int mc = min(MOEB_MT, cnt - t0);
    if (t0) __syncthreads();                             // the previous tile has been read
    for (int j = wave; j < mc; j += 4) {
      // a pair index row * 8 + slot; a row of the shared expert counts as its slot 0 here
      const int p = shared ? (row0 + t0 + j) * 8 : (int)a.lists[(size_t)e * GROUP_CAP + t0 + j];
      if (lane == 0) s_pair[j] = p;
      uint4* dst = xs + (j * 64 + lane) * 5;
      if (a.xsum) {                                        // the stored halves are the packed pairs; their sums came with the row
        const uint16_t* src = a.xn + (size_t)(p >> 3) * H + 32 * lane;
#pragma unroll
        for (int q = 0; q < 4; ++q) dst[q] = ld16(src + 8 * q);
        dst[4] = make_uint4(__float_as_uint(a.xsum[(size_t)(p >> 3) * 64 + lane]), 0u, 0u, 0u);
        continue;
      }
      float x[32];
      load32(a.xn + (size_t)(p >> 3) * H + 32 * lane, x);
      const float sx = share_sum(x);
      uint32_t xp[16];
      pack_x(x, xp);
#pragma unroll
      for (int q = 0; q < 4; ++q) dst[q] = make_uint4(xp[4 * q], xp[4 * q + 1], xp[4 * q + 2], xp[4 * q + 3]);
      dst[4] = make_uint4(__float_as_uint(sx), 0u, 0u, 0u);
    }
    __syncthreads();
    if (t0 == 0) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        word_masks(wv[r].x, mk[r]); word_masks(wv[r].y, mk[r] + 4);
        word_masks(wv[r].z, mk[r] + 8); word_masks(wv[r].w, mk[r] + 12);
      }
    }
    // The sums of pair j are parked on lanes 8j and 8j + 1 (gate and up of the wave's two rows), and the SwiGLU of
    // the whole tile is formed once, sixteen lanes at a time: per pair it would cost every lane of the wave two
    // evaluations of the exact sigmoid, a quarter of the kernel's instructions.
    float G = 0.0f, U = 0.0f;
    for (int j = 0; j < mc; ++j) {
      const uint4* src = xs + (j * 64 + lane) * 5;
      uint32_t xp[16];
#pragma unroll
      for (int q = 0; q < 4; ++q) { const uint4 v = src[q]; xp[4 * q] = v.x; xp[4 * q + 1] = v.y; xp[4 * q + 2] = v.z; xp[4 * q + 3] = v.w; }
      const float sx = __uint_as_float(reinterpret_cast<const uint32_t*>(src + 4)[0]);
      float o[4];                                          // rows 0..3 in the lower quad of every eight lanes
      quad_values(tree_sum4(share_term_masked(mk[0], sb[0], xp, sx), share_term_masked(mk[1], sb[1], xp, sx),
                            share_term_masked(mk[2], sb[2], xp, sx), share_term_masked(mk[3], sb[3], xp, sx), lane), o);
      const bool mine = (lane >> 3) == j;
      G = mine ? ((lane & 1) ? o[1] : o[0]) : G;
      U = mine ? ((lane & 1) ? o[3] : o[2]) : U;
    }
    const float y = swiglu16(f16r(G), f16r(U));
    if ((lane & 7) < 2 && (lane >> 3) < mc) {
      const int p = s_pair[lane >> 3];
      (shared ? a.sh_act + (size_t)(p >> 3) * 512 : a.act + (size_t)p * 512)[i0 + (lane & 1)] = f2h(y);
    }
  }
}
template <bool ROUTE>
__global__ __launch_bounds__(256) void k_moe_b(MoeBArgs a) {
  const int m = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int p0 = (blockIdx.x * 4 + wave) * 4;          // row index in [0, 8*512)
  const int k = p0 >> 9, i0 = p0 & 511;
  __shared__ int s_inds[ROUTE ? 4 : 1][8];
  __shared__ float s_sc[ROUTE ? 4 : 1][8];
  int expert;
  if constexpr (ROUTE) {
    route_wave(a.rlogits + (size_t)m * 256, a.E, lane, s_inds[wave], s_sc[wave]);
    __syncthreads();
    expert = s_inds[wave][k];
    if (blockIdx.x == 0 && wave == 0 && lane < 8) { a.inds_out[m * 8 + lane] = s_inds[0][lane]; a.scores_out[m * 8 + lane] = f2h(s_sc[0][lane]); }
  } else {
    expert = a.inds[m * 8 + k];
  }
  const size_t base = (size_t)expert * 512 + i0;
  uint4 gw[4], uw[4];
  uint32_t gs[4], us[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    gw[r] = ld16(a.g_w + (base + r) * 256 + 4 * lane); gs[r] = a.g_sb[(base + r) * 32 + (lane >> 1)];
    uw[r] = ld16(a.u_w + (base + r) * 256 + 4 * lane); us[r] = a.u_sb[(base + r) * 32 + (lane >> 1)];
  }
  float sx;
  uint32_t xp[16];
  if (a.xsum) {                                          // the stored halves are the packed pairs
    const uint16_t* src = a.xn + (size_t)m * H + 32 * lane;
#pragma unroll
    for (int j = 0; j < 4; ++j) { const uint4 v = ld16(src + 8 * j); xp[4 * j] = v.x; xp[4 * j + 1] = v.y; xp[4 * j + 2] = v.z; xp[4 * j + 3] = v.w; }
    sx = a.xsum[(size_t)m * 64 + lane];
  } else {
    float x[32];
    load32(a.xn + (size_t)m * H + 32 * lane, x);
    sx = share_sum(x);
    pack_x(x, xp);
  }
  // the four gate sums and the four up sums each reduced in one register: lane r (r < 4) holds row r of both and
  // forms its SwiGLU
  const float g = tree_sum4(share_term(gw[0], gs[0], xp, sx), share_term(gw[1], gs[1], xp, sx),
                            share_term(gw[2], gs[2], xp, sx), share_term(gw[3], gs[3], xp, sx), lane);
  const float u = tree_sum4(share_term(uw[0], us[0], xp, sx), share_term(uw[1], us[1], xp, sx),
                            share_term(uw[2], us[2], xp, sx), share_term(uw[3], us[3], xp, sx), lane);
  const float o = swiglu16(f16r(g), f16r(u));
  if (lane < 4) a.act[((size_t)m * 8 + k) * 512 + i0 + lane] = f2h(o);
}

// MoE stage C: routed down-proj, half-precision combine in routing order, shared down-proj and the
// sigmoid-gated shared add.  References: gqmm4_rows SeedlessMetalForward.swift:4017; combine_rows
// SeedlessFusedVerify.swift:462-470; shared_gate_combine_rows :1051-1109.
struct MoeCArgs {
  const uint16_t* act;         // [M, 8, 512]
  const uint16_t* sh_act;      // [M, 512]
  const int32_t* inds;         // [M, 8]
  const uint16_t* scores;      // [M, 8]
  const uint16_t* sgate;       // [M]
  const uint32_t *d_w, *d_sb;  // [E*2048, 512]
  const uint32_t *shd_w, *shd_sb;   // [2048, 512]
  uint16_t* out;               // [M, 2048]
};
// Grid (128, M), four waves: 16 lanes per output row, 16 rows per workgroup.  The nine activation rows (the stored
// halves as they are) are parked in LDS once per workgroup, 64 bytes per lane at an 80-byte pitch so that the 16 lanes
// of a row read them without bank conflicts, and their share sums are formed once per workgroup.
__global__ __launch_bounds__(256) void k_moe_c(MoeCArgs a) {
  constexpr int XP = 20;                                  // words per lane slot: 16 + 4 pad
  __shared__ float s_sx[9 * 16];
  __shared__ __align__(16) uint32_t s_x[9 * 16 * XP];
  const int m = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int sub = lane >> 4, li = lane & 15;
  const int n = (blockIdx.x * 4 + wave) * 4 + sub;
  // every load of the eight experts and of the shared expert is issued before the first dot
  uint4 wv[9];
  uint32_t sb[9];
  float sc[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const size_t row = (size_t)a.inds[m * 8 + k] * 2048 + n;
    wv[k] = ld16(a.d_w + row * 64 + 4 * li);
    sb[k] = a.d_sb[row * 8 + (li >> 1)];
    sc[k] = h2f(a.scores[m * 8 + k]);
  }
  wv[8] = ld16(a.shd_w + (size_t)n * 64 + 4 * li);
  sb[8] = a.shd_sb[(size_t)n * 8 + (li >> 1)];
  for (int c = tid; c < 9 * 64; c += 256) {              // 16-byte pieces: row k, lane slot l, quarter j
    const int k = c >> 6, l = (c >> 2) & 15, j = c & 3;
    const uint16_t* src = (k < 8 ? a.act + ((size_t)m * 8 + k) * 512 : a.sh_act + (size_t)m * 512) + 32 * l + 8 * j;
    st16(&s_x[(k * 16 + l) * XP + 4 * j], ld16(src));
  }
  __syncthreads();
  if (tid < 9 * 16) {
    float x[32];
#pragma unroll
    for (int j = 0; j < 4; ++j) unpack8(ld16(&s_x[tid * XP + 4 * j]), x + 8 * j);
    s_sx[tid] = share_sum(x);
  }
  __syncthreads();
  float acc = 0.0f, sy = 0.0f;
#pragma unroll
  for (int k = 0; k < 9; ++k) {
    uint32_t xp[16];
#pragma unroll
    for (int j = 0; j < 4; ++j) { const uint4 v = ld16(&s_x[(k * 16 + li) * XP + 4 * j]); xp[4 * j] = v.x; xp[4 * j + 1] = v.y; xp[4 * j + 2] = v.z; xp[4 * j + 3] = v.w; }
    const float d = f16r(tree_sum<16>(share_term(wv[k], sb[k], xp, s_sx[k * 16 + li])));
    if (k < 8) acc = f16r(acc + f16r(d * sc[k]));
    else sy = d;
  }
  const float s = sigmoid16(h2f(a.sgate[m]));
  if (li == 0) a.out[(size_t)m * H + n] = f2h(f16r(acc + f16r(s * sy)));
}

// Stage C by expert (steps of many rows): the down-projections of the pairs that chose expert e, with e's rows
// fetched and unpacked into masks once per step instead of once per pair (reference: the grouped family
// moe_count / moe_csr / gqmm4_grouped, SeedlessMetalForward.swift:3116-3556).  Grid (64, ceil(M / 64) + E): the shared
// expert's rows in segments of 64, then the experts.  A workgroup holds 32 output rows of its expert, two per group
// of 16 lanes (K = 512: a lane owns 32 activations), and walks the list in tiles of MOEC_MT pairs whose activation
// rows are parked in LDS with their share sums.  Same arithmetic per (pair, output row) as k_moe_c:
// d = half(tree_sum<16>(share term)).  The results go out by pair (routed) or by row (shared);
// k_moe_combine_rows adds them up in routing order.
struct MoeCGroupArgs {
  const uint16_t* act;         // [M, 8, 512]
  const uint16_t* sh_act;      // [M, 512]
  const uint32_t *d_w, *d_sb;  // [E*2048, 512]
  const uint32_t *shd_w, *shd_sb;   // [2048, 512]
  const uint16_t* lists;       // [E, GROUP_CAP] pair indices row*8 + slot
  const int32_t* counts;       // [E]
  const int32_t* order;        // [E] experts by falling count
  uint16_t* d;                 // [M*8, 2048] routed down results by pair
  uint16_t* sy;                // [M, 2048] shared down results by row
  int M, E;
};
constexpr int MOEC_MT = 16;
__global__ __launch_bounds__(256, 3) void k_moe_c_grouped(MoeCGroupArgs a) {
  constexpr int XP = 20;                                  // words per lane slot: 16 + 4 pad
  constexpr int PIECES = MOEC_MT * 64 / 256;              // 16-byte pieces of a tile per thread
  __shared__ __align__(16) uint32_t s_x[MOEC_MT * 16 * XP];
  __shared__ float s_sx[MOEC_MT * 16];
  __shared__ int s_dst[MOEC_MT];
  // blockIdx.y < S: segment of 64 rows of the shared expert (first, and cut up: as one list of M rows it would run
  // thirty times longer than an expert's and end the launch with 64 workgroups); then the experts by falling count
  const int S = (a.M + 63) / 64;
  const bool shared = (int)blockIdx.y < S;
  const int e = shared ? 0 : a.order[blockIdx.y - S];
  const int row0 = shared ? 64 * blockIdx.y : 0;
  const int cnt = shared ? min(64, a.M - row0) : min(a.counts[e], GROUP_CAP);
  if (cnt == 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int sub = lane >> 4, li = lane & 15;
  const int n0 = blockIdx.x * 32 + (wave * 4 + sub) * 2;  // this 16-lane group's two output rows
  uint4 wv[2];
  uint32_t sb[2];
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const size_t row = (shared ? 0 : (size_t)e * 2048) + n0 + r;
    wv[r] = ld16((shared ? a.shd_w : a.d_w) + row * 64 + 4 * li);
    sb[r] = (shared ? a.shd_sb : a.d_sb)[row * 8 + (li >> 1)];
  }
  // a tile's pieces travel through registers one tile ahead (pair j = piece / 64, lane slot l, quarter q; pairs beyond
  // the list repeat its last one and are not used)
  uint4 px[PIECES];
  int pp[PIECES];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int c = tid + 256 * i, j = min(t0 + (c >> 6), cnt - 1), l = (c >> 2) & 15, q = c & 3;
      pp[i] = shared ? row0 + j : (int)a.lists[(size_t)e * GROUP_CAP + j];
      px[i] = ld16((shared ? a.sh_act : a.act) + (size_t)pp[i] * 512 + 32 * l + 8 * q);
    }
  };
  fetch(0);
  h2_t mk[2][16];
  for (int t0 = 0; t0 < cnt; t0 += MOEC_MT) {
    const int mc = min(MOEC_MT, cnt - t0);
    if (t0) __syncthreads();                             // the previous tile has been read
#pragma unroll
    for (int i = 0; i < PIECES; ++i) {
      const int c = tid + 256 * i, j = c >> 6, l = (c >> 2) & 15, q = c & 3;
      if ((c & 63) == 0) s_dst[j] = pp[i];
      st16(&s_x[(j * 16 + l) * XP + 4 * q], px[i]);
    }
    __syncthreads();
    if (t0 + MOEC_MT < cnt) fetch(t0 + MOEC_MT);
    if (tid < mc * 16) {
      float x[32];
#pragma unroll
      for (int q = 0; q < 4; ++q) unpack8(ld16(&s_x[tid * XP + 4 * q]), x + 8 * q);
      s_sx[tid] = share_sum(x);
    }
    if (t0 == 0) {
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        word_masks(wv[r].x, mk[r]); word_masks(wv[r].y, mk[r] + 4);
        word_masks(wv[r].z, mk[r] + 8); word_masks(wv[r].w, mk[r] + 12);
      }
    }
    __syncthreads();
    for (int j = 0; j < mc; ++j) {
      uint32_t xp[16];
#pragma unroll
      for (int q = 0; q < 4; ++q) { const uint4 v = ld16(&s_x[(j * 16 + li) * XP + 4 * q]); xp[4 * q] = v.x; xp[4 * q + 1] = v.y; xp[4 * q + 2] = v.z; xp[4 * q + 3] = v.w; }
      const float sx = s_sx[j * 16 + li];
      const float d0 = tree_sum<16>(share_term_masked(mk[0], sb[0], xp, sx));
      const float d1 = tree_sum<16>(share_term_masked(mk[1], sb[1], xp, sx));
      if (li == 0) {
        uint16_t* dst = (shared ? a.sy : a.d) + (size_t)s_dst[j] * H + n0;
        *reinterpret_cast<uint32_t*>(dst) = pack2(d0, d1);
      }
    }
  }
}

// -------------------------------------------------------------------------------------------------
// Attention prep: per-head rmsnorm with weight, partial NeoX RoPE on the first 64 dims from a
// (cos, sin) table, K and V appended to the cache.  Blocks 0..15: query heads; 16..17: kv heads.
// References: attn_q_prep_rows / attn_k_prep_rows SeedlessFusedVerify.swift:1183-1330; write_kv_rows :487.
// -------------------------------------------------------------------------------------------------
struct AttnPrepArgs {
  const uint16_t* proj;        // [M, PROJ_STRIDE]: q(+gate) 16x512 | k 2x256 | v 2x256
  const uint16_t *q_norm, *k_norm;
  const float *rope_cos, *rope_sin;   // [maxSeq, 32]
  const int32_t* st;           // st[0] = position of row 0
  uint16_t* qrot;              // [M, 16, 256]
  uint16_t *kcache, *vcache;   // [2, maxSeq, 256]
  int maxSeq;
  const LaneRef* lanes;        // lane batch: row m is the next token of lanes[m]
};
__global__ __launch_bounds__(64) void k_attn_prep(AttnPrepArgs a) {
  __shared__ float s_n[256];
  const int m = blockIdx.y, hb = blockIdx.x, lane = threadIdx.x;
  int pos = a.st[0] + m;
  if (a.lanes) {
    const LaneRef& r = a.lanes[m];
    pos = r.st[0]; a.kcache = r.kcache; a.vcache = r.vcache; a.maxSeq = r.max_seq;
  }
  const bool isq = hb < 16;
  const uint16_t* src = a.proj + (size_t)m * PROJ_STRIDE + (isq ? hb * 512 : 8192 + (hb - 16) * 256);
  const uint16_t* nw = isq ? a.q_norm : a.k_norm;
  const uint2 raw = *reinterpret_cast<const uint2*>(src + 4 * lane);
  const uint2 wraw = *reinterpret_cast<const uint2*>(nw + 4 * lane);
  const float xv[4] = {lo_h(raw.x), hi_h(raw.x), lo_h(raw.y), hi_h(raw.y)};
  const float wv[4] = {lo_h(wraw.x), hi_h(wraw.x), lo_h(wraw.y), hi_h(wraw.y)};
  const float ss = tree_sum<64>(fmaf(xv[1], xv[1], xv[0] * xv[0]) + fmaf(xv[3], xv[3], xv[2] * xv[2]));
  const float inv = 1.0f / sqrtf(ss / 256.0f + EPS);
#pragma unroll
  for (int i = 0; i < 4; ++i) s_n[4 * lane + i] = f16r(wv[i] * f16r(xv[i] * inv));
  __syncthreads();
  float o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = 4 * lane + i;
    if (d >= SL_ROPE_DIM) { o[i] = s_n[d]; continue; }
    const int ii = d & 31;
    const float c = a.rope_cos[(size_t)pos * 32 + ii], s = a.rope_sin[(size_t)pos * 32 + ii];
    const float x0 = s_n[ii], x1 = s_n[ii + 32];
    o[i] = (d < 32) ? f16r(fmaf(-x1, s, x0 * c)) : f16r(fmaf(x1, c, x0 * s));
  }
  const uint2 packed = make_uint2(pack2(o[0], o[1]), pack2(o[2], o[3]));
  if (isq) {
    *reinterpret_cast<uint2*>(a.qrot + ((size_t)m * 16 + hb) * 256 + 4 * lane) = packed;
  } else {
    const int h = hb - 16;
    const size_t off = ((size_t)h * a.maxSeq + pos) * 256 + 4 * lane;
    *reinterpret_cast<uint2*>(a.kcache + off) = packed;
    *reinterpret_cast<uint2*>(a.vcache + off) =
        *reinterpret_cast<const uint2*>(a.proj + (size_t)m * PROJ_STRIDE + 8192 + 512 + h * 256 + 4 * lane);
  }
}

// -------------------------------------------------------------------------------------------------
// Decode attention, tile pass: one workgroup of four waves per (key tile of 64, kv head, row), a wave per pair of
// query heads.  The tile's keys are
// staged in LDS; lane j scores key j against the query heads of its wave (eight fmaf chains over 32 dims
// each, combined by a balanced tree), then p = exp(s - tile max), l = butterfly sum of p, o = two fmaf chains over
// the halves of the tile's keys with the value tile parked in LDS (fetched once per workgroup).  Reference semantics: sdpa_rows
// SeedlessMetalForward.swift:4922-4989 (q scaled by 1/16, fp32 softmax).
// -------------------------------------------------------------------------------------------------
struct SdpaArgs {
  const uint16_t* qrot;        // [M, 16, 256]
  const uint16_t *kcache, *vcache;
  const int32_t* st;
  int maxSeq, maxTiles;
  float *pm, *pl;              // [M, 16, maxTiles]
  float* po;                   // [M, 16, maxTiles, 256]
  const LaneRef* lanes;        // lane batch: row m attends to the cache of lanes[m]
};
__global__ __launch_bounds__(256) void k_sdpa_tile(SdpaArgs a) {
  __shared__ __align__(16) uint16_t s_k[SDPA_TILE * KT_STRIDE];
  __shared__ __align__(16) float s_q[8 * 256];
  const int kvh = blockIdx.y, m = blockIdx.z, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int N = a.st[0] + m + 1;
  if (a.lanes) {
    const LaneRef& r = a.lanes[m];
    N = r.st[0] + 1; a.kcache = r.kcache; a.vcache = r.vcache; a.maxSeq = r.max_seq;
  }
  const int tile = blockIdx.x;
  if (tile * SDPA_TILE >= N) return;
  const int nk = min(SDPA_TILE, N - tile * SDPA_TILE);
  const uint16_t* const kc = a.kcache + (size_t)kvh * a.maxSeq * 256;
  const uint16_t* const vc = a.vcache + (size_t)kvh * a.maxSeq * 256;
  // The key tile is requested as a whole before anything waits for it (eight 16-byte pieces per thread, staged once
  // they are all here), the value tile behind it: it is parked in the key tile's space once the scores are done.
  // Rows beyond the context are zero (such keys are never read, such values must be zero).  Walking several tiles
  // per workgroup with the next keys in flight was measured and is no faster (32 lanes 10.03 against 9.82 ms).
  uint4 kr[8], vr[8];
  auto fetch = [&](uint4 (&dst)[8], const uint16_t* src) __attribute__((always_inline)) {
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int row = it * 8 + (tid >> 5), c8 = (tid & 31) * 8;
      dst[it] = make_uint4(0, 0, 0, 0);
      if (row < nk) dst[it] = ld16(src + (size_t)(tile * SDPA_TILE + row) * 256 + c8);
    }
  };
  fetch(kr, kc);
  fetch(vr, vc);
  {
    const int idx = tid * 8;                         // 0..2047 step 8: the group's 8 scaled queries; wave w then owns heads 2w, 2w+1
    float f[8];
    unpack8(ld16(a.qrot + ((size_t)m * 16 + kvh * 8) * 256 + idx), f);
#pragma unroll
    for (int i = 0; i < 8; ++i) s_q[idx + i] = 0.0625f * f[i];
  }
  const float NEG = -__int_as_float(0x7f800000);
  const int h0 = 2 * wave;
#pragma unroll
  for (int it = 0; it < 8; ++it) st16(&s_k[(it * 8 + (tid >> 5)) * KT_STRIDE + (tid & 31) * 8], kr[it]);
  __syncthreads();
  // scores: eight fmaf chains over 32 dims each (the staged key row is read in step with its use, the queries come
  // as LDS broadcasts), combined by a balanced tree
  float sc[2];
  {
    // (the sixteen chains of a lane advance side by side, four dims at a time: a chain on its own would wait for
    // every multiply-add before it)
    float c[2][8];
#pragma unroll
    for (int g = 0; g < 8; ++g) { c[0][g] = 0.0f; c[1][g] = 0.0f; }
    const uint16_t* krow = &s_k[(lane < nk ? lane : 0) * KT_STRIDE];
#pragma unroll
    for (int gh = 0; gh < 8; gh += 4) {                // four chains (times two heads) at a time
#pragma unroll
      for (int l = 0; l < 8; ++l) {
#pragma unroll
        for (int g = gh; g < gh + 4; ++g) {
          const int d = 32 * g + 4 * l;
          const uint2 kraw = *reinterpret_cast<const uint2*>(krow + d);
          const h2_t k01 = as_h2(kraw.x), k23 = as_h2(kraw.y);
#pragma unroll
          for (int h = 0; h < 2; ++h) {
            const float4 q4 = *reinterpret_cast<const float4*>(&s_q[(h0 + h) * 256 + d]);
            c[h][g] = fmaf(q4.x, (float)k01.x, c[h][g]);
            c[h][g] = fmaf(q4.y, (float)k01.y, c[h][g]);
            c[h][g] = fmaf(q4.z, (float)k23.x, c[h][g]);
            c[h][g] = fmaf(q4.w, (float)k23.y, c[h][g]);
          }
        }
        // (the chains' values are pinned here and the LDS reads of later steps stay behind: left to itself the
        //  scheduler hoists every read of the unrolled loops and spills)
        asm volatile("" : "+v"(c[0][gh]), "+v"(c[0][gh + 1]), "+v"(c[0][gh + 2]), "+v"(c[0][gh + 3]),
                          "+v"(c[1][gh]), "+v"(c[1][gh + 1]), "+v"(c[1][gh + 2]), "+v"(c[1][gh + 3]) : : "memory");
      }
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float t = ((c[h][0] + c[h][1]) + (c[h][2] + c[h][3])) + ((c[h][4] + c[h][5]) + (c[h][6] + c[h][7]));
      sc[h] = (lane < nk) ? t : NEG;
    }
  }
  float p[2], o[2][4];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const float mx = tree_max<64>(sc[h]);
    p[h] = (lane < nk) ? exp_c(sc[h] - mx) : 0.0f;
    const float l = tree_sum<64>(p[h]);
    if (lane == 0) {
      const size_t pi = ((size_t)m * 16 + kvh * 8 + h0 + h) * a.maxTiles + tile;
      a.pm[pi] = mx; a.pl[pi] = l;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) o[h][i] = 0.0f;
  }
  // Weighted value sums: one chain of fmaf over the tile's first 32 keys in order, one over its other 32, added at
  // the end.  All 64 keys are walked: beyond nk the weight and the parked value are zero, and fmaf(0, 0, o) returns o
  // as it is.  Eight keys at a time: their weights come over as scalars (lane reads), their value pieces from LDS.
  __syncthreads();                                   // every wave is done with the keys
  uint16_t* s_v = s_k;                               // [64][256] halves
#pragma unroll
  for (int it = 0; it < 8; ++it) st16(&s_v[(it * 8 + (tid >> 5)) * 256 + (tid & 31) * 8], vr[it]);
  __syncthreads();
  float oa[2][4];
#pragma unroll
  for (int j0v = 0; j0v < SDPA_TILE; j0v += 8) {
    if (j0v == SDPA_TILE / 2) {                        // the first half's chain is complete: the second starts from zero
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i) { oa[h][i] = o[h][i]; o[h][i] = 0.0f; }
    }
    uint2 vraw[8];
    float pj[2][8];
#pragma unroll
    for (int u = 0; u < 8; ++u) vraw[u] = *reinterpret_cast<const uint2*>(&s_v[(j0v + u) * 256 + 4 * lane]);
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int u = 0; u < 8; ++u) pj[h][u] = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(p[h]), j0v + u));
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const float vf[4] = {lo_h(vraw[u].x), hi_h(vraw[u].x), lo_h(vraw[u].y), hi_h(vraw[u].y)};
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[h][i] = fmaf(pj[h][u], vf[i], o[h][i]);
    }
  }
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const size_t pi = ((size_t)m * 16 + kvh * 8 + h0 + h) * a.maxTiles + tile;
    *reinterpret_cast<float4*>(a.po + pi * 256 + 4 * lane) =
        make_float4(oa[h][0] + o[h][0], oa[h][1] + o[h][1], oa[h][2] + o[h][2], oa[h][3] + o[h][3]);
  }
}

// Merge pass + output gate: tiles combined in order with the global max, out = half(O/L),
// gated = out * sigmoid16(gate) with the gate half of the q projection (sigmoid_mul,
// SeedlessMetalForward.swift:1012-1022).
struct SdpaMergeArgs {
  const float *pm, *pl, *po;
  const uint16_t* proj;        // gate at [m, h*512 + 256 + d]
  const int32_t* st;
  int maxTiles;
  uint16_t* gated;             // [M, 4096]
  float* gsum;                 // [M, 128] share sums of the gated rows for the projection that follows (k_sdpa_merge), or null
  const LaneRef* lanes;
  int group = 0;               // > 1: one partial per `group` key tiles at index tile / group (k_sdpa_merge_par only)
};
// The same merge for few rows and long contexts (decode steps, lane batches, verify rows): one workgroup of 16 waves
// per (head, row).  The chains over the tiles stay what they are -- in tile order, one fmaf per tile and element --
// but the work around them is spread: twelve waves fetch the tiles' partial sums a block of 64 tiles ahead and park
// them in LDS, the scale of a tile, exp(max_t - max), is formed once per tile (lane = tile) instead of once per lane
// and tile, and four waves carry the chains, 64 of the head's 256 dims each (every one of them also carries the chain
// of the sums, so that none has to wait for another).  One barrier per block (of the kind that leaves loads in flight).
constexpr int MERGE_BLOCK = 64;
constexpr int MERGE_DYN_LDS = 2 * MERGE_BLOCK * 256 * (int)sizeof(float);
__global__ __launch_bounds__(1024) void k_sdpa_merge_long(SdpaMergeArgs a) {
  extern __shared__ __align__(16) float s_park[];          // [2][MERGE_BLOCK tiles][256 dims]
  const int h = blockIdx.x, m = blockIdx.y, tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int N = a.lanes ? a.lanes[m].st[0] + 1 : a.st[0] + m + 1;
  const int nt = (N + SDPA_TILE - 1) / SDPA_TILE, nb = (nt + MERGE_BLOCK - 1) / MERGE_BLOCK;
  const size_t base = ((size_t)m * 16 + h) * a.maxTiles;
  const float NEG = -__int_as_float(0x7f800000);
  if (wave >= 4) {
    // tiles i = (wave - 4) + 12 j of a block, j = 0..5; two register sets take turns, a set is parked and at once
    // requested again for the block after the next (indices clamped into the context: every load is unconditional)
    constexpr int PER = 6;
    typedef float f32x4_t __attribute__((ext_vector_type(4)));       // (a native vector: arrays of HIP's float4 ended up in scratch memory here)
    f32x4_t qa[PER], qb[PER];
    auto request = [&](f32x4_t (&dst)[PER], int blk) __attribute__((always_inline)) {
#pragma unroll
      for (int j = 0; j < PER; ++j) {
        const int t = min(MERGE_BLOCK * min(blk, nb - 1) + min((wave - 4) + 12 * j, MERGE_BLOCK - 1), nt - 1);
        dst[j] = *reinterpret_cast<const f32x4_t*>(a.po + (base + t) * 256 + 4 * lane);
      }
    };
    auto park = [&](const f32x4_t (&src)[PER], int blk) __attribute__((always_inline)) {
      float* const dst = s_park + (size_t)(blk & 1) * MERGE_BLOCK * 256;
#pragma unroll
      for (int j = 0; j < PER; ++j) {
        const int i = (wave - 4) + 12 * j;
        if (i < MERGE_BLOCK) *reinterpret_cast<f32x4_t*>(dst + i * 256 + 4 * lane) = src[j];
      }
    };
    request(qa, 0);
    request(qb, 1);
    for (int k = 0; k <= nb; k += 2) {
      if (k < nb) { park(qa, k); request(qa, k + 2); }
      lds_barrier();
      if (k + 1 <= nb) {
        if (k + 1 < nb) { park(qb, k + 1); request(qb, k + 3); }
        lds_barrier();
      }
    }
    return;
  }
  // waves 0..3: the chains.  Lane i of a block holds tile i's maximum and sum; the global maximum first.
  float Mx = NEG;
  for (int t = lane; t < nt; t += 64) Mx = fmaxf(Mx, a.pm[base + t]);
  Mx = tree_max<64>(Mx);
  const int d = 64 * wave + lane;
  const uint16_t graw = a.proj[(size_t)m * PROJ_STRIDE + h * 512 + 256 + d];
  float L = 0.0f, O = 0.0f, La = 0.0f, Oa = 0.0f;         // the block's chains (from zero), the sum of the blocks before
  float pmv = a.pm[base + min(lane, nt - 1)], plv = a.pl[base + min(lane, nt - 1)];
  for (int k = 0; k <= nb; ++k) {
    if (k >= 1) {
      const int kb = k - 1, t0 = MERGE_BLOCK * kb, cnt = min(MERGE_BLOCK, nt - t0);
      if (kb == 1) { La = L; Oa = O; } else if (kb > 1) { La = La + L; Oa = Oa + O; }
      if (kb >= 1) { L = 0.0f; O = 0.0f; }
      const float fl = (lane < cnt) ? exp_c(pmv - Mx) : 0.0f, pl = (lane < cnt) ? plv : 0.0f;
      if (k < nb) { pmv = a.pm[base + min(t0 + MERGE_BLOCK + lane, nt - 1)]; plv = a.pl[base + min(t0 + MERGE_BLOCK + lane, nt - 1)]; }
      const float* const src = s_park + (size_t)(kb & 1) * MERGE_BLOCK * 256 + d;
      int u0 = 0;
      for (; u0 + 8 <= cnt; u0 += 8) {                 // eight tiles at a time: their scales and sums as scalars, their values from LDS
        float f[8], l[8], o[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = src[(u0 + i) * 256];
        lanes8(fl, u0, f);
        lanes8(pl, u0, l);
#pragma unroll
        for (int i = 0; i < 8; ++i) { L = fmaf(l[i], f[i], L); O = fmaf(o[i], f[i], O); }
      }
      for (; u0 < cnt; ++u0) {
        const float f = row_lane_f(fl, u0), l = row_lane_f(pl, u0);
        L = fmaf(l, f, L); O = fmaf(src[u0 * 256], f, O);
      }
    }
    lds_barrier();
  }
  if (nb > 1) { L = La + L; O = Oa + O; }
  const float r = f16r(f16r(O / L) * sigmoid16(h2f(graw)));
  a.gated[(size_t)m * 4096 + h * 256 + d] = f2h(r);
  if (a.gsum) {                                          // a share of 32 values sits on 32 neighbouring lanes
    const float sw = tree_sum<32>(r);
    if ((lane & 31) == 0) a.gsum[(size_t)m * 128 + h * 8 + (d >> 5)] = sw;
  }
}
// The same merge with the blocks' chains side by side: the chain of a block of 64 tiles starts from zero and the
// blocks' chains are added in block order, so the blocks are independent until that last addition.  One workgroup of
// four waves per (head, row, quarter of the head's dims): lane = dim, wave w takes blocks w, w + 4, ... -- the 64
// partial sums of a block are 64 loads per lane in flight at once (one round trip per block instead of one per
// sixteen tiles), the next block of the wave already requested while this one is added up -- and after every group
// of four blocks wave 0 adds their chains in block order.  For steps of a few rows at long contexts, where the
// 16 x M workgroups of the other kernels leave most of the machine idle and walk the tiles one round trip after another.
constexpr int MERGE_BLOCKS_WAVES = 4;
__global__ __launch_bounds__(64 * MERGE_BLOCKS_WAVES) void k_sdpa_merge_blocks(SdpaMergeArgs a) {
  constexpr int W = MERGE_BLOCKS_WAVES;
  __shared__ float s_o[2][W][64];
  __shared__ float s_l[2][W];
  const int h = blockIdx.x, m = blockIdx.y, q = blockIdx.z, tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int N = a.lanes ? a.lanes[m].st[0] + 1 : a.st[0] + m + 1;
  const int nt = (N + SDPA_TILE - 1) / SDPA_TILE, nb = (nt + MERGE_BLOCK - 1) / MERGE_BLOCK;
  const size_t base = ((size_t)m * 16 + h) * a.maxTiles;
  const int d = 64 * q + lane;
  const float* const po = a.po + base * 256 + d;
  float v[MERGE_BLOCK], vn[MERGE_BLOCK];
  auto request = [&](float (&dst)[MERGE_BLOCK], int b) __attribute__((always_inline)) {
    const int t0 = MERGE_BLOCK * b;                        // (tiles beyond the context repeat its last tile and are not used)
#pragma unroll
    for (int i = 0; i < MERGE_BLOCK; ++i) dst[i] = po[(size_t)min(t0 + i, nt - 1) * 256];
  };
  if (wave < nb) request(v, wave);
  // lane i: {max, sum} of tile i of the wave's block (requested with the block, ahead of the maximum over all tiles)
  auto tile_ml = [&](int b, float& pm, float& pl) __attribute__((always_inline)) {
    const size_t i = base + min(MERGE_BLOCK * min(b, nb - 1) + lane, nt - 1);
    pm = a.pm[i]; pl = a.pl[i];
  };
  float pmv, plv, pmn = 0.0f, pln = 0.0f;
  tile_ml(wave, pmv, plv);
  float Mx = -__int_as_float(0x7f800000);
  for (int t = lane; t < nt; t += 64) Mx = fmaxf(Mx, a.pm[base + t]);
  Mx = tree_max<64>(Mx);
  const uint16_t graw = a.proj[(size_t)m * PROJ_STRIDE + h * 512 + 256 + d];
  float L = 0.0f, O = 0.0f;                                // wave 0: the blocks' chains added up so far
  for (int g0 = 0, k = 0; g0 < nb; g0 += W, k ^= 1) {
    const int b = g0 + wave;
    if (b < nb) {
      const int t0 = MERGE_BLOCK * b, cnt = min(MERGE_BLOCK, nt - t0);
      if (b + W < nb) { request(vn, b + W); tile_ml(b + W, pmn, pln); }
      const float fl = (lane < cnt) ? exp_c(pmv - Mx) : 0.0f, pl = (lane < cnt) ? plv : 0.0f;
      float Lb = 0.0f, Ob = 0.0f;
#pragma unroll
      for (int u0 = 0; u0 < MERGE_BLOCK; u0 += 8) {
        if (u0 < cnt) {                                    // uniform for the wave
          float f[8], l[8];
          lanes8(fl, u0, f);
          lanes8(pl, u0, l);
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (u0 + i < cnt) { Lb = fmaf(l[i], f[i], Lb); Ob = fmaf(v[u0 + i], f[i], Ob); }
        }
      }
      s_o[k][wave][lane] = Ob;
      if (lane == 0) s_l[k][wave] = Lb;
#pragma unroll
      for (int i = 0; i < MERGE_BLOCK; ++i) v[i] = vn[i];
      pmv = pmn; plv = pln;
    }
    __syncthreads();                                       // (the other buffer is written next: one barrier per group)
    if (wave == 0) {
      for (int w = 0; w < W && g0 + w < nb; ++w) {
        const float ob = s_o[k][w][lane], lb = s_l[k][w];
        if (g0 + w == 0) { O = ob; L = lb; } else { O = O + ob; L = L + lb; }
      }
    }
  }
  if (wave != 0) return;
  const float r = f16r(f16r(O / L) * sigmoid16(h2f(graw)));
  a.gated[(size_t)m * 4096 + h * 256 + d] = f2h(r);
  if (a.gsum) {                                            // a share of 32 values sits on 32 neighbouring lanes
    const float sw = tree_sum<32>(r);
    if ((lane & 31) == 0) a.gsum[(size_t)m * 128 + h * 8 + (d >> 5)] = sw;
  }
}
__global__ __launch_bounds__(64) void k_sdpa_merge(SdpaMergeArgs a) {
  const int h = blockIdx.x, m = blockIdx.y, lane = threadIdx.x;
  const int N = a.lanes ? a.lanes[m].st[0] + 1 : a.st[0] + m + 1;
  const int nt = (N + SDPA_TILE - 1) / SDPA_TILE;
  const size_t base = ((size_t)m * 16 + h) * a.maxTiles;
  float Mx = -__int_as_float(0x7f800000);
  for (int t = lane; t < nt; t += 64) Mx = fmaxf(Mx, a.pm[base + t]);
  Mx = tree_max<64>(Mx);
  // tiles are added up in order; sixteen tiles' partials are requested together (one memory round trip per sixteen tiles)
  // (a chain per block of 64 tiles, the blocks' chains added in block order)
  float L = 0.0f, O[4] = {0.0f, 0.0f, 0.0f, 0.0f}, La = 0.0f, Oa[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int t0 = 0; t0 < nt; t0 += 16) {
    if (t0 >= MERGE_BLOCK && t0 % MERGE_BLOCK == 0) {
      const bool first = t0 == MERGE_BLOCK;
      La = first ? L : La + L; L = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; ++i) { Oa[i] = first ? O[i] : Oa[i] + O[i]; O[i] = 0.0f; }
    }
    float4 o[16];
    float pmv[16], plv[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const size_t pi = base + min(t0 + u, nt - 1);
      o[u] = *reinterpret_cast<const float4*>(a.po + pi * 256 + 4 * lane);
      pmv[u] = a.pm[pi]; plv[u] = a.pl[pi];
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      if (t0 + u < nt) {
        const float f = exp_c(pmv[u] - Mx);
        L = fmaf(plv[u], f, L);
        O[0] = fmaf(o[u].x, f, O[0]); O[1] = fmaf(o[u].y, f, O[1]); O[2] = fmaf(o[u].z, f, O[2]); O[3] = fmaf(o[u].w, f, O[3]);
      }
    }
  }
  if (nt > MERGE_BLOCK) {
    L = La + L;
#pragma unroll
    for (int i = 0; i < 4; ++i) O[i] = Oa[i] + O[i];
  }
  const uint2 graw = *reinterpret_cast<const uint2*>(a.proj + (size_t)m * PROJ_STRIDE + h * 512 + 256 + 4 * lane);
  const float gt[4] = {lo_h(graw.x), hi_h(graw.x), lo_h(graw.y), hi_h(graw.y)};
  float r[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = f16r(f16r(O[i] / L) * sigmoid16(gt[i]));
  *reinterpret_cast<uint2*>(a.gated + (size_t)m * 4096 + h * 256 + 4 * lane) = make_uint2(pack2(r[0], r[1]), pack2(r[2], r[3]));
  if (a.gsum) {                                          // a share of 32 values sits on eight neighbouring lanes
    const float sw = tree_sum<8>((r[0] + r[1]) + (r[2] + r[3]));
    if ((lane & 7) == 0) a.gsum[(size_t)m * 128 + h * 8 + (lane >> 3)] = sw;
  }
}

// -------------------------------------------------------------------------------------------------
// Head: residual + final norm + lm_head with the arg-max folded into the epilogue.  Each
// workgroup stores its 16 logits and one (value, index) candidate; k_argmax_final picks the
// first maximum.  References: SeedlessFusedVerify.swift:3855-3876, argmax_rows :572-596.
// -------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void k_head(HiddenArgs ha, const uint32_t* __restrict__ W,
                                              const uint32_t* __restrict__ SB, int V, uint16_t* __restrict__ logits,
                                              float* __restrict__ cand_v, int32_t* __restrict__ cand_i) {
  __shared__ float s_v[4];
  __shared__ int s_i[4];
  const int m = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float x[32], sx[1];
  hidden_prologue(ha, m, lane, blockIdx.x == 0 && wave == 0, x);
  sx[0] = share_sum(x);
  uint32_t xp[16];
  pack_x(x, xp);
  const size_t row0 = ((size_t)blockIdx.x * 4 + wave) * 4;
  float bv = -__int_as_float(0x7f800000);
  int bi = 0x7fffffff;
  if (row0 < (size_t)V) {
    const size_t rows[4] = {row0, row0 + 1, row0 + 2, row0 + 3};
    float out[4];
    qdot_rows<1, 4>(W, SB, rows, lane, xp, sx, out);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float v = f16r(out[r]);
      if (v > bv) { bv = v; bi = (int)(row0 + r); }
    }
    if (lane == 0) {
      const uint2 pk = make_uint2(pack2(out[0], out[1]), pack2(out[2], out[3]));
      *reinterpret_cast<uint2*>(logits + (size_t)m * V + row0) = pk;
    }
  }
  if (lane == 0) { s_v[wave] = bv; s_i[wave] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 1; w < 4; ++w) if (s_v[w] > bv) { bv = s_v[w]; bi = s_i[w]; }
    cand_v[(size_t)m * gridDim.x + blockIdx.x] = bv;
    cand_i[(size_t)m * gridDim.x + blockIdx.x] = bi;
  }
}
__global__ __launch_bounds__(256) void k_argmax_final(const float* __restrict__ cand_v, const int32_t* __restrict__ cand_i,
                                                      int ncand, int32_t* __restrict__ tok_out, int out_off,
                                                      int32_t* __restrict__ feed) {
  __shared__ float s_v[256];
  __shared__ int s_i[256];
  const int m = blockIdx.x, tid = threadIdx.x;
  float bv = -__int_as_float(0x7f800000);
  int bi = 0x7fffffff;
  for (int c = tid; c < ncand; c += 256) {
    const float v = cand_v[(size_t)m * ncand + c];
    const int i = cand_i[(size_t)m * ncand + c];
    if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
  }
  s_v[tid] = bv; s_i[tid] = bi;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if (tid < s) {
      const float ov = s_v[tid + s]; const int oi = s_i[tid + s];
      if (ov > s_v[tid] || (ov == s_v[tid] && oi < s_i[tid])) { s_v[tid] = ov; s_i[tid] = oi; }
    }
    __syncthreads();
  }
  if (tid == 0) {
    tok_out[out_off + m] = s_i[0];
    if (feed) feed[0] = s_i[0];
  }
}

// Residual + optional final norm, rows out (forwardRows, SeedlessFusedVerify.swift:3641-3660).
__global__ __launch_bounds__(64) void k_final_rows(HiddenArgs ha) {
  float x[32];
  hidden_prologue(ha, blockIdx.x, threadIdx.x, true, x);
}

// Step state st = {position, parity[0..n_layers)}: the position advances by M and every layer's
// ping-pong side flips (attention layers ignore theirs).
__global__ void k_advance(int32_t* st, int M, int n_layers) {
  const int t = threadIdx.x;
  if (t == 0) st[0] += M;
  for (int i = t; i < n_layers; i += blockDim.x) st[1 + i] ^= 1;
}
// The same for every lane of a lane-batched step (one token each); blockIdx.x = lane.
__global__ void k_lane_advance(const LaneRef* lanes, int n_layers) {
  int32_t* st = lanes[blockIdx.x].st;
  const int t = threadIdx.x;
  if (t == 0) st[0] += 1;
  for (int i = t; i < n_layers; i += blockDim.x) st[1 + i] ^= 1;
}
// {scale, bias} interleave: the engine keeps one 32-bit pair per quantisation group.
__global__ __launch_bounds__(256) void k_pack_sb(const uint16_t* __restrict__ s, const uint16_t* __restrict__ b,
                                                 uint32_t* __restrict__ out, size_t n) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = (uint32_t)s[i] | ((uint32_t)b[i] << 16);
}

}  // namespace sl
