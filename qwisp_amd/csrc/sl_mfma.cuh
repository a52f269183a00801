// Matrix-core GEMM with 4-bit dequantisation for rows of a prefill chunk ("hybrid" prefill; the reference runs
// these projections on the matrix units as well and documents them as not bit-identical to its GEMV path,
// SeedlessFusedVerify.swift:4240-4247).
//
//   Y[m, n] = half( sum_k X[m, k] * half(s * q + b) ),  X fp16 [M, K], W MLX-affine 4-bit group 64 [N, K],
//   the weight formed in half arithmetic (one fused multiply-add), fp32 accumulation in v_mfma_f32_32x32x16_f16.
//
// A wave owns 32x32 tiles of Y (32 rows of X against a strip of 32 weight rows): it walks K in chunks of 64 (one
// quantisation group), dequantises its 8 weights per MFMA step in registers and feeds them as the B operand;
// the X chunk [rows, 64] is staged in LDS by the whole workgroup (double-buffered, one barrier per chunk) and
// read as the A operand.  A row's result depends only on that row of X and on W, and K is walked in a fixed
// order, so the result is independent of M and of the chunking of a prompt.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sl_kernels.cuh"

namespace sl {

typedef float mf_f16v __attribute__((ext_vector_type(16)));
typedef _Float16 mf_h2 __attribute__((ext_vector_type(2)));

// The 8 halves of a staged 16-byte piece (k = 8j .. 8j+7) in the order {0,4,1,5, 2,6,3,7}, the order in which
// dequant8 delivers the 8 nibbles of a packed word.
SL_DEV uint4 permute8(uint4 v) {
  // v_perm_b32 picks bytes out of {first operand: bytes 4..7, second operand: bytes 0..3}
  return make_uint4(__builtin_amdgcn_perm(v.z, v.x, 0x05040100u), __builtin_amdgcn_perm(v.z, v.x, 0x07060302u),
                    __builtin_amdgcn_perm(v.w, v.y, 0x05040100u), __builtin_amdgcn_perm(v.w, v.y, 0x07060302u));
}

struct QmmArgs {
  const uint16_t* x;     // [M, x_stride] fp16
  int x_stride;
  const uint32_t* W;     // [N, K/8] packed
  const uint32_t* SB;    // [N, K/64] {scale, bias}
  int M, N, K;           // N % 32 == 0, K % 64 == 0
  uint16_t* y;           // [M, y_stride] fp16
  int y_stride;
  // optional second matrix of the same shape against the same X (grid.z = 2: blockIdx.z picks the matrix), e.g. the
  // shared expert's gate_proj and up_proj, which alone would fill a quarter of the machine each
  const uint32_t* W2 = nullptr;
  const uint32_t* SB2 = nullptr;
  uint16_t* y2 = nullptr;
  int col_blocks = 0, row_blocks = 0;   // tiles of the launch (set by launch_qmm4_mfma), see xcd_tile
};

// Which tile a workgroup takes.  Workgroups go to the 8 XCDs in turn (workgroup n runs on XCD n % 8) and every XCD has
// an L2 of its own, so the tiles are dealt out by XCD: an XCD owns the row blocks x, x + 8, ... and sweeps the column
// blocks with them, innermost over its row blocks.  The X rows of its few row blocks then stay in that L2 for the
// whole sweep and a strip of weights is used by all its row blocks while it is hot, instead of every XCD pulling
// every block of X through its own L2.  With fewer than 8 row blocks the XCDs that share a row block split the
// column blocks among them.
struct TileId { int col_block, row_block; bool valid; };
SL_DEV TileId xcd_tile(int n, int col_blocks, int row_blocks) {
  const int x = n & 7, s = n >> 3;
  TileId t;
  if (row_blocks >= 8) {
    const int per = (row_blocks + 7) >> 3;
    t.row_block = x + 8 * (s % per);
    t.col_block = s / per;
  } else {
    t.row_block = x % row_blocks;
    const int part = x / row_blocks, sharers = (8 - t.row_block + row_blocks - 1) / row_blocks;
    t.col_block = s * sharers + part;
  }
  t.valid = t.row_block < row_blocks && t.col_block < col_blocks;
  return t;
}
inline unsigned xcd_tile_grid(int col_blocks, int row_blocks) {   // workgroups to launch for xcd_tile
  if (row_blocks >= 8) return 8u * (unsigned)(((row_blocks + 7) / 8) * col_blocks);
  const int sharers_min = 8 / row_blocks;
  return 8u * (unsigned)((col_blocks + sharers_min - 1) / sharers_min);
}


// -------------------------------------------------------------------------------------------------
// The dense projections of a chunk: v_mfma_f32_32x32x16_f16, RT row tiles per wave.  A wave owns a strip of 32
// weight rows and RT x 32 rows of X (RT accumulators): it dequantises the 8 weights of a step once and feeds them
// to RT matrix instructions, so the unpacking is shared by up to 128 rows of X; the four waves of a workgroup take
// four neighbouring strips and read the same staged X chunk.  Grid (ceil(N / 128), ceil(M / (32*RT))).
// Operands of a step (16 values of k): lane (col, hh) brings the 8 values of one packed word of its row (A) / weight
// row (B) -- word st of the 64-k group on the lower half-wave, word 4+st on the upper, so that a lane fetches its four
// words of a group with one 16-byte load; the order within the eight is {0,4,1,5,2,6,3,7} on both sides.
// -------------------------------------------------------------------------------------------------
// Dequantisation of a packed word (8 weights) in packed half arithmetic.  Masking with 0x000F000F leaves the nibbles
// j and j+4 at the bottom of the two halves; or-ing a nibble into the mantissa of 1024.0 gives 1024 + q exactly and
// subtracting 1024 gives q exactly.  Masking with 0x00F000F0 instead takes the nibbles one place up without a shift:
// or-ed into 1024.0 they read 1024 + 16 q, and (1024 + 16 q) / 16 - 64 = q, again exact, is one fused multiply-add.
// So a word costs one shift (by 8, for its upper two pairs) instead of three.  half(q * s + b) is one more fused
// multiply-add per pair.  `k1024` is the pattern 0x64006400 held in a vector register, so that mask and or are one
// instruction (v_and_or_b32 takes one literal).
typedef _Float16 mf_h8 __attribute__((ext_vector_type(8)));
SL_DEV uint32_t dequant_k1024() {
  uint32_t k = 0x64006400u;
  asm volatile("" : "+v"(k));
  return k;
}
SL_DEV mf_h2 dequant_pair(uint32_t w, int j, mf_h2 s2, mf_h2 b2, uint32_t k1024) {   // nibbles j and j+4
  const mf_h2 f1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
  const mf_h2 sixteenth = {(_Float16)0.0625f, (_Float16)0.0625f}, m64 = {(_Float16)-64.0f, (_Float16)-64.0f};
  const uint32_t src = (j & 2) ? (w >> 8) : w;
  mf_h2 q;
  if (j & 1) q = __builtin_elementwise_fma(__builtin_bit_cast(mf_h2, (src & 0x00F000F0u) | k1024), sixteenth, m64);
  else q = __builtin_bit_cast(mf_h2, (src & 0x000F000Fu) | k1024) - f1024;
  return __builtin_elementwise_fma(q, s2, b2);
}
SL_DEV mf_h8 dequant8(uint32_t w, mf_h2 s2, mf_h2 b2, uint32_t k1024) {
  mf_h8 r;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const mf_h2 v = dequant_pair(w, j, s2, b2, k1024);
    r[2 * j] = v[0]; r[2 * j + 1] = v[1];
  }
  return r;
}
// The rows of a chunk on their way global -> registers -> LDS: ROWS rows x G groups x 8 pieces of 16 bytes, dealt out
// to the NT threads of the workgroup in passes (piece index = pass * NT + thread; pieces past the end repeat the
// last one, harmlessly).  `row_offset(row)` gives the element offset of a row of the tile in X.
template <int ROWS, int G, int NT>
struct RowStager {
  static constexpr int XS = 64 * G + 8;                  // halves per staged row (rows 16 bytes off a multiple of 128)
  static constexpr int TOTAL = ROWS * G * 8, PASSES = (TOTAL + NT - 1) / NT;
  uint32_t src[PASSES];                                  // element offset in X of the thread's piece within chunk 0
  uint32_t dst[PASSES];                                  // halves offset in a staging buffer
  uint4 r[PASSES];
  template <typename F>
  SL_DEV void init(int tid, F row_offset) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      const int idx = min(p * NT + tid, TOTAL - 1);
      const int piece = idx & 7, row = (idx >> 3) % ROWS, g = (idx >> 3) / ROWS;
      src[p] = row_offset(row) + (uint32_t)(g * 64 + piece * 8);
      dst[p] = (uint32_t)(row * XS + g * 64 + piece * 8);
    }
  }
  SL_DEV void fetch(const uint16_t* x, int c) {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) r[p] = ld16(x + (size_t)(src[p] + (uint32_t)(c * G * 64)));
  }
  SL_DEV void put(uint16_t* buf) const {
#pragma unroll
    for (int p = 0; p < PASSES; ++p) st16(buf + dst[p], permute8(r[p]));
  }
};

// A SIMD issues one instruction at a time: unpacking, LDS reads and staging all take issue slots next to the matrix
// instructions instead of hiding behind them, so the kernel's speed is set by the instructions per matrix
// instruction.  A wave therefore owns NS strips of 32 weight rows and RT x 32 rows of X (RT x NS accumulators): a row
// operand read from LDS feeds NS matrix instructions, an unpacked weight operand RT, and the staged rows are shared
// by the WPB waves of the workgroup.
template <int RT, int NS, int G, int WPB>      // G quantisation groups (64 k) per staged chunk and barrier; K % (64*G) == 0
__global__ __launch_bounds__(64 * WPB) void k_qmm4_mfma16(QmmArgs a) {
  constexpr int NT = 64 * WPB;
  using Stage = RowStager<RT * 32, G, NT>;
  constexpr int XS = Stage::XS;
  __shared__ __align__(16) uint16_t xs[2][RT * 32 * XS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, hh = lane >> 5;
  const TileId tile = xcd_tile((int)blockIdx.x, a.col_blocks, a.row_blocks);
  if (!tile.valid) return;                               // uniform for the workgroup
  const int n0 = (tile.col_block * WPB + wave) * NS * 32;  // first of the wave's NS neighbouring strips
  const int m0 = tile.row_block * RT * 32;
  const int chunks = a.K / (64 * G);
  const bool second = blockIdx.z != 0;
  const uint32_t* wp[NS];
  const uint32_t* sp[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {                         // (a strip beyond N works on strip 0 and stores nothing)
    const size_t wrow = (size_t)(n0 + 32 * s < a.N ? n0 + 32 * s + col : 0);
    wp[s] = (second ? a.W2 : a.W) + wrow * (a.K / 8);
    sp[s] = (second ? a.SB2 : a.SB) + wrow * (a.K / 64);
  }
  uint16_t* yout = second ? a.y2 : a.y;
  mf_f16v acc[RT][NS];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][s][r] = 0.0f;
  // Rows beyond M repeat row M-1: a row of Y depends on its own row of X only and those rows of Y are never stored,
  // so the loads need no bounds branch.
  Stage stage;
  stage.init(tid, [&](int row) { return (uint32_t)min(m0 + row, a.M - 1) * (uint32_t)a.x_stride; });
  // of a group's 8 packed words the lower half-wave takes words 0..3 and the upper 4..7 (one 16-byte load each):
  // step st multiplies the k of word st (lower) and of word 4+st (upper), on the A side as well
  uint4 nw[NS][G];
  uint32_t nsb[NS][G];
  auto wfetch = [&](int c) {
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int g = 0; g < G; ++g) {
        nw[s][g] = ld16(wp[s] + (c * G + g) * 8 + 4 * hh);
        nsb[s][g] = sp[s][c * G + g];
      }
  };
  stage.fetch(a.x, 0);
  stage.put(xs[0]);
  if (chunks > 1) stage.fetch(a.x, 1);
  wfetch(0);
  const uint32_t k1024 = dequant_k1024();
  for (int c = 0; c < chunks; ++c) {
    const int buf = c & 1;
    uint4 w[NS][G];
    uint32_t sb[NS][G];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int g = 0; g < G; ++g) { w[s][g] = nw[s][g]; sb[s][g] = nsb[s][g]; }
    if (c + 1 < chunks) wfetch(c + 1);                   // the weights of the next chunk are requested before this one is consumed
    __syncthreads();                                     // chunk c is staged; chunk c-1 is no longer read
    if (c + 1 < chunks) { stage.put(xs[buf ^ 1]); if (c + 2 < chunks) stage.fetch(a.x, c + 2); }
    // The chunk's G x 4 steps in one software pipeline: the pairs of the next step's weights are unpacked between
    // this step's matrix instructions (the scheduling fences keep that order) and the next step's rows are read from
    // LDS at the start of the step.
    constexpr int S = G * 4;
    auto word = [&](int s, int st) { const uint4 v = w[s][st >> 2]; return (st & 3) == 0 ? v.x : (st & 3) == 1 ? v.y : (st & 3) == 2 ? v.z : v.w; };
    auto scale = [&](int s, int st) { return __builtin_bit_cast(mf_h2, (sb[s][st >> 2] & 0xffffu) * 0x10001u); };
    auto bias = [&](int s, int st) { return __builtin_bit_cast(mf_h2, (sb[s][st >> 2] >> 16) * 0x10001u); };
    auto rows = [&](int st, int t) {
      return *reinterpret_cast<const mf_h8*>(&xs[buf][(t * 32 + col) * XS + (st >> 2) * 64 + 32 * hh + 8 * (st & 3)]);
    };
    mf_h8 bw[NS], ax[RT];
#pragma unroll
    for (int s = 0; s < NS; ++s) bw[s] = dequant8(word(s, 0), scale(s, 0), bias(s, 0), k1024);
#pragma unroll
    for (int t = 0; t < RT; ++t) ax[t] = rows(0, t);
#pragma unroll
    for (int st = 0; st < S; ++st) {
      mf_h8 axn[RT], bwn[NS];
      if (st + 1 < S) {
#pragma unroll
        for (int t = 0; t < RT; ++t) axn[t] = rows(st + 1, t);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int t = 0; t < RT; ++t) {
          acc[t][s] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ax[t], bw[s], acc[t][s], 0, 0, 0);
          if (st + 1 < S) {                              // strip s's next word is unpacked behind strip s's products
#pragma unroll
            for (int j = 4 * t / RT; j < 4 * (t + 1) / RT; ++j) {
              const mf_h2 v = dequant_pair(word(s, st + 1), j, scale(s, st + 1), bias(s, st + 1), k1024);
              bwn[s][2 * j] = v[0]; bwn[s][2 * j + 1] = v[1];
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      if (st + 1 < S) {
#pragma unroll
        for (int s = 0; s < NS; ++s) bw[s] = bwn[s];
#pragma unroll
        for (int t = 0; t < RT; ++t) ax[t] = axn[t];
      }
    }
  }
  // D layout of a 32x32 tile: register r of lane (col, hh) holds row 8*(r/4) + 4*hh + r%4, column col.  Stored from
  // there a value is a two-byte store with an address of its own; where the workgroup's tile fits the staging space
  // (and rows of Y start on 16-byte boundaries) it is laid down in LDS [row][column] and goes out in 16-byte pieces.
  constexpr int TC = WPB * NS * 32, YS = TC + 8;         // columns of the workgroup's tile, halves per row in LDS
  if constexpr (RT * 32 * YS <= 2 * RT * 32 * XS) {
    if ((a.y_stride & 7) == 0 && (reinterpret_cast<uintptr_t>(yout) & 15) == 0) {     // uniform
      uint16_t* const ys = &xs[0][0];
      __syncthreads();                                   // the last chunk has been read
#pragma unroll
      for (int s = 0; s < NS; ++s)
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            ys[(t * 32 + 8 * (r >> 2) + 4 * hh + (r & 3)) * YS + (wave * NS + s) * 32 + col] = f2h(acc[t][s][r]);
      __syncthreads();
      const int nwg = tile.col_block * TC;
      constexpr int PPR = TC / 8, PIECES = RT * 32 * PPR;  // 16-byte pieces per row, per tile
#pragma unroll
      for (int p = 0; p < (PIECES + NT - 1) / NT; ++p) {
        const int idx = p * NT + tid, row = idx / PPR, piece = idx % PPR;
        if (idx < PIECES && m0 + row < a.M && nwg + piece * 8 < a.N)
          st16(yout + (size_t)(m0 + row) * a.y_stride + nwg + piece * 8, *reinterpret_cast<const uint4*>(&ys[row * YS + piece * 8]));
      }
      return;
    }
  }
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    if (n0 + 32 * s >= a.N) continue;
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + t * 32 + 8 * (r >> 2) + 4 * hh + (r & 3);
        if (m < a.M) yout[(size_t)m * a.y_stride + n0 + 32 * s + col] = f2h(acc[t][s][r]);
      }
  }
}

// -------------------------------------------------------------------------------------------------
// Router and shared-gate logits of a prefill chunk (hybrid mode): Y[m, n] = half(sum_k X[m, k] * W[n, k]) with fp16
// weights [N, K] (the router's 256 rows, row 256 = the shared expert's gate row, zero rows up to a multiple of 32).
// Same tiling and operand order as k_qmm4_mfma16 with one row tile per wave; the B operand is eight halves of the
// weight row itself.  Columns below 256 go to the router logits [M, 256], column 256 to the gate logits [M].
// -------------------------------------------------------------------------------------------------
struct RouterMmArgs {
  const uint16_t* x;     // [M, 2048] fp16 normed rows
  const uint16_t* W;     // [N, 2048] fp16, N % 32 == 0
  int M, N;
  uint16_t* rlogits;     // [M, 256]
  uint16_t* sgate;       // [M]
};
__global__ __launch_bounds__(256) void k_router_mfma(RouterMmArgs a) {
  constexpr int G = 4, XS = 64 * G + 8, K = 2048;        // 256 k per barrier: the launch is short of workgroups, so a chunk's round trips show
  __shared__ __align__(16) uint16_t xs[2][32 * XS];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 31, hh = lane >> 5;
  const int n0 = (blockIdx.x * 4 + wave) * 32;
  const int m0 = blockIdx.y * 32;
  const bool live = n0 < a.N;
  const uint16_t* wp = a.W + (size_t)(live ? n0 + col : 0) * K;
  constexpr int chunks = K / (64 * G);
  mf_f16v acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
  uint4 xr[G];
  auto fetch = [&](int c) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
      const int row = m0 + (tid >> 3);
      xr[g] = make_uint4(0, 0, 0, 0);
      if (row < a.M) xr[g] = ld16(a.x + (size_t)row * K + (c * G + g) * 64 + (tid & 7) * 8);
    }
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int g = 0; g < G; ++g) st16(&xs[buf][(tid >> 3) * XS + g * 64 + (tid & 7) * 8], permute8(xr[g]));
  };
  // a lane's weights of a 64-k group: the four 16-byte pieces k = 32 hh + 8 st .. + 7 (st = 0..3), the k order of the A side
  uint4 nw[G][4];
  auto wfetch = [&](int c) {
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int st = 0; st < 4; ++st) nw[g][st] = ld16(wp + (c * G + g) * 64 + 32 * hh + 8 * st);
  };
  fetch(0);
  put(0);
  if (chunks > 1) fetch(1);
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int st = 0; st < 4; ++st) nw[g][st] = make_uint4(0, 0, 0, 0);
  if (live) wfetch(0);
  for (int c = 0; c < chunks; ++c) {
    const int buf = c & 1;
    uint4 w[G][4];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int st = 0; st < 4; ++st) w[g][st] = nw[g][st];
    if (live && c + 1 < chunks) wfetch(c + 1);
    __syncthreads();
    if (c + 1 < chunks) { put(buf ^ 1); if (c + 2 < chunks) fetch(c + 2); }
    if (!live) continue;
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        const mf_h8 ax = *reinterpret_cast<const mf_h8*>(&xs[buf][col * XS + g * 64 + 32 * hh + 8 * st]);
        const mf_h8 bw = __builtin_bit_cast(mf_h8, permute8(w[g][st]));
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(ax, bw, acc, 0, 0, 0);
      }
  }
  if (!live) return;
  const int n = n0 + col;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int m = m0 + 8 * (r >> 2) + 4 * hh + (r & 3);
    if (m < a.M) {
      if (n < 256) a.rlogits[(size_t)m * 256 + n] = f2h(acc[r]);
      else if (n == 256) a.sgate[m] = f2h(acc[r]);
    }
  }
}

// -------------------------------------------------------------------------------------------------
// Routed experts of a prefill chunk, grouped by expert (reference: steelMoEGather,
// SeedlessFusedVerify.swift:4174): the (row, slot) pairs that chose expert e are gathered, multiplied with that
// expert's matrix once, and scattered back by pair.  Workgroup = (strip block, expert); experts nobody chose exit.
// -------------------------------------------------------------------------------------------------

struct QmmGroupArgs {
  const uint16_t* x;     // source rows, fp16
  int x_stride;
  int x_by_pair;         // 0: source row = token row (pair >> 3); 1: source row = pair index (m * 8 + slot)
  const uint32_t* W;     // [E * NE, K/8]: expert e owns rows e*NE .. e*NE + NE - 1
  const uint32_t* SB;    // [E * NE, K/64]
  const uint32_t *W2, *SB2;  // second matrix of the dual form (else unused)
  int NE, K;
  const uint16_t* lists; // [E, GROUP_CAP] pair indices
  const int32_t* counts; // [E]
  const int32_t* order;  // [E] experts by falling count: blockIdx.y walks this order
  uint16_t* y;           // [pairs, y_stride]
  int y_stride;
};

// DUAL: two weight matrices of the same shape against the same rows (the experts' gate_proj and up_proj): one
// staging of X, two weight streams in flight per wave, and y = half(silu(g) * u) of the two rounded results
// written directly (the SwiGLU of the GEMV path, swiglu16).
// A pass multiplies RT tiles of 32 gathered rows with the expert's weights, so that a dequantised operand feeds RT
// matrix instructions and the expert's weights are streamed once per pass: an expert with up to 128 rows takes one
// pass of ceil(rows / 32) tiles, a larger one passes of four tiles first.  The staged chunk is G quantisation
// groups wide, narrower for more tiles (the same LDS).  Rows of a tile beyond the expert's count repeat its last
// row and are not stored; a wave without a strip works on strip 0 and stores nothing.
// SwiGLU of the matrix-core path: the rounding points of swiglu16 (sigmoid, g * sigmoid and the product with u each
// rounded to half) with the sigmoid from the hardware exponential and reciprocal, a tenth of the instructions of the
// bit-exact form (this path is tolerance-level anyway).
SL_DEV float swiglu_mm(float g, float u) {
  const float sg = f16r(__builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g)));
  return f16r(f16r(g * sg) * u);
}
// two staging buffers of 128 rows x GW groups (the largest shape of a pass): gate|up walks K = 2048 with two groups
// per barrier, the down projection (K = 512, four times the workgroups) with one, which leaves room for three workgroups
// per compute unit
template <bool DUAL> constexpr int GQ_WIDE = DUAL ? 2 : 1;
template <bool DUAL> constexpr int GQ_LDS_HALVES = 2 * 128 * (64 * GQ_WIDE<DUAL> + 8);
template <bool DUAL, int RT, int G>
SL_DEV void grouped_pass(const QmmGroupArgs& a, uint16_t* xsb, const uint16_t* list, int cnt, const uint32_t* const (&wp)[2],
                         const uint32_t* const (&sp)[2], bool live, int n0) {
  constexpr int NW = DUAL ? 2 : 1;
  constexpr int XS = 64 * G + 8;                         // halves per staged row
  constexpr int BUF = RT * 32 * XS;                      // halves per staging buffer
  static_assert(2 * BUF <= GQ_LDS_HALVES<DUAL>, "staging buffers exceed the workgroup's LDS");
  const int tid = threadIdx.x, lane = tid & 63;
  const int col = lane & 31, hh = lane >> 5;
  const int chunks = a.K / (64 * G);
  // the rows this thread stages: RT x 32 rows x G x 8 pieces of 16 bytes, RT x G pieces per thread
  uint32_t xoff[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int pr = list[min(t * 32 + (tid >> 3), cnt - 1)];
    xoff[t] = (uint32_t)(a.x_by_pair ? pr : (pr >> 3)) * (uint32_t)a.x_stride + (tid & 7) * 8;
  }
  mf_f16v acc[RT][NW];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int q = 0; q < NW; ++q)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[t][q][r] = 0.0f;
  uint4 xr[RT][G];
  auto fetch = [&](int c) {
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int g = 0; g < G; ++g) xr[t][g] = ld16(a.x + (size_t)(xoff[t] + (uint32_t)((c * G + g) * 64)));
  };
  auto put = [&](int buf) {
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int g = 0; g < G; ++g) st16(&xsb[buf * BUF + (t * 32 + (tid >> 3)) * XS + g * 64 + (tid & 7) * 8], permute8(xr[t][g]));
  };
  uint4 nw[NW][G];                                       // words 4*hh .. 4*hh+3 of each group (see k_qmm4_mfma16)
  uint32_t nsb[NW][G];
  auto wfetch = [&](int c) {
#pragma unroll
    for (int q = 0; q < NW; ++q)
#pragma unroll
      for (int g = 0; g < G; ++g) {
        nw[q][g] = ld16(wp[q] + (c * G + g) * 8 + 4 * hh);
        nsb[q][g] = sp[q][c * G + g];
      }
  };
  __syncthreads();                                       // the pass before has finished reading the staging buffers
  fetch(0);
  put(0);
  if (chunks > 1) fetch(1);
  wfetch(0);
  const uint32_t k1024 = dequant_k1024();
  for (int c = 0; c < chunks; ++c) {
    const int buf = c & 1;
    uint4 w[NW][G];
    uint32_t sb[NW][G];
#pragma unroll
    for (int q = 0; q < NW; ++q)
#pragma unroll
      for (int g = 0; g < G; ++g) { w[q][g] = nw[q][g]; sb[q][g] = nsb[q][g]; }
    if (c + 1 < chunks) wfetch(c + 1);
    __syncthreads();
    if (c + 1 < chunks) { put(buf ^ 1); if (c + 2 < chunks) fetch(c + 2); }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      mf_h2 s2[NW], b2[NW];
#pragma unroll
      for (int q = 0; q < NW; ++q) {
        s2[q] = __builtin_bit_cast(mf_h2, (sb[q][g] & 0xffffu) * 0x10001u);
        b2[q] = __builtin_bit_cast(mf_h2, (sb[q][g] >> 16) * 0x10001u);
      }
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        mf_h8 ax[RT];
#pragma unroll
        for (int t = 0; t < RT; ++t) ax[t] = *reinterpret_cast<const mf_h8*>(&xsb[buf * BUF + (t * 32 + col) * XS + g * 64 + 32 * hh + 8 * st]);
#pragma unroll
        for (int q = 0; q < NW; ++q) {
          const uint4 w0 = w[q][g];
          const uint32_t wsel = st == 0 ? w0.x : st == 1 ? w0.y : st == 2 ? w0.z : w0.w;
          const mf_h8 bw = dequant8(wsel, s2[q], b2[q], k1024);
#pragma unroll
          for (int t = 0; t < RT; ++t) acc[t][q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ax[t], bw, acc[t][q], 0, 0, 0);
        }
      }
    }
  }
  // The results leave through LDS: a lane holds sixteen rows of one column, and stored from there every value would
  // be a two-byte store with a row look-up and an address of its own (a third of the instructions of a short
  // K = 512 pass).  The tile is laid down [row][128 columns of the workgroup] in the staging space instead and goes
  // out in 16-byte pieces, two per thread and 32-row tile.
  constexpr int YS = 128 + 8;                            // halves per row of the result tile
  static_assert(RT * 32 * YS <= 2 * BUF, "the result tile fits the staging buffers");
  __syncthreads();                                       // the last chunk has been read
  const int wcol = (tid >> 6) * 32 + col;
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = t * 32 + 8 * (r >> 2) + 4 * hh + (r & 3);
      float v = acc[t][0][r];
      if constexpr (DUAL) v = swiglu_mm(f16r(v), f16r(acc[t][1][r]));
      xsb[row * YS + wcol] = f2h(v);
    }
  __syncthreads();
  const int nwg = n0 - (tid >> 6) * 32;                  // first column of the workgroup
#pragma unroll
  for (int p = 0; p < RT * 2; ++p) {
    const int idx = p * 256 + tid, row = idx >> 4, piece = idx & 15;
    if (row < cnt && nwg + piece * 8 < a.NE)
      st16(a.y + (size_t)list[row] * a.y_stride + nwg + piece * 8, *reinterpret_cast<const uint4*>(&xsb[row * YS + piece * 8]));
  }
}
template <bool DUAL>
__global__ __launch_bounds__(256, 2) void k_qmm4_mfma_grouped(QmmGroupArgs a) {
  __shared__ __align__(16) uint16_t xs[GQ_LDS_HALVES<DUAL>];
  constexpr int GW = GQ_WIDE<DUAL>;
  const int e = a.order[blockIdx.y];
  const int cnt_all = min(a.counts[e], GROUP_CAP);
  if (cnt_all == 0) return;                              // uniform for the workgroup
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 31;
  const int n0 = (blockIdx.x * 4 + wave) * 32;
  const bool live = n0 < a.NE;
  const size_t wrow = (size_t)e * a.NE + (live ? n0 + col : 0);
  const uint32_t* const wp[2] = {a.W + wrow * (a.K / 8), DUAL ? a.W2 + wrow * (a.K / 8) : nullptr};
  const uint32_t* const sp[2] = {a.SB + wrow * (a.K / 64), DUAL ? a.SB2 + wrow * (a.K / 64) : nullptr};
  const uint16_t* lists = a.lists + (size_t)e * GROUP_CAP;
  int r0 = 0;
  for (; cnt_all - r0 > 128; r0 += 128) grouped_pass<DUAL, 4, GW>(a, xs, lists + r0, 128, wp, sp, live, n0);
  const int rest = cnt_all - r0;                         // 1 .. 128; K % 256 == 0 for both shapes
  if (rest > 96) grouped_pass<DUAL, 4, GW>(a, xs, lists + r0, rest, wp, sp, live, n0);
  else if (rest > 64) grouped_pass<DUAL, 3, GW>(a, xs, lists + r0, rest, wp, sp, live, n0);
  else if (rest > 32) grouped_pass<DUAL, 2, 2>(a, xs, lists + r0, rest, wp, sp, live, n0);
  else grouped_pass<DUAL, 1, 4>(a, xs, lists + r0, rest, wp, sp, live, n0);
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

constexpr int VT_STRIDE = 72;     // halves per row of a transposed value tile (and of the lane kernel's P patch): 64 + 8 pad

// -------------------------------------------------------------------------------------------------
// Attention of a prefill chunk with running softmax sums (hybrid mode): workgroup = (part of the key range, kv head,
// block of 32 query rows), eight waves = the eight query heads of the group.  The workgroup walks its key tiles:
// keys [key][dim] and values transposed [dim][key] staged in LDS once for the eight heads (the next tile's pieces on
// their way in registers).  Both products are formed transposed, S^T = K Q^T and O^T = V^T P^T, so that a lane owns
// one query row: its 32 of the tile's 64 scores sit in its own registers (the other 32 in the lane 32 further), the
// row's running maximum and sum are one value per lane, and the accumulated output of the lane's row is rescaled by
// the lane's own factor when the maximum moved -- no cross-lane reductions apart from one exchange between the
// half-waves.  The softmax weights go from the score registers straight into the operand of the second product: the
// k slots of a matrix step are any eight keys as long as both operands agree, so a step takes the eight keys a lane
// already holds and the transposed value tile is stored with its keys in that order (key_slot below).  One partial
// (max, sum, unnormalised output) per part and row goes to the arrays of the per-tile kernels at index `part`;
// k_sdpa_merge_par finishes it with `group` = SDPA_FLASH_TILES.  Tolerance-level.
// -------------------------------------------------------------------------------------------------
constexpr int SDPA_FLASH_TILES = 8;   // key tiles per part (fixed: see the launch)
struct SdpaFlashArgs {
  SdpaArgs s;
  int M;
  int TP;                      // key tiles per part
};
// position of key (0..63) of a tile in a row of the transposed value tile: S^T register r of half-wave hh and 32-key
// block c holds key 32c + 8(r/4) + 4hh + r%4; step st = 2c + (r/8) of the second product takes registers 8(st%2) .. +7
SL_DEV int key_slot(int key) {
  const int c = key >> 5, g = (key >> 3) & 3, h = (key >> 2) & 1, i = key & 3;
  return 16 * (2 * c + (g >> 1)) + 8 * h + 4 * (g & 1) + i;
}
__global__ __launch_bounds__(512, 2) void k_sdpa_flash_mfma(SdpaFlashArgs a) {
  __shared__ __align__(16) uint16_t s_k[SDPA_TILE * KT_STRIDE];
  __shared__ __align__(16) uint16_t s_vt[256 * VT_STRIDE];
  const int part = blockIdx.x, kvh = blockIdx.y, m0 = blockIdx.z * 32;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 31, hh = lane >> 5;
  const int pos0 = a.s.st[0];
  const int rows = min(32, a.M - m0);
  const int nmax = pos0 + m0 + rows;                     // keys visible to the block's last row
  const int nt = (nmax + SDPA_TILE - 1) / SDPA_TILE;
  const int t_begin = part * a.TP, t_end = min(t_begin + a.TP, nt);
  if (t_begin >= nt) return;                             // uniform for the workgroup
  const uint16_t* kbase = a.s.kcache + (size_t)kvh * a.s.maxSeq * 256;
  const uint16_t* vbase = a.s.vcache + (size_t)kvh * a.s.maxSeq * 256;
  // a tile's pieces: keys 4 rows of 16 per thread (a row on 32 neighbouring lanes), values key tid & 63, eight dims
  // each; keys beyond the visible range repeat the last visible one (masked below, their values meet a weight of zero)
  uint4 pk[4], pv[4];
  auto fetch = [&](int t) {
    const int j0 = t * SDPA_TILE;
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int row = min(j0 + it * 16 + (tid >> 5), nmax - 1), key = min(j0 + (tid & 63), nmax - 1);
      pk[it] = ld16(kbase + (size_t)row * 256 + (tid & 31) * 8);
      pv[it] = ld16(vbase + (size_t)key * 256 + ((tid >> 6) + 8 * it) * 8);
    }
  };
  const float NEG = -__int_as_float(0x7f800000);
  const float C = 0.0625f * 1.44269504f;                 // scale 1/16 and log2(e) in one factor: weights are 2^(C s - max)
  const int head = kvh * 8 + wave;
  const int qrow = m0 + col;                             // this lane's query row
  const bool live = qrow < a.M;
  const uint16_t* qp = a.s.qrot + ((size_t)min(qrow, a.M - 1) * 16 + head) * 256 + 8 * hh;
  const int vslot = key_slot(tid & 63);
  float mrun = NEG, lrun = 0.0f;                         // of the lane's row, in units of log2: running max of C s, sum of 2^(C s - max)
  mf_f16v O[8];                                          // O^T: register r of block d is dim 32d + 8(r/4) + 4hh + r%4 of the lane's row
#pragma unroll
  for (int d = 0; d < 8; ++d)
#pragma unroll
    for (int r = 0; r < 16; ++r) O[d][r] = 0.0f;
  fetch(t_begin);
  for (int t = t_begin; t < t_end; ++t) {
    const int j0 = t * SDPA_TILE;
    __syncthreads();                                     // the tile before is no longer read
#pragma unroll
    for (int it = 0; it < 4; ++it) st16(&s_k[(it * 16 + (tid >> 5)) * KT_STRIDE + (tid & 31) * 8], pk[it]);
#pragma unroll
    for (int it = 0; it < 4; ++it) {
      const int c8 = ((tid >> 6) + 8 * it) * 8;
      const uint32_t w[4] = {pv[it].x, pv[it].y, pv[it].z, pv[it].w};
#pragma unroll
      for (int i = 0; i < 8; ++i) s_vt[(c8 + i) * VT_STRIDE + vslot] = (uint16_t)(w[i >> 1] >> (16 * (i & 1)));
    }
    fetch(min(t + 1, t_end - 1));
    __syncthreads();
    // S^T = K Q^T: lane (col, hh) brings dims 16*st + 8*hh .. +7 of key 32*c + col / of its query row
    mf_f16v S[2];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r) S[c][r] = 0.0f;
#pragma unroll
    for (int st = 0; st < 16; ++st) {
      const mf_h8 bq = __builtin_bit_cast(mf_h8, ld16(qp + 16 * st));
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const mf_h8 ak = *reinterpret_cast<const mf_h8*>(&s_k[(32 * c + col) * KT_STRIDE + 16 * st + 8 * hh]);
        S[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ak, bq, S[c], 0, 0, 0);
      }
    }
    // register r of block c is key j0 + 32c + 8(r/4) + 4hh + r%4 against the lane's row; the row sees keys up to
    // pos0 + qrow
    const int lim = live ? pos0 + qrow - j0 - 4 * hh : -1;   // largest visible value of 32c + 8(r/4) + r%4
    float mx = NEG;
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        S[c][r] = (32 * c + 8 * (r >> 2) + (r & 3) <= lim) ? C * S[c][r] : NEG;
        mx = fmaxf(mx, S[c][r]);
      }
    {
      const unsigned u = __float_as_uint(mx);
      const auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
      mx = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
    }
    const float mn = fmaxf(mrun, mx);
    const float alpha = (mn == mrun) ? 1.0f : __builtin_amdgcn_exp2f(mrun - mn);   // (mrun = -inf, mn finite: 0)
    float sum = 0.0f;
    mf_h8 ap[4];
#pragma unroll
    for (int c = 0; c < 2; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = (S[c][r] == NEG) ? 0.0f : __builtin_amdgcn_exp2f(S[c][r] - mn);
        sum += p;
        ap[2 * c + (r >> 3)][r & 7] = (_Float16)p;
      }
    {
      const unsigned u = __float_as_uint(sum);
      const auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
      sum = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
    }
    lrun = fmaf(lrun, alpha, sum);
    mrun = mn;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {   // some row's maximum moved: what it has accumulated shrinks with it
#pragma unroll
      for (int d = 0; d < 8; ++d)
#pragma unroll
        for (int r = 0; r < 16; ++r) O[d][r] *= alpha;
    }
    // O^T += V^T P^T: lane (col, hh) brings key slots 16*st + 8*hh .. +7 of dim 32*d + col / of its row of P
#pragma unroll
    for (int st = 0; st < 4; ++st)
#pragma unroll
      for (int d = 0; d < 8; ++d) {
        const mf_h8 av = *reinterpret_cast<const mf_h8*>(&s_vt[(32 * d + col) * VT_STRIDE + 16 * st + 8 * hh]);
        O[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av, ap[st], O[d], 0, 0, 0);
      }
  }
  if (live) {
    const size_t pi = ((size_t)qrow * 16 + head) * a.s.maxTiles + part;
    // the merge works with natural logarithms: max back from log2 units
    if (hh == 0) { a.s.pm[pi] = (mrun == NEG) ? NEG : mrun * 0.6931471805599453f; a.s.pl[pi] = lrun; }
    float* po = a.s.po + pi * 256 + 4 * hh;
#pragma unroll
    for (int d = 0; d < 8; ++d)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *reinterpret_cast<float4*>(po + 32 * d + 8 * g) = make_float4(O[d][4 * g], O[d][4 * g + 1], O[d][4 * g + 2], O[d][4 * g + 3]);
  }
}


// -------------------------------------------------------------------------------------------------
// Decode attention of a lane batch on the matrix cores (hybrid mode): every row is one new token of its own
// sequence, so a key tile is shared only by the 8 query heads of a kv group.  Workgroup = (key tile of 64, kv head,
// lane); the heads take rows 0..7 of a 32-row matrix operand (rows 8..31 carry nothing and their results are never
// read).  Waves 0 and 1 form S = Q K^T for 32 keys each (16 matrix instructions), every wave then turns two heads'
// scores into softmax pieces (fp32, hardware exp2; P rounded to half), and wave w forms dims 64w .. 64w+63 of
// O = P V (8 matrix instructions).  A workgroup walks T consecutive tiles with the keys and values of
// the next two tiles on their way while it works on the current one.  Same per-tile partials as k_sdpa_tile; k_sdpa_merge_par adds them up.
// -------------------------------------------------------------------------------------------------
struct SdpaLaneArgs {
  SdpaArgs s;
  int T;                       // consecutive key tiles per workgroup
};
// Workgroup barrier that waits for the wave's LDS traffic only: global loads issued before it stay in flight across it
// (__syncthreads would wait for them as well).
__global__ __launch_bounds__(256) void k_sdpa_lane_mfma(SdpaLaneArgs la) {
  __shared__ __align__(16) uint16_t s_k[SDPA_TILE * KT_STRIDE];
  __shared__ __align__(16) uint16_t s_vt[256 * VT_STRIDE];
  __shared__ __align__(16) uint16_t s_p[8 * VT_STRIDE];
  __shared__ __align__(16) uint16_t s_q[8 * KT_STRIDE];
  __shared__ float s_s[8 * SDPA_TILE];
  const SdpaArgs& a = la.s;
  const int kvh = blockIdx.y, m = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 31, hh = lane >> 5;
  const LaneRef& ref = a.lanes[m];
  const int N = ref.st[0] + 1;                           // keys visible to the lane's new token, itself included
  const int nt = (N + SDPA_TILE - 1) / SDPA_TILE;
  const int t_begin = blockIdx.x * la.T, t_end = min(t_begin + la.T, nt);
  if (t_begin >= nt) return;                             // uniform for the workgroup
  const uint16_t* kbase = ref.kcache + (size_t)kvh * ref.max_seq * 256;
  const uint16_t* vbase = ref.vcache + (size_t)kvh * ref.max_seq * 256;
  // A tile's keys and values (a row on 32 neighbouring lanes each) as they are fetched;
  // rows at or beyond N are zero.  The next tile's pieces are requested while the current tile is worked on.
  struct Piece { uint4 k[8], v[8]; };
  Piece pa, pb;
  auto fetch = [&](Piece& pc, int t) {
    const int j0 = t * SDPA_TILE;
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int row = it * 8 + (tid >> 5), c8 = (tid & 31) * 8;
      pc.k[it] = make_uint4(0, 0, 0, 0);
      if (j0 + row < N) pc.k[it] = ld16(kbase + (size_t)(j0 + row) * 256 + c8);
    }
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int row = it * 8 + (tid >> 5), c8 = (tid & 31) * 8;
      pc.v[it] = make_uint4(0, 0, 0, 0);
      if (j0 + row < N) pc.v[it] = ld16(vbase + (size_t)(j0 + row) * 256 + c8);
    }
  };
  fetch(pa, t_begin);
  if (t_begin + 1 < t_end) fetch(pb, t_begin + 1);
  // the group's 8 query rows wait in LDS (first read after the first tile's barrier)
  st16(&s_q[(tid >> 5) * KT_STRIDE + (tid & 31) * 8], ld16(a.qrot + ((size_t)m * 16 + kvh * 8 + (tid >> 5)) * 256 + (tid & 31) * 8));
  const float NEG = -__int_as_float(0x7f800000);
  // one tile from the piece that holds it; the piece is then free for the tile after the next, requested at once so
  // that two tiles are in flight while this one is worked on
  auto work = [&](Piece& pc, int tile) {
    const int j0 = tile * SDPA_TILE;
#pragma unroll
    for (int it = 0; it < 8; ++it) st16(&s_k[(it * 8 + (tid >> 5)) * KT_STRIDE + (tid & 31) * 8], pc.k[it]);
    // values transposed [dim][key]; the eight-key blocks of a dim's row are permuted by (dim / 8) % 8, so that the 32
    // lanes that hold one key (dims 8 apart, 1152 bytes in LDS) do not all write to the same two banks
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int c = tid & 31, kpos = ((it ^ (c & 7)) << 3) | (tid >> 5);       // key it*8 + (tid >> 5)
      const uint32_t w[4] = {pc.v[it].x, pc.v[it].y, pc.v[it].z, pc.v[it].w};
#pragma unroll
      for (int i = 0; i < 8; ++i) s_vt[(8 * c + i) * VT_STRIDE + kpos] = (uint16_t)(w[i >> 1] >> (16 * (i & 1)));
    }
    lds_barrier();
    if (tile + 2 < t_end) fetch(pc, tile + 2);
    if (wave < 2) {
      mf_f16v S;
#pragma unroll
      for (int r = 0; r < 16; ++r) S[r] = 0.0f;
#pragma unroll
      for (int st = 0; st < 16; ++st) {
        // A: lane (col, hh) brings dims 16*st + 8*hh .. +7 of head col (rows 8..31 carry no head)
        mf_h8 aq = *reinterpret_cast<const mf_h8*>(&s_q[(col & 7) * KT_STRIDE + 16 * st + 8 * hh]);
        if (col >= 8) aq = __builtin_bit_cast(mf_h8, make_uint4(0, 0, 0, 0));
        const mf_h8 bk = *reinterpret_cast<const mf_h8*>(&s_k[(32 * wave + col) * KT_STRIDE + 16 * st + 8 * hh]);
        S = __builtin_amdgcn_mfma_f32_32x32x16_f16(aq, bk, S, 0, 0, 0);
      }
      // registers 0..3 of lane (col, hh) are heads 4*hh .. 4*hh+3 against key 32*wave + col
      const int key = 32 * wave + col;
#pragma unroll
      for (int r = 0; r < 4; ++r) s_s[(4 * hh + r) * SDPA_TILE + key] = (j0 + key < N) ? 0.0625f * S[r] : NEG;
    }
    lds_barrier();
#pragma unroll
    for (int hq = 0; hq < 2; ++hq) {
      const int h8 = 2 * wave + hq;
      const float sv = s_s[h8 * SDPA_TILE + lane];
      const float mx = tree_max<64>(sv);                 // the tile's first key is always visible: finite
      const float p = (sv == NEG) ? 0.0f : __builtin_amdgcn_exp2f((sv - mx) * 1.44269504f);
      const float l = tree_sum<64>(p);
      if (lane == 0) {
        const size_t pi = ((size_t)m * 16 + kvh * 8 + h8) * a.maxTiles + tile;
        a.pm[pi] = mx; a.pl[pi] = l;
      }
      s_p[h8 * VT_STRIDE + lane] = f2h(p);
    }
    lds_barrier();
    mf_f16v O[2];
#pragma unroll
    for (int d = 0; d < 2; ++d)
#pragma unroll
      for (int r = 0; r < 16; ++r) O[d][r] = 0.0f;
#pragma unroll
    for (int st = 0; st < 4; ++st) {
      mf_h8 ap = *reinterpret_cast<const mf_h8*>(&s_p[(col & 7) * VT_STRIDE + 16 * st + 8 * hh]);
      if (col >= 8) ap = __builtin_bit_cast(mf_h8, make_uint4(0, 0, 0, 0));      // rows without a head
#pragma unroll
      for (int d = 0; d < 2; ++d) {
        const int dim = 32 * (2 * wave + d) + col;
        const mf_h8 bv = *reinterpret_cast<const mf_h8*>(&s_vt[dim * VT_STRIDE + (((2 * st + hh) ^ ((dim >> 3) & 7)) << 3)]);
        O[d] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ap, bv, O[d], 0, 0, 0);
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float* po = a.po + (((size_t)m * 16 + kvh * 8 + 4 * hh + r) * a.maxTiles + tile) * 256 + col;
#pragma unroll
      for (int d = 0; d < 2; ++d) po[32 * (2 * wave + d)] = O[d][r];
    }
    lds_barrier();                                       // the tile's LDS is read out before the next one is written
  };
  for (int tile = t_begin; tile < t_end; tile += 2) {
    work(pa, tile);
    if (tile + 1 < t_end) work(pb, tile + 1);
  }
}

// Merge of the tile partials on several waves (hybrid mode; tolerance-level: the tiles are not added up in tile order):
// workgroup = (head, row); the global maximum first, then wave w takes tiles w, w + MERGE_WAVES, ... with eight loads in
// flight, and wave 0 adds the waves' partial sums and applies the output gate like k_sdpa_merge.  Sixteen waves for a
// lane batch (few rows, each with up to hundreds of tiles), four for the rows of a prefill chunk (thousands of
// workgroups: bound by the bytes, and slower with large workgroups).
template <int MERGE_WAVES>
__global__ __launch_bounds__(64 * MERGE_WAVES) void k_sdpa_merge_par(SdpaMergeArgs a) {
  __shared__ float s_mx[MERGE_WAVES], s_l[MERGE_WAVES];
  __shared__ __align__(16) float s_o[MERGE_WAVES][256];
  const int h = blockIdx.x, m = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int N = a.lanes ? a.lanes[m].st[0] + 1 : a.st[0] + m + 1;
  int nt = (N + SDPA_TILE - 1) / SDPA_TILE;
  if (a.group > 1) nt = (nt + a.group - 1) / a.group;    // partials per part of `group` tiles (k_sdpa_flash_mfma)
  const size_t base = ((size_t)m * 16 + h) * a.maxTiles;
  const float NEG = -__int_as_float(0x7f800000);
  float mx = NEG;
  for (int t = tid; t < nt; t += 64 * MERGE_WAVES) mx = fmaxf(mx, a.pm[base + t]);
  mx = tree_max<64>(mx);
  if (lane == 0) s_mx[wave] = mx;
  __syncthreads();
  float Mx = s_mx[0];
#pragma unroll
  for (int w = 1; w < MERGE_WAVES; ++w) Mx = fmaxf(Mx, s_mx[w]);
  float L = 0.0f, O[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int t0 = wave; t0 < nt; t0 += 8 * MERGE_WAVES) {
    float4 o[8]; float f[8], l[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int t = t0 + MERGE_WAVES * i;
      const bool ok = t < nt;
      const size_t pi = base + (ok ? t : t0);
      o[i] = *reinterpret_cast<const float4*>(a.po + pi * 256 + 4 * lane);
      f[i] = ok ? exp_c(a.pm[pi] - Mx) : 0.0f;
      l[i] = a.pl[pi];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      L = fmaf(l[i], f[i], L);
      O[0] = fmaf(o[i].x, f[i], O[0]); O[1] = fmaf(o[i].y, f[i], O[1]); O[2] = fmaf(o[i].z, f[i], O[2]); O[3] = fmaf(o[i].w, f[i], O[3]);
    }
  }
  if (lane == 0) s_l[wave] = L;
  *reinterpret_cast<float4*>(&s_o[wave][4 * lane]) = make_float4(O[0], O[1], O[2], O[3]);
  __syncthreads();
  if (wave != 0) return;
  float Ls = 0.0f, Os[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int w = 0; w < MERGE_WAVES; ++w) {
    Ls += s_l[w];
    const float4 v = *reinterpret_cast<const float4*>(&s_o[w][4 * lane]);
    Os[0] += v.x; Os[1] += v.y; Os[2] += v.z; Os[3] += v.w;
  }
  const uint2 graw = *reinterpret_cast<const uint2*>(a.proj + (size_t)m * PROJ_STRIDE + h * 512 + 256 + 4 * lane);
  const float gt[4] = {lo_h(graw.x), hi_h(graw.x), lo_h(graw.y), hi_h(graw.y)};
  float r[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) r[i] = f16r(f16r(Os[i] / Ls) * sigmoid16(gt[i]));
  *reinterpret_cast<uint2*>(a.gated + (size_t)m * 4096 + h * 256 + 4 * lane) = make_uint2(pack2(r[0], r[1]), pack2(r[2], r[3]));
}

// Arg-max of rows of logits (first maximum, i.e. the lowest index on ties, of the half values): one workgroup per row.
__global__ __launch_bounds__(1024) void k_argmax_logits(const uint16_t* __restrict__ logits, int V, int32_t* __restrict__ tok_out,
                                                        int out_off) {
  __shared__ float s_v[1024];
  __shared__ int s_i[1024];
  const int m = blockIdx.x, tid = threadIdx.x;
  const uint16_t* row = logits + (size_t)m * V;
  float bv = -__int_as_float(0x7f800000);
  int bi = 0x7fffffff;
  for (int c = tid * 8; c < V; c += 1024 * 8) {          // V % 8 == 0
    float f[8];
    unpack8(ld16(row + c), f);
#pragma unroll
    for (int i = 0; i < 8; ++i) if (f[i] > bv) { bv = f[i]; bi = c + i; }
  }
  s_v[tid] = bv; s_i[tid] = bi;
  __syncthreads();
  for (int s = 512; s > 0; s >>= 1) {
    if (tid < s) {
      const float ov = s_v[tid + s]; const int oi = s_i[tid + s];
      if (ov > s_v[tid] || (ov == s_v[tid] && oi < s_i[tid])) { s_v[tid] = ov; s_i[tid] = oi; }
    }
    __syncthreads();
  }
  if (tid == 0) tok_out[out_off + m] = s_i[0];
}

template <int RT, int NS, int WPB>
inline void launch_qmm4_rt(QmmArgs a, int row_blocks, unsigned nz, hipStream_t stream) {
  const dim3 block(64 * WPB);
  a.col_blocks = (a.N / 32 + WPB * NS - 1) / (WPB * NS);
  a.row_blocks = row_blocks;
  const dim3 grid(xcd_tile_grid(a.col_blocks, a.row_blocks), 1, nz);
  constexpr int GMAX = RT == 1 ? 4 : NS == 2 ? 1 : 2;    // staging buffers of at most ~70 KB; two strips per wave leave registers for one group
  if (GMAX == 4 && a.K % 256 == 0) hipLaunchKernelGGL((k_qmm4_mfma16<RT, NS, GMAX, WPB>), grid, block, 0, stream, a);
  else if (GMAX >= 2 && a.K % 128 == 0) hipLaunchKernelGGL((k_qmm4_mfma16<RT, NS, 2, WPB>), grid, block, 0, stream, a);
  else hipLaunchKernelGGL((k_qmm4_mfma16<RT, NS, 1, WPB>), grid, block, 0, stream, a);
}
// Host-side launch: row tiles per wave chosen so that there are at least about as many wave tasks as SIMDs (1024):
// wide projections of many rows share the unpacking over 128 rows, narrow ones spread over more waves instead.
// (Two strips per wave, NS = 2, halve the LDS reads and the staging per matrix instruction but measured slower on
// the 2048 x 12352 x 2048 projection, 136-146 us against 129 us: 784 workgroups of one per compute unit leave a
// fourth round of 16, and one wave per SIMD has nothing to run while it waits at the chunk barrier.)
inline void launch_qmm4_mfma(const QmmArgs& a, hipStream_t stream) {
  const unsigned nz = a.W2 ? 2 : 1;
  const int strips = a.N / 32 * (int)nz, tiles = (a.M + 31) / 32;
  if (tiles >= 4 && strips * (tiles / 4) >= 768) launch_qmm4_rt<4, 1, 4>(a, (tiles + 3) / 4, nz, stream);
  else if (tiles >= 2 && strips * (tiles / 2) >= 768) launch_qmm4_rt<2, 1, 4>(a, (tiles + 1) / 2, nz, stream);
  else launch_qmm4_rt<1, 1, 4>(a, tiles, nz, stream);
}

}  // namespace sl
