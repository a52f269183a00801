// Chunked form of the gated delta rule for the rows of a prefill chunk (hybrid mode), on the matrix cores.
//
// The recurrence of one value head (GatedDelta.swift:63-124 in the reference; k_gdn_core here), state S [dv][dk]:
//     S_t = g_t S_{t-1} + u_t k_t^T,   u_t = beta_t (v_t - g_t S_{t-1} k_t),   y_t = S_t q_t
// is sequential in t.  Over a block of C = 64 rows it can be written with matrices (the "WY" / UT-transform form of
// the delta rule).  With G_t = g_1 ... g_t inside the block and S_0 the state at its start:
//     u_t = beta_t v_t - beta_t G_t S_0 k_t - beta_t sum_{i<t} (G_t / G_i) (k_t . k_i) u_i
// i.e. (I + A) U = B V - B diag(G) K S_0^T with A[t][i] = beta_t (G_t / G_i)(k_t . k_i) below the diagonal, so with
// T = (I + A)^-1:      U = (T B V) - (T B diag(G) K) S_0^T = UV - Wm S_0^T
//     Y = diag(G) Q S_0^T + (M o Q K^T) U,   M[t][i] = G_t / G_i for i <= t
//     S_C = G_C S_0 + U^T diag(G_C / G) K.
// T, UV, Wm, P = M o Q K^T, Qg = diag(G) Q and Kd = diag(G_C / G) K do not depend on the state: k_gdn_chunk_prep
// forms them for all blocks and heads at once (products on the matrix cores, the 64 x 64 triangular inverse by
// forward substitution in fp32).  k_gdn_chunk_scan then walks the blocks of a head in order with four small matrix
// products per block.  Ratios of decays are formed as exp of differences of log-decays, so nothing overflows.
//
// Tolerance-level like the rest of the hybrid path (operands of the matrix instructions are rounded to half); used
// for calls whose row count and start position are multiples of 64, so a row's result does not depend on how a
// prompt is cut into such calls.
#pragma once
#include "sl_mfma.cuh"

namespace sl {

constexpr int GC = 64;                      // rows per block
constexpr int GC_KS = 128 + 8;              // halves per staged row of a [*, 128] matrix
constexpr int GC_CS = 64 + 8;               // halves per staged row of a [*, 64] matrix
constexpr int GC_AS = 64 + 4;               // floats per row of the triangular matrix (rows 16-byte aligned)
// Scratch of one (block, value head), in bytes: Wm (negated) [64][128] half, Qg [64][128] half, KdT [128][64] half,
// P [64][64] half, UV [64][128] float, G_C float (padded to 256 bytes)
constexpr size_t GC_OFF_WM = 0, GC_OFF_QG = 16384, GC_OFF_KDT = 32768, GC_OFF_P = 49152, GC_OFF_UV = 57344, GC_OFF_GC = 90112;
constexpr size_t GC_UNIT_BYTES = 90368;

struct GdnChunkArgs {
  const uint16_t *qn, *kn;   // [M, 2048] normed, scaled query / key rows (k_gdn_prep_rows)
  const uint16_t* vc;        // [M, 4096] value rows
  const float* gb;           // [M, 64] decay g (32 heads), beta (32 heads)
  unsigned char* scratch;    // [blocks][32][GC_UNIT_BYTES]
  float* state[2];           // [32][128][128] ping-pong
  uint16_t* hist[2];
  const uint16_t* proj;      // projection rows (for the conv-history shift)
  const int32_t* st;         // st[1] = parity (read side)
  uint16_t* ycore;           // [M, 4096]
  int M;                     // multiple of 64
};

// One 32 x 32 tile: acc += A[32 rows][K] * Bt[32 rows][K]^T, both operands row-major halves in LDS with the given strides.
SL_DEV void mma_tile(mf_f16v& acc, const uint16_t* A, int lda, const uint16_t* Bt, int ldb, int K, int lane) {
  const int col = lane & 31, hh = lane >> 5;
  for (int k0 = 0; k0 < K; k0 += 16) {
    const mf_h8 a = *reinterpret_cast<const mf_h8*>(A + col * lda + k0 + 8 * hh);
    const mf_h8 b = *reinterpret_cast<const mf_h8*>(Bt + col * ldb + k0 + 8 * hh);
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc, 0, 0, 0);
  }
}
SL_DEV void acc_zero(mf_f16v& a) {
#pragma unroll
  for (int r = 0; r < 16; ++r) a[r] = 0.0f;
}
// row of register r within a 32 x 32 result tile (column = lane & 31)
SL_DEV int acc_row(int r, int lane) { return 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3); }

// ---- state-independent part: grid (blocks, 32 value heads), 256 threads ---------------------------------
__global__ __launch_bounds__(256) void k_gdn_chunk_prep(GdnChunkArgs a) {
  // 73 KB of LDS, so that two workgroups share a compute unit and one's triangular solve (a chain on a single wave)
  // runs beside the other's matrix products.  Three areas are used twice: K and Q rows are dead once K K^T, Q K^T, Qg
  // and KdT are formed, and make room for T and its two scaled half copies; the value tile is staged only after the
  // solve, into the space of A.
  __shared__ __align__(16) uint16_t area_k[GC * GC_KS], area_q[2 * GC * GC_CS];
  __shared__ __align__(16) uint16_t KT[128 * GC_CS];                     // [d][t]
  __shared__ __align__(16) float area_a[128 * GC_CS / 2];                // A [64][GC_AS] floats, later V^T [128][GC_CS] halves
  __shared__ float Lg[GC], Bt[GC], Eg[GC], Ec[GC];                        // log-decays, betas, G_t, G_C / G_t
  static_assert(GC * GC_AS <= 128 * GC_CS / 2 && GC * GC * 4 <= GC * GC_KS * 2 && GC * GC_KS <= 2 * GC * GC_CS, "aliased areas");
  uint16_t* Ks = area_k;                                                  // [t][d]
  uint16_t* Qs = area_q;
  float* Tl = reinterpret_cast<float*>(area_k);                           // T, rows as they are solved (after Ks is dead)
  uint16_t* T1 = area_q;                                                  // T diag(beta G) negated, T diag(beta): [t][i] (after Qs is dead)
  uint16_t* T2 = area_q + GC * GC_CS;
  float* Am = area_a;                                                     // A, strictly lower triangle used
  uint16_t* VT = reinterpret_cast<uint16_t*>(area_a);                     // [d][t], staged after the solve
  const int blk = blockIdx.x, hv = blockIdx.y, hk = hv >> 1;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int row0 = blk * GC;
  unsigned char* unit = a.scratch + ((size_t)blk * 32 + hv) * GC_UNIT_BYTES;
  // stage K, Q (rows) and K transposed
  for (int i = tid; i < GC * 16; i += 256) {
    const int t = i >> 4, p = i & 15;                       // 16 pieces of 8 halves per row
    const uint4 kq = ld16(a.kn + (size_t)(row0 + t) * 2048 + hk * 128 + 8 * p);
    const uint4 qq = ld16(a.qn + (size_t)(row0 + t) * 2048 + hk * 128 + 8 * p);
    st16(&Ks[t * GC_KS + 8 * p], kq);
    st16(&Qs[t * GC_KS + 8 * p], qq);
    const uint32_t kw[4] = {kq.x, kq.y, kq.z, kq.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      KT[(8 * p + 2 * j) * GC_CS + t] = (uint16_t)(kw[j] & 0xffffu);
      KT[(8 * p + 2 * j + 1) * GC_CS + t] = (uint16_t)(kw[j] >> 16);
    }
  }
  if (tid < GC) {
    const float g = a.gb[(size_t)(row0 + tid) * 64 + hv];
    Lg[tid] = fmaxf(log_c(fmaxf(g, 1e-37f)), -80.0f);      // a decay of zero: as good as e^-80
    Bt[tid] = a.gb[(size_t)(row0 + tid) * 64 + 32 + hv];
  }
  __syncthreads();
  if (tid == 0) {                                           // log-decays accumulated along the block
    float s = 0.0f;
    for (int t = 0; t < GC; ++t) { s += Lg[t]; Lg[t] = s; }
  }
  __syncthreads();
  if (tid < GC) { Eg[tid] = exp_c(Lg[tid]); Ec[tid] = exp_c(Lg[GC - 1] - Lg[tid]); }
  // K K^T -> A and Q K^T -> P: wave w takes tile (w >> 1, w & 1) of both
  {
    const int rt = wave >> 1, ct = wave & 1, col = lane & 31;
    mf_f16v kk, qk;
    acc_zero(kk); acc_zero(qk);
    mma_tile(kk, Ks + rt * 32 * GC_KS, GC_KS, Ks + ct * 32 * GC_KS, GC_KS, 128, lane);
    mma_tile(qk, Qs + rt * 32 * GC_KS, GC_KS, Ks + ct * 32 * GC_KS, GC_KS, 128, lane);
    uint16_t* P = reinterpret_cast<uint16_t*>(unit + GC_OFF_P);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int t = rt * 32 + acc_row(r, lane), i = ct * 32 + col;
      const float dec = (i <= t) ? exp_c(Lg[t] - Lg[i]) : 0.0f;
      Am[t * GC_AS + i] = (i < t) ? Bt[t] * dec * kk[r] : 0.0f;
      P[t * 64 + i] = f2h(dec * qk[r]);
    }
  }
  __syncthreads();                                            // G_t and G_C / G_t are written, the products have read K and Q
  // Qg = diag(G) Q and KdT = (diag(G_C / G) K)^T (all waves; the last readers of the Q rows)
  {
    uint16_t* Qg = reinterpret_cast<uint16_t*>(unit + GC_OFF_QG);
    uint16_t* KdT = reinterpret_cast<uint16_t*>(unit + GC_OFF_KDT);
    for (int i = tid; i < GC * 128; i += 256) {
      const int t = i >> 7, d = i & 127;
      Qg[t * 128 + d] = f2h(Eg[t] * h2f(Qs[t * GC_KS + d]));
      const int d2 = i >> 6, t2 = i & 63;
      KdT[d2 * 64 + t2] = f2h(Ec[t2] * h2f(KT[d2 * GC_CS + t2]));
    }
    if (tid == 64) *reinterpret_cast<float*>(unit + GC_OFF_GC) = Eg[GC - 1];
  }
  __syncthreads();                                            // K and Q rows are dead, A is complete
  for (int i = tid; i < GC * GC; i += 256) Tl[i] = 0.0f;      // rows not solved yet are read (times a zero of A): keep them finite
  // the value rows of the block, requested now and staged once A is no longer needed
  uint4 vq[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = tid + 256 * j, t = i >> 4, p = i & 15;
    vq[j] = ld16(a.vc + (size_t)(row0 + t) * 4096 + hv * 128 + 8 * p);
  }
  __syncthreads();
  // T = (I + A)^-1 by forward substitution, lane j = column j (wave 0); rows in registers
  if (wave == 0) {
    // Row t needs A[t][0 .. t-1] (the same for every lane: read four at a time; entries at and beyond t are zero) and
    // the column's earlier rows, which are kept in LDS (same wave, so reads follow writes in program order).  Four
    // partial sums keep the chains of dependent multiply-adds short.
    // (rows are solved in four bands of 16: a band's rows read the finished bands with a fixed trip count, so those
    // reads are issued together, and the band's own earlier rows likewise)
    for (int band = 0; band < 4; ++band) {
      for (int tt = 0; tt < 16; ++tt) {
        const int t = 16 * band + tt;
        float p[4] = {(t == lane) ? 1.0f : 0.0f, 0.0f, 0.0f, 0.0f};
        for (int b = 0; b < band; ++b) {
#pragma unroll
          for (int i4 = 0; i4 < 4; ++i4) {
            const float4 a4 = *reinterpret_cast<const float4*>(&Am[t * GC_AS + 16 * b + 4 * i4]);
            p[0] = fmaf(-a4.x, Tl[(16 * b + 4 * i4) * GC + lane], p[0]);
            p[1] = fmaf(-a4.y, Tl[(16 * b + 4 * i4 + 1) * GC + lane], p[1]);
            p[2] = fmaf(-a4.z, Tl[(16 * b + 4 * i4 + 2) * GC + lane], p[2]);
            p[3] = fmaf(-a4.w, Tl[(16 * b + 4 * i4 + 3) * GC + lane], p[3]);
          }
        }
#pragma unroll
        for (int i4 = 0; i4 < 4; ++i4) {             // the band's own rows (those at and beyond t are still zero)
          const float4 a4 = *reinterpret_cast<const float4*>(&Am[t * GC_AS + 16 * band + 4 * i4]);
          p[0] = fmaf(-a4.x, Tl[(16 * band + 4 * i4) * GC + lane], p[0]);
          p[1] = fmaf(-a4.y, Tl[(16 * band + 4 * i4 + 1) * GC + lane], p[1]);
          p[2] = fmaf(-a4.z, Tl[(16 * band + 4 * i4 + 2) * GC + lane], p[2]);
          p[3] = fmaf(-a4.w, Tl[(16 * band + 4 * i4 + 3) * GC + lane], p[3]);
        }
        Tl[t * GC + lane] = (p[0] + p[1]) + (p[2] + p[3]);
      }
    }
    const float bj = Bt[lane], gj = Eg[lane];
    for (int t = 0; t < GC; ++t) {
      const float tv = Tl[t * GC + lane];
      T1[t * GC_CS + lane] = f2h(-(tv * bj * gj));
      T2[t * GC_CS + lane] = f2h(tv * bj);
    }
  }
  __syncthreads();                                            // A is dead: the value tile takes its place
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = tid + 256 * j, t = i >> 4, p = i & 15;
    const uint32_t vw[4] = {vq[j].x, vq[j].y, vq[j].z, vq[j].w};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      VT[(8 * p + 2 * q) * GC_CS + t] = (uint16_t)(vw[q] & 0xffffu);
      VT[(8 * p + 2 * q + 1) * GC_CS + t] = (uint16_t)(vw[q] >> 16);
    }
  }
  __syncthreads();
  // -Wm = T1 K and UV = T2 V: 2 x 4 tiles each; wave w takes column tile w of both row tiles
  {
    uint16_t* Wm = reinterpret_cast<uint16_t*>(unit + GC_OFF_WM);
    float* UV = reinterpret_cast<float*>(unit + GC_OFF_UV);
    const int col = lane & 31;
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      mf_f16v w, u;
      acc_zero(w); acc_zero(u);
      mma_tile(w, T1 + rt * 32 * GC_CS, GC_CS, KT + wave * 32 * GC_CS, GC_CS, 64, lane);
      mma_tile(u, T2 + rt * 32 * GC_CS, GC_CS, VT + wave * 32 * GC_CS, GC_CS, 64, lane);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int t = rt * 32 + acc_row(r, lane);
        Wm[t * 128 + wave * 32 + col] = f2h(w[r]);
        UV[t * 128 + wave * 32 + col] = u[r];
      }
    }
  }
}

// ---- the blocks of a value head in order: grid 32, 256 threads; wave w owns value dims 32 w .. 32 w + 31 ------------
// Everything the wave carries from product to product stays in registers.  The state slice is kept transposed, as four
// result tiles T[c] of S^T (rows = 32 key dims, columns = the wave's 32 value dims): a lane then holds, for its
// value dim, sixteen key dims of each tile, and since the k slots of a matrix step may be any eight indices as long
// as both operands agree, those registers -- rounded to half -- are the right-hand operand of the products that
// contract over the key dim (U = UV - Wm S_0^T and Q_g S_0^T), the result tiles U (rows = block rows, columns = value
// dims) are in turn the right-hand operand of the products that contract over the block row (P U and the state update
// Kd^T U), and the state update delivers S^T tiles again.  The left-hand operands come from LDS, staged with the
// contraction index of each 32-block in the matching order (kslot32).  Two sets of staging buffers: one barrier per
// block; the block after the next is on its way from memory meanwhile.
// position of contraction index k in a staged row: matrix step st (0, 1) of 32-block c takes, on half-wave hh, the
// eight indices that registers 8 st .. 8 st + 7 of a result tile hold there: 32 c + 8 (2 st + j / 4) + 4 hh + j % 4
SL_DEV int kslot32(int k) {
  const int g = (k >> 3) & 3, h = (k >> 2) & 1, i = k & 3;
  return (k & ~31) + 16 * (g >> 1) + 8 * h + 4 * (g & 1) + i;
}
// a 16-byte piece (eight consecutive indices from k0, a multiple of 8) into its two places of a staged row
SL_DEV void stage_piece(uint16_t* row, int k0, uint4 v) {
  uint16_t* p = row + kslot32(k0);
  *reinterpret_cast<uint2*>(p) = make_uint2(v.x, v.y);
  *reinterpret_cast<uint2*>(p + 8) = make_uint2(v.z, v.w);
}
// registers 8 st .. 8 st + 7 of a result tile as a matrix operand
SL_DEV mf_h8 tile_operand(const mf_f16v& t, int st) {
  mf_h8 o;
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = (_Float16)t[8 * st + j];
  return o;
}
constexpr int GC_SCAN_BUF = 2 * GC * GC_KS + 128 * GC_CS + GC * GC_CS;   // halves per set: Wm, Qg, KdT, P
constexpr int GC_SCAN_LDS = 2 * GC_SCAN_BUF * 2;
__global__ __launch_bounds__(256) void k_gdn_chunk_scan(GdnChunkArgs a) {
  extern __shared__ __align__(16) uint16_t gcs[];
  const int hv = blockIdx.x, hk = hv >> 1;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 31, hh = lane >> 5;
  const bool par = a.st[1] != 0;
  const float* sin_ = par ? a.state[1] : a.state[0];
  float* sout = par ? a.state[0] : a.state[1];
  const int dv0 = wave * 32;
  // T[c][r] = S[dv0 + col][32 c + acc_row(r)]
  mf_f16v T[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float4 v = *reinterpret_cast<const float4*>(sin_ + ((size_t)hv * 128 + dv0 + col) * 128 + 32 * c + 8 * g + 4 * hh);
      T[c][4 * g] = v.x; T[c][4 * g + 1] = v.y; T[c][4 * g + 2] = v.z; T[c][4 * g + 3] = v.w;
    }
  const int nblk = a.M / GC;
  uint4 pw[4], pq[4], pk[4], pp[2];
  float uvn[2][16];                            // UV of the block after the current one (start value of its U)
  float gcn = 0.0f;
  auto fetch = [&](int blk) {
    const unsigned char* unit = a.scratch + ((size_t)min(blk, nblk - 1) * 32 + hv) * GC_UNIT_BYTES;
    const uint16_t* gWm = reinterpret_cast<const uint16_t*>(unit + GC_OFF_WM);
    const uint16_t* gQg = reinterpret_cast<const uint16_t*>(unit + GC_OFF_QG);
    const uint16_t* gKd = reinterpret_cast<const uint16_t*>(unit + GC_OFF_KDT);
    const uint16_t* gP = reinterpret_cast<const uint16_t*>(unit + GC_OFF_P);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = tid + 256 * j;
      pw[j] = ld16(gWm + (i >> 4) * 128 + 8 * (i & 15));
      pq[j] = ld16(gQg + (i >> 4) * 128 + 8 * (i & 15));
      pk[j] = ld16(gKd + (i >> 3) * 64 + 8 * (i & 7));
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int i = tid + 256 * j;
      pp[j] = ld16(gP + (i >> 3) * 64 + 8 * (i & 7));
    }
  };
  auto fetch_uv = [&](int blk) {
    const unsigned char* unit = a.scratch + ((size_t)min(blk, nblk - 1) * 32 + hv) * GC_UNIT_BYTES;
    const float* UV = reinterpret_cast<const float*>(unit + GC_OFF_UV);
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int r = 0; r < 16; ++r) uvn[rt][r] = UV[(rt * 32 + acc_row(r, lane)) * 128 + dv0 + col];
    gcn = *reinterpret_cast<const float*>(unit + GC_OFF_GC);
  };
  auto stage = [&](int set) {                  // the fetched block into staging set `set`; its UV and G_C become current
    uint16_t* Wm = gcs + set * GC_SCAN_BUF;
    uint16_t* Qg = Wm + GC * GC_KS;
    uint16_t* KdT = Qg + GC * GC_KS;
    uint16_t* P = KdT + 128 * GC_CS;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = tid + 256 * j;
      stage_piece(Wm + (i >> 4) * GC_KS, 8 * (i & 15), pw[j]);
      stage_piece(Qg + (i >> 4) * GC_KS, 8 * (i & 15), pq[j]);
      stage_piece(KdT + (i >> 3) * GC_CS, 8 * (i & 7), pk[j]);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int i = tid + 256 * j;
      stage_piece(P + (i >> 3) * GC_CS, 8 * (i & 7), pp[j]);
    }
  };
  if (nblk > 0) { fetch(0); stage(0); fetch_uv(0); }
  if (nblk > 1) fetch(1);
  for (int blk = 0; blk < nblk; ++blk) {
    const int set = blk & 1;
    lds_barrier();                             // set `set` is staged; the other set is no longer read (loads stay in flight)
    const uint16_t* Wm = gcs + set * GC_SCAN_BUF;
    const uint16_t* Qg = Wm + GC * GC_KS;
    const uint16_t* KdT = Qg + GC * GC_KS;
    const uint16_t* P = KdT + 128 * GC_CS;
    // this block's accumulator start and decay; then the next block goes to the other set and the one after it is requested
    mf_f16v U[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int r = 0; r < 16; ++r) U[rt][r] = uvn[rt][r];
    const float GCd = gcn;
    if (blk + 1 < nblk) {
      stage(set ^ 1);
      fetch(blk + 2);
      fetch_uv(blk + 1);
    }
    // the state in half as the right-hand operand of the products that contract over the key dim
    mf_h8 Th[4][2];
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int st = 0; st < 2; ++st) Th[c][st] = tile_operand(T[c], st);
    // U = UV - Wm S_0^T and Y = Qg S_0^T for this wave's value dims (rows = block rows, columns = value dims).  The
    // left-hand operands of a group of products are read from LDS together, ahead of the matrix instructions (the
    // fences keep it that way: a read waited for in front of every matrix instruction costs its full latency each time).
    mf_f16v Y[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      mf_h8 aw[8], aq[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int off = (rt * 32 + col) * GC_KS + 16 * i + 8 * hh;
        aw[i] = *reinterpret_cast<const mf_h8*>(Wm + off);
        aq[i] = *reinterpret_cast<const mf_h8*>(Qg + off);
      }
      acc_zero(Y[rt]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        U[rt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aw[i], Th[i >> 1][i & 1], U[rt], 0, 0, 0);
        Y[rt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aq[i], Th[i >> 1][i & 1], Y[rt], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    mf_h8 Uh[2][2];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int st = 0; st < 2; ++st) Uh[sb][st] = tile_operand(U[sb], st);
    // S^T = G_C S^T + Kd^T U first (the next block waits for it), then Y += P U
    {
      mf_h8 ak[16];
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i) ak[4 * c + i] = *reinterpret_cast<const mf_h8*>(KdT + (32 * c + col) * GC_CS + 16 * i + 8 * hh);
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) T[c][r] *= GCd;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int c = 0; c < 4; ++c) T[c] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ak[4 * c + i], Uh[i >> 1][i & 1], T[c], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    {
      mf_h8 ap[8];
#pragma unroll
      for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) ap[4 * rt + i] = *reinterpret_cast<const mf_h8*>(P + (rt * 32 + col) * GC_CS + 16 * i + 8 * hh);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) Y[rt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ap[4 * rt + i], Uh[i >> 1][i & 1], Y[rt], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        a.ycore[(size_t)(blk * GC + rt * 32 + acc_row(r, lane)) * 4096 + hv * 128 + dv0 + col] = f2h(Y[rt][r]);
  }
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int g = 0; g < 4; ++g)
      *reinterpret_cast<float4*>(sout + ((size_t)hv * 128 + dv0 + col) * 128 + 32 * c + 8 * g + 4 * hh) =
          make_float4(T[c][4 * g], T[c][4 * g + 1], T[c][4 * g + 2], T[c][4 * g + 3]);
  // conv-history shift: rows M .. M+2 of [hist | qkv]; q and k channels by the even heads, value channels by every head
  const uint16_t* hin = par ? a.hist[1] : a.hist[0];
  uint16_t* hout = par ? a.hist[0] : a.hist[1];
  if ((hv & 1) == 0) {
    const int qk_ch = (tid < 128) ? (hk * 128 + tid) : (2048 + hk * 128 + (tid - 128));
#pragma unroll
    for (int j = 0; j < 3; ++j) hout[j * SL_CONV_DIM + qk_ch] = f2h(conv_tap(a.proj, hin, a.M + j, qk_ch));
  }
  if (tid < 128) {
    const int v_ch = 4096 + hv * 128 + tid;
#pragma unroll
    for (int j = 0; j < 3; ++j) hout[j * SL_CONV_DIM + v_ch] = f2h(conv_tap(a.proj, hin, a.M + j, v_ch));
  }
}

}  // namespace sl
