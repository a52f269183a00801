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
  __shared__ __align__(16) uint16_t Ks[GC * GC_KS], Qs[GC * GC_KS];      // [t][d]
  __shared__ __align__(16) uint16_t KT[128 * GC_CS], VT[128 * GC_CS];    // [d][t]
  __shared__ __align__(16) uint16_t T1[GC * GC_CS], T2[GC * GC_CS];      // T diag(beta G) negated, T diag(beta): [t][i]
  __shared__ __align__(16) float Am[GC * GC_AS];                          // A, strictly lower triangle used
  __shared__ float Tl[GC * GC];                                           // T, rows as they are solved
  __shared__ float Lg[GC], Bt[GC], Eg[GC], Ec[GC];                        // log-decays, betas, G_t, G_C / G_t
  const int blk = blockIdx.x, hv = blockIdx.y, hk = hv >> 1;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int row0 = blk * GC;
  unsigned char* unit = a.scratch + ((size_t)blk * 32 + hv) * GC_UNIT_BYTES;
  // stage K, Q (rows) and K, V transposed
  for (int i = tid; i < GC * 16; i += 256) {
    const int t = i >> 4, p = i & 15;                       // 16 pieces of 8 halves per row
    const uint4 kq = ld16(a.kn + (size_t)(row0 + t) * 2048 + hk * 128 + 8 * p);
    const uint4 qq = ld16(a.qn + (size_t)(row0 + t) * 2048 + hk * 128 + 8 * p);
    const uint4 vq = ld16(a.vc + (size_t)(row0 + t) * 4096 + hv * 128 + 8 * p);
    st16(&Ks[t * GC_KS + 8 * p], kq);
    st16(&Qs[t * GC_KS + 8 * p], qq);
    const uint32_t kw[4] = {kq.x, kq.y, kq.z, kq.w}, vw[4] = {vq.x, vq.y, vq.z, vq.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      KT[(8 * p + 2 * j) * GC_CS + t] = (uint16_t)(kw[j] & 0xffffu);
      KT[(8 * p + 2 * j + 1) * GC_CS + t] = (uint16_t)(kw[j] >> 16);
      VT[(8 * p + 2 * j) * GC_CS + t] = (uint16_t)(vw[j] & 0xffffu);
      VT[(8 * p + 2 * j + 1) * GC_CS + t] = (uint16_t)(vw[j] >> 16);
    }
  }
  for (int i = tid; i < GC * GC; i += 256) Tl[i] = 0.0f;      // rows not solved yet are read (times a zero of A): keep them finite
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
  } else {
    // meanwhile: Qg = diag(G) Q and KdT = (diag(G_C / G) K)^T
    uint16_t* Qg = reinterpret_cast<uint16_t*>(unit + GC_OFF_QG);
    uint16_t* KdT = reinterpret_cast<uint16_t*>(unit + GC_OFF_KDT);
    for (int i = tid - 64; i < GC * 128; i += 192) {
      const int t = i >> 7, d = i & 127;
      Qg[t * 128 + d] = f2h(Eg[t] * h2f(Qs[t * GC_KS + d]));
      const int d2 = i >> 6, t2 = i & 63;
      KdT[d2 * 64 + t2] = f2h(Ec[t2] * h2f(KT[d2 * GC_CS + t2]));
    }
    if (tid == 64) *reinterpret_cast<float*>(unit + GC_OFF_GC) = Eg[GC - 1];
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
__global__ __launch_bounds__(256) void k_gdn_chunk_scan(GdnChunkArgs a) {
  extern __shared__ __align__(16) uint16_t gcs[];
  uint16_t* Wm = gcs;                          // [64][GC_KS]
  uint16_t* Qg = Wm + GC * GC_KS;              // [64][GC_KS]
  uint16_t* KdT = Qg + GC * GC_KS;             // [128][GC_CS]
  uint16_t* P = KdT + 128 * GC_CS;             // [64][GC_CS]
  uint16_t* S16 = P + GC * GC_CS;              // [128 dv][GC_KS]
  uint16_t* UT = S16 + 128 * GC_KS;            // [128 dv][GC_CS]
  const int hv = blockIdx.x, hk = hv >> 1;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 31;
  const bool par = a.st[1] != 0;
  const float* sin_ = par ? a.state[1] : a.state[0];
  float* sout = par ? a.state[0] : a.state[1];
  const int dv0 = wave * 32;
  // the state slice as four result tiles: S[dv0 + row][32 j + col]
  mf_f16v S[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) S[j][r] = sin_[((size_t)hv * 128 + dv0 + acc_row(r, lane)) * 128 + 32 * j + col];
  const int nblk = a.M / GC;
  // A block's matrices travel global -> registers -> LDS one block ahead: the loads of block b + 1 are in flight
  // while block b is multiplied (a block's arithmetic is shorter than a trip to memory).
  uint4 pw[4], pq[4], pk[4], pp[2];
  float uvr[2][16];
  float gcd_next = 0.0f;
  auto prefetch = [&](int blk) {
    const unsigned char* unit = a.scratch + ((size_t)blk * 32 + hv) * GC_UNIT_BYTES;
    const uint16_t* gWm = reinterpret_cast<const uint16_t*>(unit + GC_OFF_WM);
    const uint16_t* gQg = reinterpret_cast<const uint16_t*>(unit + GC_OFF_QG);
    const uint16_t* gKd = reinterpret_cast<const uint16_t*>(unit + GC_OFF_KDT);
    const uint16_t* gP = reinterpret_cast<const uint16_t*>(unit + GC_OFF_P);
    const float* UV = reinterpret_cast<const float*>(unit + GC_OFF_UV);
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
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int r = 0; r < 16; ++r) uvr[rt][r] = UV[(rt * 32 + acc_row(r, lane)) * 128 + dv0 + col];
    gcd_next = *reinterpret_cast<const float*>(unit + GC_OFF_GC);
  };
  if (nblk > 0) prefetch(0);
  for (int blk = 0; blk < nblk; ++blk) {
    __syncthreads();                           // the block before is done with the staged matrices
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = tid + 256 * j;
      st16(&Wm[(i >> 4) * GC_KS + 8 * (i & 15)], pw[j]);
      st16(&Qg[(i >> 4) * GC_KS + 8 * (i & 15)], pq[j]);
      st16(&KdT[(i >> 3) * GC_CS + 8 * (i & 7)], pk[j]);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int i = tid + 256 * j;
      st16(&P[(i >> 3) * GC_CS + 8 * (i & 7)], pp[j]);
    }
    // the state in half as the right-hand operand of the products with S_0^T
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) S16[(dv0 + acc_row(r, lane)) * GC_KS + 32 * j + col] = f2h(S[j][r]);
    const float GCd = gcd_next;
    mf_f16v U[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int r = 0; r < 16; ++r) U[rt][r] = uvr[rt][r];
    __syncthreads();
    if (blk + 1 < nblk) prefetch(blk + 1);
    // U = UV - Wm S_0^T for this wave's value dims (rows t, columns dv0 + col), kept transposed in half for what follows
    mf_f16v Y[2];
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      mma_tile(U[rt], Wm + rt * 32 * GC_KS, GC_KS, S16 + dv0 * GC_KS, GC_KS, 128, lane);
#pragma unroll
      for (int r = 0; r < 16; ++r) UT[(dv0 + col) * GC_CS + rt * 32 + acc_row(r, lane)] = f2h(U[rt][r]);
      acc_zero(Y[rt]);
      mma_tile(Y[rt], Qg + rt * 32 * GC_KS, GC_KS, S16 + dv0 * GC_KS, GC_KS, 128, lane);
    }
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      mma_tile(Y[rt], P + rt * 32 * GC_CS, GC_CS, UT + dv0 * GC_CS, GC_CS, 64, lane);
#pragma unroll
      for (int r = 0; r < 16; ++r)
        a.ycore[(size_t)(blk * GC + rt * 32 + acc_row(r, lane)) * 4096 + hv * 128 + dv0 + col] = f2h(Y[rt][r]);
    }
    // S = G_C S + U^T Kd
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int r = 0; r < 16; ++r) S[j][r] *= GCd;
      mma_tile(S[j], UT + dv0 * GC_CS, GC_CS, KdT + 32 * j * GC_CS, GC_CS, 64, lane);
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) sout[((size_t)hv * 128 + dv0 + acc_row(r, lane)) * 128 + 32 * j + col] = S[j][r];
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
constexpr int GC_SCAN_LDS = (2 * GC * GC_KS + 128 * GC_CS + GC * GC_CS + 128 * GC_KS + 128 * GC_CS) * 2;

}  // namespace sl
