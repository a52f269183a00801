// Persistent single-token decode kernel for gfx950.
//
// One launch runs a whole batch-1 step (embed -> all layers -> final norm -> lm_head -> argmax)
// on a grid of one 1024-thread workgroup per compute unit.  The ~250 dependent stages of a step
// are separated by a two-level grid barrier (about 1.7 us) instead of kernel boundaries, and each
// wave issues the weight loads of its next stage before it waits, so HBM keeps streaming while
// the 4 KB activation vector of the previous stage crosses the chip.
//
// Cross-workgroup traffic (activations, barrier words) uses agent-scope atomic loads/stores, which
// are coherent across the 8 XCDs without cache maintenance.  Weights, KV rows of earlier tokens
// and the recurrent state are only read after a launch boundary and use plain 16-byte loads.
//
// The arithmetic is that of sl_kernels.cuh (same helpers, same reduction order), so a step here
// equals a step of the multi-kernel path bit for bit.
#pragma once
#include "sl_kernels.cuh"

namespace sl {

constexpr int DEC_THREADS = 1024;
constexpr int DEC_WAVES = DEC_THREADS / 64;
constexpr int BAR_GROUP = 32;            // workgroups per first-level barrier counter
constexpr unsigned BAR_SPIN_LIMIT = 1u << 21;

struct LayerP {
  int is_linear;
  const uint16_t *input_ln, *post_ln;
  const uint32_t *in_w, *in_sb;          // GDN in_proj [12352,2048] or attention q|k|v [9216,2048]
  const uint32_t *out_w, *out_sb;        // GDN out_proj or attention o_proj [2048,4096]
  const float *conv_w, *a_log, *dt_bias;
  const uint16_t* gdn_norm_w;
  uint16_t* hist[2];
  float* state[2];
  const uint16_t *q_norm, *k_norm;
  uint16_t *kcache, *vcache;
  const uint16_t *router_w, *sgate_w;
  const uint32_t *swg_w, *swg_sb, *swu_w, *swu_sb, *swd_w, *swd_sb;
  const uint32_t *shg_w, *shg_sb, *shu_w, *shu_sb, *shd_w, *shd_sb;
  int32_t* route_inds;
  uint16_t* route_scores;
};

struct DecodeP {
  int n_layers, E, vocab, max_seq, max_tiles;
  const LayerP* layers;
  const uint32_t *emb_w, *emb_sb, *lm_w, *lm_sb;
  const uint16_t* final_norm;
  const float *rope_cos, *rope_sin;
  uint16_t *hA, *hB, *proj, *ycore, *mix, *rlogits, *sgate, *sh_act, *act, *moe_out, *normed, *logits;
  float *pm, *pl, *po, *cand_v;
  int32_t *cand_i, *tok_in, *tok_out, *st;
  unsigned long long* tstamp;   // optional: workgroup 0 records the clock after every barrier wait
  unsigned* bar;   // [0] epoch base, [32] abort flag, [64 + 32g] first-level counters, [1024] second-level counter, [2048 + 32g] release flags
};

// ---- coherent access to activations ----------------------------------------------------------------
// Agent-scope traffic goes through raw buffer instructions with the sc1 cache policy (coherent across
// the XCDs' L2s).  Unlike atomic builtins they come in 2..16-byte widths and need no wait per access.
#define SL_AG __HIP_MEMORY_SCOPE_AGENT
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;
constexpr int CO_SC1 = 16;
SL_DEV rsrc_t co_rsrc(const void* p) { return __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, 0x7fffffff, 0x00020000); }
SL_DEV uint32_t ld_co32(const void* p) { return __hip_atomic_load((const uint32_t*)p, __ATOMIC_RELAXED, SL_AG); }
SL_DEV void st_co32(void* p, uint32_t v) { __hip_atomic_store((uint32_t*)p, v, __ATOMIC_RELAXED, SL_AG); }
// element-indexed helpers; `idx` counts elements of the buffer's type
SL_DEV float ld_coh(rsrc_t r, int idx) { return h2f(__builtin_amdgcn_raw_buffer_load_b16(r, idx * 2, 0, CO_SC1)); }
SL_DEV void st_co16(rsrc_t r, int idx, uint16_t v) { __builtin_amdgcn_raw_buffer_store_b16(v, r, idx * 2, 0, CO_SC1); }
SL_DEV float ld_cof(rsrc_t r, int idx) { return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, idx * 4, 0, CO_SC1)); }
SL_DEV void st_cof(rsrc_t r, int idx, float v) { __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, idx * 4, 0, CO_SC1); }
SL_DEV void ld_co_f4(rsrc_t r, int idx, float* x) {
  const u32x4_t v = __builtin_amdgcn_raw_buffer_load_b128(r, idx * 4, 0, CO_SC1);
  x[0] = __uint_as_float(v.x); x[1] = __uint_as_float(v.y); x[2] = __uint_as_float(v.z); x[3] = __uint_as_float(v.w);
}
SL_DEV void st_co_f4(rsrc_t r, int idx, const float* x) {
  u32x4_t v; v.x = __float_as_uint(x[0]); v.y = __float_as_uint(x[1]); v.z = __float_as_uint(x[2]); v.w = __float_as_uint(x[3]);
  __builtin_amdgcn_raw_buffer_store_b128(v, r, idx * 4, 0, CO_SC1);
}
// 32 halves (64 bytes) owned by one lane, starting at half index idx
SL_DEV void ld_co_h32(rsrc_t r, int idx, float* x) {
  u32x4_t v[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) v[j] = __builtin_amdgcn_raw_buffer_load_b128(r, idx * 2 + 16 * j, 0, CO_SC1);
#pragma unroll
  for (int j = 0; j < 4; ++j) unpack8(make_uint4(v[j].x, v[j].y, v[j].z, v[j].w), x + 8 * j);
}
SL_DEV void st_co_h32(rsrc_t r, int idx, const float* x) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const uint4 q = pack8(x + 8 * j);
    u32x4_t v; v.x = q.x; v.y = q.y; v.z = q.z; v.w = q.w;
    __builtin_amdgcn_raw_buffer_store_b128(v, r, idx * 2 + 16 * j, 0, CO_SC1);
  }
}
SL_DEV void ld_co_h4(rsrc_t r, int idx, float* x) {
  const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(r, idx * 2, 0, CO_SC1);
  x[0] = lo_h(v.x); x[1] = hi_h(v.x); x[2] = lo_h(v.y); x[3] = hi_h(v.y);
}
SL_DEV void st_co_h4(rsrc_t r, int idx, const float* x) {
  u32x2_t v; v.x = pack2(x[0], x[1]); v.y = pack2(x[2], x[3]);
  __builtin_amdgcn_raw_buffer_store_b64(v, r, idx * 2, 0, CO_SC1);
}

// ---- grid barrier -----------------------------------------------------------------------------------
// Two levels: 32 workgroups share a first-level counter; the last of a group bumps the second-level
// counter; the last of all writes one release flag per group.  Waits are bounded: a workgroup that
// spins too long raises the abort flag and every workgroup leaves the kernel at its next barrier.
struct GridBar {
  unsigned* mem;
  unsigned ep;       // barriers passed so far (monotonic across launches)
  int ngroups, grp;
  bool dead;
  unsigned long long* ts;   // null unless stage timing is on
  int nts;
  unsigned long long* dbg;  // all workgroups: arrive / wait-done clocks of barriers [dbg_k0, dbg_k0 + 16)
  int kbar;
};
constexpr int DBG_K0 = 30;
// ---- activation vector in LDS ------------------------------------------------------------------------
// Packed pair i (elements 2i, 2i+1) of lane l of block b lives at xs[(16*b + i)*64 + l]; word sums at
// sxs[(4*b + j)*64 + l].
struct Lds {
  union {                                    // the staged key tile is only live while xs is not
    struct { uint32_t xs[2048]; float sxs[512]; };
    uint16_t kt[SDPA_TILE * KT_STRIDE];
  };
  float red[64];
  int ired[64];
  float q[128], k[128], v[32], gb[2];      // GDN head scratch
  int inds[8];
  float scores[8];
  float dbuf[2 * 9 * 4];
  int pf[4];                                // poll verdict slots (three in rotation) and the give-up flag
  uint32_t pub[64];                         // a stage's tagged outputs, gathered for the publishing wave
  float sq[8 * 256];                        // attention: scaled queries of one kv group
  float knew[256], vnew[256];
  float sm[8 * 64];                         // attention: per head softmax weights of the tile
  float part[16 * 64];                      // attention: half-tree score partials; router: logits and exps
  GridBar bar;
  int dead;
};
__shared__ Lds g_L;
extern __shared__ __align__(16) uint16_t g_vt[];   // dynamic: staged value tile [64][256] halves
constexpr int DEC_DYN_LDS = SDPA_TILE * 256 * 2;

// Pulls lines into this XCD's L2 (and their translations into the TLB) one stage ahead: lane i < nlines
// loads one dword of line i.  The value is never used.
SL_DEV void l2_touch(const void* p, int nlines, int lane) {
  if (lane < nlines) (void)*reinterpret_cast<const volatile uint32_t*>(reinterpret_cast<const char*>(p) + 128 * lane);
}
// Rows of K = 2048*NBLK of a 4-bit matrix: 8*NBLK lines of weights per row, up to 4 rows per call.
template <int NBLK>
SL_DEV void l2_touch_rows(const uint32_t* W, const uint32_t* SB, const size_t* rows, const bool* valid, int nrows, int lane) {
  constexpr int LPR = 8 * NBLK;                  // 128-byte lines per row
  const int r = lane / LPR, l = lane % LPR;
  if (r < nrows && valid[r]) (void)*reinterpret_cast<const volatile uint32_t*>(reinterpret_cast<const char*>(W + rows[r] * (NBLK * 256)) + 128 * l);
  if (lane < nrows && valid[lane]) (void)*reinterpret_cast<const volatile uint32_t*>(SB + rows[lane] * (NBLK * 32));
}

// ---- grid barrier on the workgroup's shared state -------------------------------------------------------
SL_DEV void bar_arrive() {
  __builtin_amdgcn_s_waitcnt(0);          // this wave's stores have been acknowledged
  __syncthreads();
  if (threadIdx.x == 0) {
    GridBar& b = g_L.bar;
    b.ep++;
    if (b.dbg && b.kbar >= DBG_K0 && b.kbar < DBG_K0 + 16) b.dbg[((b.kbar - DBG_K0) * gridDim.x + blockIdx.x) * 2] = wall_clock64();
    const unsigned old = __hip_atomic_fetch_add(&b.mem[64 + 32 * b.grp], 1u, __ATOMIC_RELAXED, SL_AG);
    if (old == b.ep * BAR_GROUP - 1) {
      const unsigned o2 = __hip_atomic_fetch_add(&b.mem[1024], 1u, __ATOMIC_RELAXED, SL_AG);
      if (o2 == b.ep * (unsigned)b.ngroups - 1)
        for (int g = 0; g < b.ngroups; ++g) st_co32(&b.mem[2048 + 32 * g], b.ep);
    }
  }
}
// Returns false if the step was aborted; every thread calls it.
SL_DEV bool bar_wait() {
  if (threadIdx.x == 0) {
    GridBar& b = g_L.bar;
    unsigned spins = 0;
    while ((int)(ld_co32(&b.mem[2048 + 32 * b.grp]) - b.ep) < 0) {
      if (++spins > BAR_SPIN_LIMIT || ((spins & 1023u) == 0 && ld_co32(&b.mem[32]) != 0)) {
        st_co32(&b.mem[32], 1u);
        g_L.dead = 1;
        break;
      }
    }
    if (b.ts && b.nts < 1000) b.ts[1 + b.nts++] = wall_clock64();
    if (b.dbg && b.kbar >= DBG_K0 && b.kbar < DBG_K0 + 16) b.dbg[((b.kbar - DBG_K0) * gridDim.x + blockIdx.x) * 2 + 1] = wall_clock64();
    b.kbar++;
  }
  __syncthreads();
  return g_L.dead == 0;
}

SL_DEV void lds_put_x(int b, int lane, const float* x) {
#pragma unroll
  for (int i = 0; i < 16; ++i) g_L.xs[(16 * b + i) * 64 + lane] = pack2(x[2 * i], x[2 * i + 1]);
  float sx[4];
  word_sums(x, sx);
#pragma unroll
  for (int j = 0; j < 4; ++j) g_L.sxs[(4 * b + j) * 64 + lane] = sx[j];
}
SL_DEV void lds_get_x(int b, int lane, uint32_t* xp, float* sx) {
#pragma unroll
  for (int i = 0; i < 16; ++i) xp[i] = g_L.xs[(16 * b + i) * 64 + lane];
#pragma unroll
  for (int j = 0; j < 4; ++j) sx[j] = g_L.sxs[(4 * b + j) * 64 + lane];
}

// Hidden prologue, run by one wave: x = half(h + r), optional rmsnorm, result into LDS.
SL_DEV void dec_hidden(const uint16_t* h_in, const uint16_t* r_in, const uint16_t* lnw, uint16_t* h_out,
                                        uint16_t* xn_out, int writer) {
  const int lane = threadIdx.x & 63;
  float x[32], w[32];
  if (lnw) load32(lnw + 32 * lane, w);
  ld_co_h32(co_rsrc(h_in), 32 * lane, x);
  if (r_in) {
    float r[32];
    ld_co_h32(co_rsrc(r_in), 32 * lane, r);
#pragma unroll
    for (int i = 0; i < 32; ++i) x[i] = f16r(x[i] + r[i]);
  }
  if (writer && h_out) st_co_h32(co_rsrc(h_out), 32 * lane, x);
  if (lnw) {
    const float inv = inv_rms_2048(x);
#pragma unroll
    for (int i = 0; i < 32; ++i) x[i] = f16r(w[i] * f16r(x[i] * inv));
  }
  if (writer && xn_out) st_co_h32(co_rsrc(xn_out), 32 * lane, x);
  lds_put_x(0, lane, x);
}

// ---- weight prefetch: R rows of K = 2048*NBLK held in registers ----------------------------------------
template <int NBLK, int R>
struct WRegs {
  uint4 w[R][NBLK];
  uint32_t sb[R][NBLK];
};
template <int NBLK>
SL_DEV void wload_row(uint4* w, uint32_t* sb, const uint32_t* __restrict__ W, const uint32_t* __restrict__ SB, size_t row,
                      bool valid, int lane) {
#pragma unroll
  for (int b = 0; b < NBLK; ++b) {
    if (valid) {
      w[b] = ld16(W + row * (NBLK * 256) + b * 256 + 4 * lane);
      sb[b] = SB[row * (NBLK * 32) + b * 32 + (lane >> 1)];
    } else {
      w[b] = make_uint4(0, 0, 0, 0);
      sb[b] = 0;
    }
  }
}
struct F4 { float v[4]; };
struct F2 { float v[2]; };
// The three dot shapes of a step, each compiled once (arguments travel in registers):
// 4 rows x 2048, 2 rows x 2048, 1 row x 4096.
SL_DEV F4 dot_1x4_(uint4 w0, uint4 w1, uint4 w2, uint4 w3, uint32_t s0, uint32_t s1, uint32_t s2, uint32_t s3) {
  const int lane = threadIdx.x & 63;
  uint32_t x[16]; float sx[4];
  lds_get_x(0, lane, x, sx);
  F4 o;
  o.v[0] = tree_sum<64>(quad_term(w0, s0, x, sx));
  o.v[1] = tree_sum<64>(quad_term(w1, s1, x, sx));
  o.v[2] = tree_sum<64>(quad_term(w2, s2, x, sx));
  o.v[3] = tree_sum<64>(quad_term(w3, s3, x, sx));
  return o;
}
SL_DEV F2 dot_1x2_(uint4 w0, uint4 w1, uint32_t s0, uint32_t s1) {
  const int lane = threadIdx.x & 63;
  uint32_t x[16]; float sx[4];
  lds_get_x(0, lane, x, sx);
  F2 o;
  o.v[0] = tree_sum<64>(quad_term(w0, s0, x, sx));
  o.v[1] = tree_sum<64>(quad_term(w1, s1, x, sx));
  return o;
}
SL_DEV float dot_2x1_(uint4 w0, uint4 w1, uint32_t s0, uint32_t s1) {
  const int lane = threadIdx.x & 63;
  uint32_t x[16]; float sx[4];
  lds_get_x(0, lane, x, sx);
  float acc = quad_term(w0, s0, x, sx);
  lds_get_x(1, lane, x, sx);
  acc = acc + quad_term(w1, s1, x, sx);
  return tree_sum<64>(acc);
}
SL_DEV F4 dot_1x4(const WRegs<1, 4>& r) { return dot_1x4_(r.w[0][0], r.w[1][0], r.w[2][0], r.w[3][0], r.sb[0][0], r.sb[1][0], r.sb[2][0], r.sb[3][0]); }
SL_DEV F2 dot_1x2(const WRegs<1, 2>& r) { return dot_1x2_(r.w[0][0], r.w[1][0], r.sb[0][0], r.sb[1][0]); }
SL_DEV float dot_2x1(const WRegs<2, 1>& r) { return dot_2x1_(r.w[0][0], r.w[0][1], r.sb[0][0], r.sb[0][1]); }

// ---- stages ---------------------------------------------------------------------------------------------
#define DEC_IDS const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6; \
                const int wg = blockIdx.x, G = gridDim.x, NW = G * DEC_WAVES, gw = wg * DEC_WAVES + wave; \
                (void)tid; (void)lane; (void)wave; (void)wg; (void)G; (void)NW; (void)gw

// stage 1: input norm + in-projection (GDN qkv|z|b|a or attention q|k|v); wave gw owns rows gw + j*NW
SL_DEV bool stage_in(const DecodeP& P, const LayerP& Y, int li, int pos) {
  DEC_IDS;
  const int N = Y.is_linear ? SL_GDN_IN_N : SL_ATT_QKV_N;
  WRegs<1, 4> wr;
  bool valid[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) valid[j] = gw + j * NW < N;
  // the wave whose thread 0 polls the barrier keeps its load queue empty so that the poll is not
  // returned behind 4 KB of weights; it fetches its rows after the wait (they are in L2 by then)
  if (wave != 0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) wload_row<1>(wr.w[j], wr.sb[j], Y.in_w, Y.in_sb, (size_t)(valid[j] ? gw + j * NW : 0), valid[j], lane);
  }
  // next stage's first touches: this workgroup's recurrent-state rows, or its key/value tile
  if (Y.is_linear) {
    if (wg < 256 && wave < 8) {
      const int hv = wg >> 3, dvb = wg & 7, par = P.st[1 + li];
      l2_touch(Y.state[par] + ((size_t)hv * 128 + dvb * 16 + wave * 2) * 128, 8, lane);
    }
  } else {
    const int nt = (pos + SDPA_TILE) / SDPA_TILE;
    if (wg < nt * SL_ATT_KV) {
      // rows already in the arena only (the row of this step is written later): 4 rows x 4 lines per wave
      const int tile = wg >> 1, kvh = wg & 1;
      const int row = tile * SDPA_TILE + wave * 4 + (lane >> 2);
      if (lane < 16 && row < pos) {
        const size_t off = ((size_t)kvh * P.max_seq + row) * 256 + (size_t)(lane & 3) * 64;
        (void)*reinterpret_cast<const volatile uint32_t*>(Y.kcache + off);
        (void)*reinterpret_cast<const volatile uint32_t*>(Y.vcache + off);
      }
    }
  }
  if (li > 0 && !bar_wait()) return false;
  if (wave == 0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) wload_row<1>(wr.w[j], wr.sb[j], Y.in_w, Y.in_sb, (size_t)(valid[j] ? gw + j * NW : 0), valid[j], lane);
    dec_hidden(P.hA, li > 0 ? P.moe_out : nullptr, Y.input_ln, P.hB, nullptr, wg == 0);
  }
  __syncthreads();
  const F4 o = dot_1x4(wr);
  if (lane == 0) {
    const rsrc_t rp = co_rsrc(P.proj);
#pragma unroll
    for (int j = 0; j < 4; ++j) if (valid[j]) st_co16(rp, gw + j * NW, f2h(o.v[j]));
  }
  bar_arrive();
  return true;
}

// GDN stage 2: conv + prep + gated delta rule; 256 units of (value head, 16 state rows)
SL_DEV bool stage_gdn(const DecodeP& P, const LayerP& Y, int li) {
  DEC_IDS;
  Lds& L = g_L;
  const int par = P.st[1 + li];
  const uint16_t* hin = Y.hist[par];
  uint16_t* hout = Y.hist[par ^ 1];
  for (int u = wg; u < 256; u += G) {
    const int hv = u >> 3, dvb = u & 7, hk = hv >> 1;
    const int half = lane >> 5, l32 = lane & 31;
    float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (wave < 8) {
      const int dv = dvb * 16 + wave * 2 + half;
      const float4 v4 = *reinterpret_cast<const float4*>(Y.state[par] + ((size_t)hv * 128 + dv) * 128 + 4 * l32);
      s[0] = v4.x; s[1] = v4.y; s[2] = v4.z; s[3] = v4.w;
    }
    // conv taps of the history do not depend on this step: fetch them before the wait
    int ch = -1;
    if (tid < 128) ch = hk * 128 + tid;
    else if (tid < 256) ch = 2048 + hk * 128 + (tid - 128);
    else if (tid < 272) ch = 4096 + hv * 128 + dvb * 16 + (tid - 256);
    float tap[3] = {0.0f, 0.0f, 0.0f}, cw[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (ch >= 0) {
#pragma unroll
      for (int k = 0; k < 3; ++k) tap[k] = h2f(hin[k * SL_CONV_DIM + ch]);
#pragma unroll
      for (int k = 0; k < 4; ++k) cw[k] = Y.conv_w[ch * 4 + k];
    }
    if (u == wg) {
      const size_t orow[1] = {(size_t)(gw < H ? gw : 0)}; const bool ov[1] = {gw < H};
      l2_touch_rows<2>(Y.out_w, Y.out_sb, orow, ov, 1, lane);
      if (!bar_wait()) return false;
    }
    float newest = 0.0f;
    if (ch >= 0) {
      newest = ld_coh(co_rsrc(P.proj), ch);
      float acc = 0.0f;
#pragma unroll
      for (int k = 0; k < 3; ++k) acc = fmaf(tap[k], cw[k], acc);
      acc = fmaf(newest, cw[3], acc);
      const float c = f16r(acc * sigmoid32(acc));
      if (tid < 128) L.q[tid] = c; else if (tid < 256) L.k[tid - 128] = c; else L.v[tid - 256] = c;
    }
    __syncthreads();
    if (wave < 2) {
      float* buf = wave ? L.k : L.q;
      const float x0 = buf[2 * lane], x1 = buf[2 * lane + 1];
      float ss = fmaf(x1, x1, fmaf(x0, x0, 0.0f));
      ss = tree_sum<64>(ss);
      const float inv = 1.0f / sqrtf(ss / 128.0f + EPS);
      const float sc = wave ? f16r(0.08838834764831845f) : f16r(0.0078125f);
      const float y0 = f16r(sc * f16r(x0 * inv)), y1 = f16r(sc * f16r(x1 * inv));
      buf[2 * lane] = y0; buf[2 * lane + 1] = y1;
    } else if (tid == 128) {
      const rsrc_t rp = co_rsrc(P.proj);
      const float bP = ld_coh(rp, 12288 + hv), aP = ld_coh(rp, 12320 + hv);
      L.gb[0] = exp_c(-(exp_c(Y.a_log[hv]) * softplus_c(aP + Y.dt_bias[hv])));
      L.gb[1] = sigmoid16(bP);
    }
    __syncthreads();
    if (wave < 8) {
      const float g = L.gb[0], beta = L.gb[1];
      const int dvl = wave * 2 + half;
      float kk[4], qq[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { kk[i] = L.k[4 * l32 + i]; qq[i] = L.q[4 * l32 + i]; }
      float acc = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; ++i) { s[i] = s[i] * g; acc = fmaf(s[i], kk[i], acc); }
      const float kv = tree_sum<32>(acc);
      const float delta = (L.v[dvl] - kv) * beta;
      acc = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; ++i) { s[i] = fmaf(kk[i], delta, s[i]); acc = fmaf(s[i], qq[i], acc); }
      const float y = tree_sum<32>(acc);
      const int dv = dvb * 16 + dvl;
      if (l32 == 0) st_co16(co_rsrc(P.ycore), hv * 128 + dv, f2h(y));
      *reinterpret_cast<float4*>(Y.state[par ^ 1] + ((size_t)hv * 128 + dv) * 128 + 4 * l32) = make_float4(s[0], s[1], s[2], s[3]);
    }
    // history shift: rows 1,2 of the old history and the new sample
    if (ch >= 0 && (tid >= 256 || ((hv & 1) == 0 && dvb == 0))) {
      hout[ch] = f2h(tap[1]);
      hout[SL_CONV_DIM + ch] = f2h(tap[2]);
      hout[2 * SL_CONV_DIM + ch] = f2h(newest);
    }
    __syncthreads();
  }
  if (wg >= 256 && !bar_wait()) return false;      // workgroups without a unit still pass the barrier
  bar_arrive();
  return true;
}

// K = 4096 projection: GDN out_proj with the gated rmsnorm as prologue, or attention o_proj after the
// tile merge (done by workgroup 0 in an extra barrier phase).
SL_DEV bool stage_out(const DecodeP& P, const LayerP& Y, int nt) {
  DEC_IDS;
  const float NEG = -__int_as_float(0x7f800000);
  WRegs<2, 1> wr;
  const bool valid = gw < H;
  wload_row<2>(wr.w[0], wr.sb[0], Y.out_w, Y.out_sb, (size_t)(valid ? gw : 0), valid, lane);
  if (gw <= P.E) l2_touch((gw < P.E ? Y.router_w + (size_t)gw * H : Y.sgate_w), 32, lane);
  if (gw >= 512 && gw < 1024) {
    const size_t pr[1] = {(size_t)(gw - 512)}; const bool pv[1] = {true};
    l2_touch_rows<1>(Y.shg_w, Y.shg_sb, pr, pv, 1, lane);
    l2_touch_rows<1>(Y.shu_w, Y.shu_sb, pr, pv, 1, lane);
  }
  if (!bar_wait()) return false;
  if (!Y.is_linear) {
    if (wg == 0) {
      // merge the attention tiles in order with the global max; out = half(O/L) * sigmoid16(gate)
      const int h = wave;
      const int base = h * P.max_tiles;
      const rsrc_t rpm = co_rsrc(P.pm), rpl = co_rsrc(P.pl), rpo = co_rsrc(P.po);
      float Mx = NEG;
      for (int t = 0; t < nt; ++t) Mx = fmaxf(Mx, ld_cof(rpm, base + t));
      float Ls = 0.0f, O[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      for (int t = 0; t < nt; ++t) {
        const float f = exp_c(ld_cof(rpm, base + t) - Mx);
        Ls = fmaf(ld_cof(rpl, base + t), f, Ls);
        float o4[4];
        ld_co_f4(rpo, (base + t) * 256 + 4 * lane, o4);
#pragma unroll
        for (int i = 0; i < 4; ++i) O[i] = fmaf(o4[i], f, O[i]);
      }
      float gt[4], r[4];
      ld_co_h4(co_rsrc(P.proj), h * 512 + 256 + 4 * lane, gt);
#pragma unroll
      for (int i = 0; i < 4; ++i) r[i] = f16r(f16r(O[i] / Ls) * sigmoid16(gt[i]));
      st_co_h4(co_rsrc(P.ycore), h * 256 + 4 * lane, r);
    }
    bar_arrive();
    if (!bar_wait()) return false;
  }
  {
    // every thread prepares 4 consecutive elements of the 4096-long activation (a value head spans 32 lanes)
    const int e0 = 256 * wave + 4 * lane;
    float out[4];
    ld_co_h4(co_rsrc(P.ycore), e0, out);
    if (Y.is_linear) {
      float z[4], nw[4];
      ld_co_h4(co_rsrc(P.proj), 8192 + e0, z);
      const uint2 wraw = *reinterpret_cast<const uint2*>(Y.gdn_norm_w + (e0 & 127));
      nw[0] = lo_h(wraw.x); nw[1] = hi_h(wraw.x); nw[2] = lo_h(wraw.y); nw[3] = hi_h(wraw.y);
      const float la = fmaf(out[1], out[1], fmaf(out[0], out[0], 0.0f));
      const float lb = fmaf(out[3], out[3], fmaf(out[2], out[2], 0.0f));
      const float ss = tree_sum<32>(la + lb);
      const float inv = 1.0f / sqrtf(ss / 128.0f + EPS);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float nrm = f16r(nw[i] * f16r(out[i] * inv));
        out[i] = f16r((z[i] * sigmoid32(z[i])) * nrm);
      }
    }
    const int b = e0 >> 11, r = e0 & 2047, lo = r >> 5, i0 = r & 31;
    g_L.xs[(16 * b + (i0 >> 1)) * 64 + lo] = pack2(out[0], out[1]);
    g_L.xs[(16 * b + (i0 >> 1) + 1) * 64 + lo] = pack2(out[2], out[3]);
    // left-to-right sum of each word of 8: the even lane starts it, the odd lane finishes it
    float sfirst = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) sfirst = sfirst + out[i];
    float srest = __shfl_up(sfirst, 1, 64);
#pragma unroll
    for (int i = 0; i < 4; ++i) srest = srest + out[i];
    if (lane & 1) g_L.sxs[(4 * b + (i0 >> 3)) * 64 + lo] = srest;
  }
  __syncthreads();
  const float o = dot_2x1(wr);
  if (lane == 0 && valid) st_co16(co_rsrc(P.mix), gw, f2h(o));
  bar_arrive();
  return true;
}

// 8 leaves (32 dims) of the score tree of one key against one query head: balanced sub-tree.
SL_DEV float score_leaf8(const uint16_t* kr, const float* qh) {
  float n[8];
#pragma unroll
  for (int l = 0; l < 8; ++l) {
    const uint2 kraw = *reinterpret_cast<const uint2*>(kr + 4 * l);
    float node = fmaf(qh[4 * l], lo_h(kraw.x), 0.0f);
    node = fmaf(qh[4 * l + 1], hi_h(kraw.x), node);
    node = fmaf(qh[4 * l + 2], lo_h(kraw.y), node);
    n[l] = fmaf(qh[4 * l + 3], hi_h(kraw.y), node);
  }
  return ((n[0] + n[1]) + (n[2] + n[3])) + ((n[4] + n[5]) + (n[6] + n[7]));
}

// attention stage 2: q/k prep, KV append, tile pass; units of (key tile, kv head)
SL_DEV bool stage_sdpa(const DecodeP& P, const LayerP& Y, int pos) {
  DEC_IDS;
  Lds& L = g_L;
  const float NEG = -__int_as_float(0x7f800000);
  const int N = pos + 1, nt = (N + SDPA_TILE - 1) / SDPA_TILE;
  {
    const size_t orow[1] = {(size_t)(gw < H ? gw : 0)}; const bool ov[1] = {gw < H};
    l2_touch_rows<2>(Y.out_w, Y.out_sb, orow, ov, 1, lane);     // o_proj row for the stage after next
  }
  if (!bar_wait()) return false;
  for (int u = wg; u < nt * SL_ATT_KV; u += G) {
    const int tile = u >> 1, kvh = u & 1;
    const int j0 = tile * SDPA_TILE, nk = min(SDPA_TILE, N - j0);
    const bool has_new = (pos >= j0) && (pos < j0 + SDPA_TILE);
    // stage the tile's old keys and values: 1024 threads x 16 bytes = 32 rows per pass
    const uint16_t* kbase = Y.kcache + ((size_t)kvh * P.max_seq + j0) * 256;
    const uint16_t* vbase = Y.vcache + ((size_t)kvh * P.max_seq + j0) * 256;
#pragma unroll
    for (int it = 0; it < 2; ++it) {
      const int row = it * 32 + (tid >> 5), c8 = (tid & 31) * 8;
      if (row < nk && j0 + row != pos) {
        st16(&L.kt[row * KT_STRIDE + c8], ld16(kbase + (size_t)row * 256 + c8));
        st16(&g_vt[row * 256 + c8], ld16(vbase + (size_t)row * 256 + c8));
      }
    }
    // waves 0..7: query heads of the group; wave 8: the new key; wave 9: the new value
    if (wave < 9) {
      const bool isq = wave < 8;
      const int src = isq ? (kvh * 8 + wave) * 512 : 8192 + kvh * 256;
      const uint16_t* nwp = isq ? Y.q_norm : Y.k_norm;
      float xv[4], wv[4];
      ld_co_h4(co_rsrc(P.proj), src + 4 * lane, xv);
      const uint2 wraw = *reinterpret_cast<const uint2*>(nwp + 4 * lane);
      wv[0] = lo_h(wraw.x); wv[1] = hi_h(wraw.x); wv[2] = lo_h(wraw.y); wv[3] = hi_h(wraw.y);
      float ss = 0.0f;
#pragma unroll
      for (int i = 0; i < 4; ++i) ss = fmaf(xv[i], xv[i], ss);
      ss = tree_sum<64>(ss);
      const float inv = 1.0f / sqrtf(ss / 256.0f + EPS);
      float* dst = isq ? &L.sq[wave * 256] : L.knew;
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[4 * lane + i] = f16r(wv[i] * f16r(xv[i] * inv));
      // partial rotary on the first 64 dims (lanes 0..15); pairs (i, i+32)
      float o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = dst[4 * lane + i];
      if (lane < 16) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int d = 4 * lane + i, ii = d & 31;
          const float c = P.rope_cos[(size_t)pos * 32 + ii], sn = P.rope_sin[(size_t)pos * 32 + ii];
          const float x0 = dst[ii], x1 = dst[ii + 32];
          o[i] = (d < 32) ? f16r(fmaf(-x1, sn, x0 * c)) : f16r(fmaf(x1, c, x0 * sn));
        }
      }
      // every lane of the wave has read dst before any lane overwrites it (one wave, in-order LDS)
#pragma unroll
      for (int i = 0; i < 4; ++i) dst[4 * lane + i] = isq ? 0.0625f * o[i] : o[i];
      if (!isq && has_new) {
        st_co_h4(co_rsrc(Y.kcache + ((size_t)kvh * P.max_seq + pos) * 256), 4 * lane, o);
        *reinterpret_cast<uint2*>(&L.kt[(pos - j0) * KT_STRIDE + 4 * lane]) = make_uint2(pack2(o[0], o[1]), pack2(o[2], o[3]));
      }
    } else if (wave == 9) {
      const u32x2_t v = __builtin_amdgcn_raw_buffer_load_b64(co_rsrc(P.proj), (8192 + 512 + kvh * 256 + 4 * lane) * 2, 0, CO_SC1);
      if (has_new) {
        __builtin_amdgcn_raw_buffer_store_b64(v, co_rsrc(Y.vcache + ((size_t)kvh * P.max_seq + pos) * 256), 8 * lane, 0, CO_SC1);
        *reinterpret_cast<uint2*>(&g_vt[(pos - j0) * 256 + 4 * lane]) = make_uint2(v.x, v.y);
      }
    }
    __syncthreads();
    // scores: wave (head, half) takes the 32 leaves of its half of the 256 dims, lane j is key j
    {
      const int h = wave >> 1, half = wave & 1;
      const uint16_t* kr = &L.kt[(lane < nk ? lane : 0) * KT_STRIDE + 128 * half];
      const float* qh = &L.sq[h * 256 + 128 * half];
      const float g0 = score_leaf8(kr, qh), g1 = score_leaf8(kr + 32, qh + 32);
      const float g2 = score_leaf8(kr + 64, qh + 64), g3 = score_leaf8(kr + 96, qh + 96);
      L.part[wave * 64 + lane] = (g0 + g1) + (g2 + g3);
    }
    __syncthreads();
    if ((wave & 1) == 0) {
      const int h = wave >> 1;
      const float dotv = L.part[wave * 64 + lane] + L.part[(wave + 1) * 64 + lane];
      const float sc = (lane < nk) ? dotv : NEG;
      const float mx = tree_max<64>(sc);
      const float p = (lane < nk) ? exp_c(sc - mx) : 0.0f;
      const float l = tree_sum<64>(p);
      L.sm[h * 64 + lane] = p;
      const int head = kvh * 8 + h;
      if (lane == 0) { st_cof(co_rsrc(P.pm), head * P.max_tiles + tile, mx); st_cof(co_rsrc(P.pl), head * P.max_tiles + tile, l); }
    }
    __syncthreads();
    {
      // o = fmaf chain over the tile's keys in order; wave (head, half) owns 128 dims, 2 per lane
      const int h = wave >> 1, half = wave & 1;
      float o0 = 0.0f, o1 = 0.0f;
      const uint16_t* vt = &g_vt[128 * half + 2 * lane];
      const float* pw = &L.sm[h * 64];
      for (int j = 0; j < nk; ++j) {
        const uint32_t vv = *reinterpret_cast<const uint32_t*>(vt + j * 256);
        const float pj = pw[j];
        o0 = fmaf(pj, lo_h(vv), o0);
        o1 = fmaf(pj, hi_h(vv), o1);
      }
      const int head = kvh * 8 + h;
      u32x2_t ov; ov.x = __float_as_uint(o0); ov.y = __float_as_uint(o1);
      __builtin_amdgcn_raw_buffer_store_b64(ov, co_rsrc(P.po), ((head * P.max_tiles + tile) * 256 + 128 * half + 2 * lane) * 4, 0, CO_SC1);
    }
    __syncthreads();
  }
  bar_arrive();
  return true;
}

// MoE stage A: post norm; router rows (waves 0..E-1), shared-gate row (wave E), shared gate/up pairs (waves 512..1023)
SL_DEV bool stage_moe_a(const DecodeP& P, const LayerP& Y) {
  DEC_IDS;
  const bool is_dense = gw <= P.E;
  const bool is_pair = gw >= 512 && gw < 1024;
  float dw[32];
  WRegs<1, 2> wr;
  const size_t prow = is_pair ? (size_t)(gw - 512) : 0;
  wload_row<1>(wr.w[0], wr.sb[0], Y.shg_w, Y.shg_sb, prow, is_pair, lane);
  wload_row<1>(wr.w[1], wr.sb[1], Y.shu_w, Y.shu_sb, prow, is_pair, lane);
  if (is_dense) load32((gw < P.E ? Y.router_w + (size_t)gw * H : Y.sgate_w) + 32 * lane, dw);
  if (!bar_wait()) return false;
  if (wave == 0) dec_hidden(P.hB, P.mix, Y.post_ln, P.hA, nullptr, wg == 0);
  __syncthreads();
  if (is_dense) {
    uint32_t xp[16]; float sx[4];
    lds_get_x(0, lane, xp, sx);
    float acc = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) { acc = fmaf(lo_h(xp[i]), dw[2 * i], acc); acc = fmaf(hi_h(xp[i]), dw[2 * i + 1], acc); }
    acc = tree_sum<64>(acc);
    if (lane == 0) { if (gw < P.E) st_co16(co_rsrc(P.rlogits), gw, f2h(acc)); else st_co16(co_rsrc(P.sgate), 0, f2h(acc)); }
  }
  if (is_pair) {
    const F2 gu = dot_1x2(wr);
    if (lane == 0) st_co16(co_rsrc(P.sh_act), (int)prow, f2h(swiglu16(f16r(gu.v[0]), f16r(gu.v[1]))));
  }
  bar_arrive();
  return true;
}

// MoE stage B: routing (one wave per workgroup) + routed gate/up + SwiGLU; xs still holds the post-normed row
SL_DEV bool stage_moe_b(const DecodeP& P, const LayerP& Y) {
  DEC_IDS;
  Lds& L = g_L;
  const float NEG = -__int_as_float(0x7f800000);
  if (!bar_wait()) return false;
  // Router on the whole workgroup.  The 8 selected experts in routing order are the experts of rank 0..7
  // under "larger logit first, lower index first on ties", so each expert's rank is counted directly:
  // threads (part, e) count the experts of one quarter that precede e; wave 0 forms the softmax sums.
  float* lg = L.part;            // [256] logits
  float* ex = L.part + 256;      // [256] exp(logit - max)
  int* cnt = reinterpret_cast<int*>(g_vt);           // [4][256] partial rank counts (the value tile is idle here)
  if (tid < 256) lg[tid] = (tid < P.E) ? ld_coh(co_rsrc(P.rlogits), tid) : NEG;
  __syncthreads();
  {
    const int e = tid & 255, part = tid >> 8;
    const float me = lg[e];
    int c = 0;
#pragma unroll 8
    for (int j = 64 * part; j < 64 * part + 64; ++j) {
      const float o = lg[j];
      c += (o > me || (o == me && j < e)) ? 1 : 0;
    }
    cnt[part * 256 + e] = c;                       // the four parts of an expert live in different waves
  }
  if (wave == 0) {
    float v[4], x4[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = lg[4 * lane + i];
    const float mx = tree_max<64>(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])));
#pragma unroll
    for (int i = 0; i < 4; ++i) { x4[i] = (4 * lane + i < P.E) ? exp_c(v[i] - mx) : 0.0f; ex[4 * lane + i] = x4[i]; }
    const float Z = tree_sum<64>(((x4[0] + x4[1]) + x4[2]) + x4[3]);
    if (lane == 0) L.gb[0] = Z;
  }
  __syncthreads();
  if (tid < 256) {
    const int rank = cnt[tid] + cnt[256 + tid] + cnt[512 + tid] + cnt[768 + tid];
    if (rank < 8 && tid < P.E) { L.inds[rank] = tid; L.scores[rank] = f16r(ex[tid] / L.gb[0]); }
  }
  __syncthreads();
  if (tid == 0) {
    float ss = 0.0f;
    for (int k = 0; k < 8; ++k) ss = f16r(ss + L.scores[k]);
    for (int k = 0; k < 8; ++k) L.scores[k] = f16r(L.scores[k] / ss);
    if (wg == 0) for (int k = 0; k < 8; ++k) { Y.route_inds[k] = L.inds[k]; Y.route_scores[k] = f2h(L.scores[k]); }
  }
  // this wave's gate/up pair (issued as soon as the indices are known), then next stage's down rows
  const int p = gw;                      // 8*512 pairs over NW = 4096 waves
  WRegs<1, 2> wr;
  int k = 0, i = 0;
  const bool active = p < 8 * 512;
  if (active) {
    k = p >> 9; i = p & 511;
    const size_t row = (size_t)L.inds[k] * 512 + i;
    wload_row<1>(wr.w[0], wr.sb[0], Y.swg_w, Y.swg_sb, row, true, lane);
    wload_row<1>(wr.w[1], wr.sb[1], Y.swu_w, Y.swu_sb, row, true, lane);
  }
  {
    // down-projection rows of this workgroup's units for stage C: 4 rows x 256 bytes per unit
#pragma unroll
    for (int qq = 0; qq < 2; ++qq) {
      const int un = wave + 16 * qq, ql = un / 9, slot = un % 9;
      if (ql < 2 && slot < 8) {
        const size_t row = (size_t)L.inds[slot] * 2048 + (size_t)(wg * 2 + ql) * 4;
        l2_touch(Y.swd_w + row * 64, 8, lane);
        if (lane == 8) (void)*reinterpret_cast<const volatile uint32_t*>(Y.swd_sb + row * 8);
      }
    }
  }
  __syncthreads();                       // scores are final before stage C reads them
  if (active) {
    const F2 gu = dot_1x2(wr);
    if (lane == 0) st_co16(co_rsrc(P.act), k * 512 + i, f2h(swiglu16(f16r(gu.v[0]), f16r(gu.v[1]))));
  }
  bar_arrive();
  return true;
}

// MoE stage C: down-projections, half-precision combine in routing order, gated shared add.
// Units (quad of 4 outputs, slot): slots 0..7 routed experts, slot 8 shared; 2 quads per workgroup.
SL_DEV bool stage_moe_c(const DecodeP& P, const LayerP& Y, const uint32_t* next_w, const uint32_t* next_sb,
                                         int next_n, int next_contig) {
  DEC_IDS;
  Lds& L = g_L;
  const int sub = lane >> 4, li16 = lane & 15;
  {
    // first touches of the next projection: rows gw + j*NW (layer in-proj) or a contiguous chunk (lm_head)
    size_t rows[4]; bool rv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long r = next_contig ? (long)gw * 64 + j : (long)gw + (long)j * NW;
      rv[j] = r < next_n; rows[j] = rv[j] ? (size_t)r : 0;
    }
    l2_touch_rows<1>(next_w, next_sb, rows, rv, 4, lane);
  }
  uint4 shw[2]; uint32_t shsb[2];
#pragma unroll
  for (int qq = 0; qq < 2; ++qq) {
    const int un = wave + 16 * qq, ql = un / 9, slot = un % 9;
    const int quad = wg * 2 + ql;
    shw[qq] = make_uint4(0, 0, 0, 0); shsb[qq] = 0;
    if (ql < 2 && slot == 8) {
      const size_t row = (size_t)quad * 4 + sub;
      shw[qq] = ld16(Y.shd_w + row * 64 + 4 * li16);
      shsb[qq] = Y.shd_sb[row * 8 + (li16 >> 1)];
    }
  }
  if (!bar_wait()) return false;
#pragma unroll
  for (int qq = 0; qq < 2; ++qq) {
    const int un = wave + 16 * qq, ql = un / 9, slot = un % 9;
    const int quad = wg * 2 + ql;
    if (ql < 2) {
      float x[32], sx[4];
      uint32_t xp[16];
      ld_co_h32(co_rsrc(slot < 8 ? P.act + slot * 512 : P.sh_act), 32 * li16, x);
      word_sums(x, sx);
      pack_x(x, xp);
      float d;
      if (slot < 8) {
        const size_t row = (size_t)L.inds[slot] * 2048 + (size_t)quad * 4 + sub;
        d = qdot512(Y.swd_w, Y.swd_sb, row, li16, xp, sx);
      } else {
        d = tree_sum<16>(quad_term(shw[qq], shsb[qq], xp, sx));
      }
      if (li16 == 0) L.dbuf[(ql * 9 + slot) * 4 + sub] = f16r(d);
    }
  }
  __syncthreads();
  if (tid < 8) {
    const int ql = tid >> 2, sb4 = tid & 3;
    const int quad = wg * 2 + ql;
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; ++k) acc = f16r(acc + f16r(L.dbuf[(ql * 9 + k) * 4 + sb4] * L.scores[k]));
    const float s = sigmoid16(ld_coh(co_rsrc(P.sgate), 0));
    st_co16(co_rsrc(P.moe_out), quad * 4 + sb4, f2h(f16r(acc + f16r(s * L.dbuf[(ql * 9 + 8) * 4 + sb4]))));
  }
  bar_arrive();
  return true;
}

// head: final norm + lm_head + argmax.  Each wave owns a contiguous chunk of 64 vocabulary rows, 4 at a
// time with the next group prefetched; candidates are reduced per workgroup, then by workgroup 0.
SL_DEV bool stage_head(const DecodeP& P, int pos, int out_off, int feed) {
  DEC_IDS;
  Lds& L = g_L;
  const float NEG = -__int_as_float(0x7f800000);
  const int nchunks = (P.vocab + 63) / 64;
  float bv = NEG; int bi = 0x7fffffff;
  WRegs<1, 4> cur, nxt;
  auto load_group = [&](WRegs<1, 4>& r, int chunk, int g4) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long row = (long)chunk * 64 + g4 * 4 + j;
      const bool v = chunk < nchunks && row < P.vocab;
      wload_row<1>(r.w[j], r.sb[j], P.lm_w, P.lm_sb, (size_t)(v ? row : 0), v, lane);
    }
  };
  load_group(cur, gw, 0);
  if (!bar_wait()) return false;
  if (wave == 0) dec_hidden(P.hA, P.moe_out, P.final_norm, P.hB, P.normed, wg == 0);
  __syncthreads();
  for (int chunk = gw; chunk < nchunks; chunk += NW) {
#pragma unroll 1
    for (int g4 = 0; g4 < 16; ++g4) {
      int nchunk = chunk, ng = g4 + 1;
      if (ng == 16) { ng = 0; nchunk = chunk + NW; }
      load_group(nxt, nchunk, ng);
      const F4 o = dot_1x4(cur);
      const long r0 = (long)chunk * 64 + g4 * 4;
      if (r0 < P.vocab) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float v = f16r(o.v[j]);
          if (v > bv) { bv = v; bi = (int)(r0 + j); }
        }
        if (lane == 0) *reinterpret_cast<uint2*>(P.logits + r0) = make_uint2(pack2(o.v[0], o.v[1]), pack2(o.v[2], o.v[3]));
      }
      cur = nxt;
    }
  }
  if (lane == 0) { L.red[wave] = bv; L.ired[wave] = bi; }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < DEC_WAVES; ++w)
      if (L.red[w] > bv || (L.red[w] == bv && L.ired[w] < bi)) { bv = L.red[w]; bi = L.ired[w]; }
    st_cof(co_rsrc(P.cand_v), wg, bv);
    st_cof(co_rsrc(P.cand_i), wg, __int_as_float(bi));
  }
  bar_arrive();
  if (!bar_wait()) return false;
  if (wg == 0) {
    float v = NEG; int i = 0x7fffffff;
    if (tid < G) { v = ld_cof(co_rsrc(P.cand_v), tid); i = __float_as_int(ld_cof(co_rsrc(P.cand_i), tid)); }
#pragma unroll
    for (int msk = 1; msk < 64; msk <<= 1) {
      const float ov = __shfl_xor(v, msk, 64); const int oi = __shfl_xor(i, msk, 64);
      if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
    }
    __syncthreads();
    if (lane == 0) { L.red[wave] = v; L.ired[wave] = i; }
    __syncthreads();
    if (tid == 0) {
      for (int w = 1; w < DEC_WAVES; ++w)
        if (L.red[w] > v || (L.red[w] == v && L.ired[w] < i)) { v = L.red[w]; i = L.ired[w]; }
      P.tok_out[out_off] = i;
      if (feed) P.tok_in[0] = i;
      P.st[0] = pos + 1;
      GridBar& b = L.bar;
      st_co32(b.mem, b.ep);
      if (b.ts) { b.ts[1 + b.nts++] = wall_clock64(); b.ts[0] = (unsigned long long)b.nts; }
    }
    for (int l = tid; l < P.n_layers; l += DEC_THREADS) P.st[1 + l] ^= 1;
  }
  return true;
}

// ---- the kernel: hA already holds the embedded token row (k_embed) ----------------------------------------
__global__ __launch_bounds__(DEC_THREADS) void k_decode(const DecodeP* __restrict__ Pp, int out_off, int feed) {
  const DecodeP& P = *Pp;
  if (threadIdx.x == 0) {
    GridBar& b = g_L.bar;
    b.mem = P.bar;
    b.ep = ld_co32(P.bar);
    b.ngroups = gridDim.x / BAR_GROUP;
    b.grp = blockIdx.x / BAR_GROUP;
    b.ts = (P.tstamp && blockIdx.x == 0) ? P.tstamp : nullptr;
    b.nts = 0;
    b.dbg = P.tstamp ? P.tstamp + 2048 : nullptr;
    b.kbar = 0;
    if (b.ts) b.ts[1 + b.nts++] = wall_clock64();
    g_L.dead = 0;
  }
  __syncthreads();
  const int pos = P.st[0];
  for (int li = 0; li < P.n_layers; ++li) {
    const LayerP& Y = P.layers[li];
    if (!stage_in(P, Y, li, pos)) return;
    if (Y.is_linear) {
      if (!stage_gdn(P, Y, li)) return;
      if (!stage_out(P, Y, 0)) return;
    } else {
      if (!stage_sdpa(P, Y, pos)) return;
      if (!stage_out(P, Y, (pos + SDPA_TILE) / SDPA_TILE)) return;
    }
    if (!stage_moe_a(P, Y)) return;
    if (!stage_moe_b(P, Y)) return;
    {
      const bool last = li + 1 == P.n_layers;
      const LayerP& Z = P.layers[last ? li : li + 1];
      if (!stage_moe_c(P, Y, last ? P.lm_w : Z.in_w, last ? P.lm_sb : Z.in_sb,
                       last ? P.vocab : (Z.is_linear ? SL_GDN_IN_N : SL_ATT_QKV_N), last ? 1 : 0)) return;
    }
  }
  stage_head(P, pos, out_off, feed);
}

}  // namespace sl
