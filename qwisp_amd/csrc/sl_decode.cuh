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
  unsigned* bar;   // [0] epoch base, [32] abort flag, [64 + 32g] first-level counters, [1024] second-level counter, [2048 + 32g] release flags
};

// ---- coherent access to activations ----------------------------------------------------------------
#define SL_AG __HIP_MEMORY_SCOPE_AGENT
SL_DEV uint64_t ld_co64(const void* p) { return __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, SL_AG); }
SL_DEV uint32_t ld_co32(const void* p) { return __hip_atomic_load((const uint32_t*)p, __ATOMIC_RELAXED, SL_AG); }
SL_DEV void st_co64(void* p, uint64_t v) { __hip_atomic_store((uint64_t*)p, v, __ATOMIC_RELAXED, SL_AG); }
SL_DEV void st_co32(void* p, uint32_t v) { __hip_atomic_store((uint32_t*)p, v, __ATOMIC_RELAXED, SL_AG); }
SL_DEV void st_co16(uint16_t* p, uint16_t v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, SL_AG); }
SL_DEV float ld_cof(const float* p) { return __uint_as_float(ld_co32(p)); }
SL_DEV void st_cof(float* p, float v) { st_co32(p, __float_as_uint(v)); }
SL_DEV float ld_coh(const uint16_t* p) {       // one half, through its aligned 32-bit word
  const uint32_t w = ld_co32((const void*)((uintptr_t)p & ~(uintptr_t)3));
  return ((uintptr_t)p & 2) ? hi_h(w) : lo_h(w);
}
// 32 halves (64 bytes) owned by one lane
SL_DEV void ld_co_h32(const uint16_t* p, float* x) {
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const uint64_t v = ld_co64(p + 4 * j);
    x[4 * j] = lo_h((uint32_t)v); x[4 * j + 1] = hi_h((uint32_t)v);
    x[4 * j + 2] = lo_h((uint32_t)(v >> 32)); x[4 * j + 3] = hi_h((uint32_t)(v >> 32));
  }
}
SL_DEV void st_co_h32(uint16_t* p, const float* x) {
#pragma unroll
  for (int j = 0; j < 8; ++j)
    st_co64(p + 4 * j, (uint64_t)pack2(x[4 * j], x[4 * j + 1]) | ((uint64_t)pack2(x[4 * j + 2], x[4 * j + 3]) << 32));
}
SL_DEV void ld_co_h4(const uint16_t* p, float* x) {
  const uint64_t v = ld_co64(p);
  x[0] = lo_h((uint32_t)v); x[1] = hi_h((uint32_t)v); x[2] = lo_h((uint32_t)(v >> 32)); x[3] = hi_h((uint32_t)(v >> 32));
}
SL_DEV void st_co_h4(uint16_t* p, const float* x) {
  st_co64(p, (uint64_t)pack2(x[0], x[1]) | ((uint64_t)pack2(x[2], x[3]) << 32));
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
};
SL_DEV void bar_init(GridBar& b, unsigned* mem) {
  b.mem = mem;
  b.ep = ld_co32(mem);
  b.ngroups = gridDim.x / BAR_GROUP;
  b.grp = blockIdx.x / BAR_GROUP;
  b.dead = false;
}
// Call with all of the workgroup's outputs stored; every thread calls it.
SL_DEV void bar_arrive(GridBar& b) {
  __builtin_amdgcn_s_waitcnt(0);          // this wave's stores have been acknowledged
  __syncthreads();
  b.ep++;
  if (threadIdx.x == 0) {
    const unsigned old = __hip_atomic_fetch_add(&b.mem[64 + 32 * b.grp], 1u, __ATOMIC_RELAXED, SL_AG);
    if (old == b.ep * BAR_GROUP - 1) {
      const unsigned o2 = __hip_atomic_fetch_add(&b.mem[1024], 1u, __ATOMIC_RELAXED, SL_AG);
      if (o2 == b.ep * (unsigned)b.ngroups - 1)
        for (int g = 0; g < b.ngroups; ++g) st_co32(&b.mem[2048 + 32 * g], b.ep);
    }
  }
}
// Returns false if the step was aborted.
SL_DEV bool bar_wait(GridBar& b) {
  __shared__ int s_dead;
  if (threadIdx.x == 0) {
    int dead = 0;
    unsigned spins = 0;
    while ((int)(ld_co32(&b.mem[2048 + 32 * b.grp]) - b.ep) < 0) {
      if (++spins > BAR_SPIN_LIMIT || ((spins & 1023u) == 0 && ld_co32(&b.mem[32]) != 0)) {
        st_co32(&b.mem[32], 1u);
        dead = 1;
        break;
      }
    }
    s_dead = dead;
  }
  __syncthreads();
  if (s_dead) b.dead = true;
  return !b.dead;
}

// ---- activation vector in LDS ------------------------------------------------------------------------
// Element i of lane l of block b lives at xs[(32*b + i)*64 + l]; word sums at sxs[(4*b + j)*64 + l].
struct Lds {
  union {                                    // the staged key tile is only live while xs is not
    struct { float xs[4096]; float sxs[512]; };
    uint16_t kt[SDPA_TILE * KT_STRIDE];
  };
  float red[64];
  int ired[64];
  float q[128], k[128], v[32], gb[2];      // GDN head scratch
  int inds[8];
  float scores[8];
  float dbuf[2 * 9 * 4];
  float sq[8 * 256];                        // attention: scaled queries of one kv group
  float knew[256], vnew[256];
  float sm[8 * 64];                         // attention: per head softmax weights of the tile
};
SL_DEV void lds_put_x(Lds& L, int b, int lane, const float* x) {
#pragma unroll
  for (int i = 0; i < 32; ++i) L.xs[(32 * b + i) * 64 + lane] = x[i];
  float sx[4];
  word_sums(x, sx);
#pragma unroll
  for (int j = 0; j < 4; ++j) L.sxs[(4 * b + j) * 64 + lane] = sx[j];
}
SL_DEV void lds_get_x(const Lds& L, int b, int lane, float* x, float* sx) {
#pragma unroll
  for (int i = 0; i < 32; ++i) x[i] = L.xs[(32 * b + i) * 64 + lane];
#pragma unroll
  for (int j = 0; j < 4; ++j) sx[j] = L.sxs[(4 * b + j) * 64 + lane];
}

// Hidden prologue by wave 0: x = half(h + r), optional rmsnorm; one workgroup stores h_out/xn_out.
SL_DEV void dec_hidden(Lds& L, const uint16_t* h_in, const uint16_t* r_in, const uint16_t* lnw, uint16_t* h_out,
                       uint16_t* xn_out, bool writer, int lane, const float* preset) {
  float x[32];
  if (preset) {
#pragma unroll
    for (int i = 0; i < 32; ++i) x[i] = preset[i];
  } else {
    ld_co_h32(h_in + 32 * lane, x);
  }
  if (r_in) {
    float r[32];
    ld_co_h32(r_in + 32 * lane, r);
#pragma unroll
    for (int i = 0; i < 32; ++i) x[i] = f16r(x[i] + r[i]);
  }
  if (writer && h_out) st_co_h32(h_out + 32 * lane, x);
  if (lnw) {
    const float inv = inv_rms_2048(x);
    float w[32];
    load32(lnw + 32 * lane, w);
#pragma unroll
    for (int i = 0; i < 32; ++i) x[i] = f16r(w[i] * f16r(x[i] * inv));
  }
  if (writer && xn_out) st_co_h32(xn_out + 32 * lane, x);
  lds_put_x(L, 0, lane, x);
}

// ---- weight prefetch: up to R rows of K = 2048*NBLK held in registers --------------------------------
template <int NBLK, int R>
struct WRegs {
  uint4 w[R][NBLK];
  uint32_t sb[R][NBLK];
};
template <int NBLK, int R>
SL_DEV void wload(WRegs<NBLK, R>& r, const uint32_t* __restrict__ W, const uint32_t* __restrict__ SB, const size_t* rows,
                  const bool* valid, int lane) {
#pragma unroll
  for (int i = 0; i < R; ++i)
#pragma unroll
    for (int b = 0; b < NBLK; ++b) {
      if (valid[i]) {
        r.w[i][b] = ld16(W + rows[i] * (NBLK * 256) + b * 256 + 4 * lane);
        r.sb[i][b] = SB[rows[i] * (NBLK * 32) + b * 32 + (lane >> 1)];
      } else {
        r.w[i][b] = make_uint4(0, 0, 0, 0);
        r.sb[i][b] = 0;
      }
    }
}
template <int NBLK, int R>
SL_DEV void wdot(const WRegs<NBLK, R>& r, const Lds& L, int lane, float* out) {
  float x[32], sx[4];
  float acc[R];
#pragma unroll
  for (int b = 0; b < NBLK; ++b) {
    lds_get_x(L, b, lane, x, sx);
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const float t = quad_term(r.w[i][b], r.sb[i][b], x, sx);
      acc[i] = (b == 0) ? t : (acc[i] + t);
    }
  }
#pragma unroll
  for (int i = 0; i < R; ++i) out[i] = tree_sum<64>(acc[i]);
}

// Rows of a projection are dealt to waves 16 at a time per workgroup: wave gw owns rows gw + j*NW.
template <int R>
SL_DEV void deal_rows(int gw, int NW, int N, size_t* rows, bool* valid) {
#pragma unroll
  for (int j = 0; j < R; ++j) {
    const int r = gw + j * NW;
    valid[j] = r < N;
    rows[j] = valid[j] ? (size_t)r : 0;
  }
}

// ---- the kernel ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(DEC_THREADS) void k_decode(const DecodeP* __restrict__ Pp, int out_off, int feed) {
  __shared__ Lds L;
  const DecodeP& P = *Pp;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wg = blockIdx.x, G = gridDim.x, NW = G * DEC_WAVES, gw = wg * DEC_WAVES + wave;
  GridBar bar;
  bar_init(bar, P.bar);
  const int pos = P.st[0];
  const int tok = P.tok_in[0];
  const float NEG = -__int_as_float(0x7f800000);

  for (int li = 0; li < P.n_layers; ++li) {
    const LayerP& Y = P.layers[li];
    // ================= stage 1: input norm + in-projection =================
    {
      const int N = Y.is_linear ? SL_GDN_IN_N : SL_ATT_QKV_N;
      size_t rows[4]; bool valid[4];
      deal_rows<4>(gw, NW, N, rows, valid);
      WRegs<1, 4> wr;
      wload<1, 4>(wr, Y.in_w, Y.in_sb, rows, valid, lane);
      if (li > 0 && !bar_wait(bar)) return;
      if (wave == 0) {
        if (li == 0) {
          float e[32];
#pragma unroll
          for (int i = 0; i < 32; ++i) {
            const int j = 32 * lane + i;
            const uint32_t w = P.emb_w[(size_t)tok * 256 + (j >> 3)];
            const uint32_t sb = P.emb_sb[(size_t)tok * 32 + (j >> 6)];
            e[i] = f16r(f16r(lo_h(sb) * (float)((w >> (4 * (j & 7))) & 15u)) + hi_h(sb));
          }
          dec_hidden(L, nullptr, nullptr, Y.input_ln, P.hB, nullptr, wg == 0, lane, e);
        } else {
          dec_hidden(L, P.hA, P.moe_out, Y.input_ln, P.hB, nullptr, wg == 0, lane, nullptr);
        }
      }
      __syncthreads();
      float out[4];
      wdot<1, 4>(wr, L, lane, out);
      if (lane == 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j) if (valid[j]) st_co16(P.proj + rows[j], f2h(out[j]));
      }
      bar_arrive(bar);
    }
    if (Y.is_linear) {
      // ================= stage 2: conv + prep + gated delta rule =================
      const int par = P.st[1 + li];
      const uint16_t* hin = Y.hist[par];
      uint16_t* hout = Y.hist[par ^ 1];
      for (int u = wg; u < 256; u += G) {
        const int hv = u >> 3, dvb = u & 7, hk = hv >> 1;
        const int half = lane >> 5, l32 = lane & 31;
        float s[4];
        if (wave < 8) {
          const int dv = dvb * 16 + wave * 2 + half;
          const float4 v4 = *reinterpret_cast<const float4*>(Y.state[par] + ((size_t)hv * 128 + dv) * 128 + 4 * l32);
          s[0] = v4.x; s[1] = v4.y; s[2] = v4.z; s[3] = v4.w;
        }
        if (u == wg && !bar_wait(bar)) return;
        // conv over [hist(3) | qkv]: threads 0..255 q/k channels of head hk, 256..271 the unit's v channels
        int ch = -1;
        if (tid < 128) ch = hk * 128 + tid;
        else if (tid < 256) ch = 2048 + hk * 128 + (tid - 128);
        else if (tid < 272) ch = 4096 + hv * 128 + dvb * 16 + (tid - 256);
        float newest = 0.0f;
        if (ch >= 0) {
          newest = ld_coh(P.proj + ch);
          float acc = 0.0f;
#pragma unroll
          for (int k = 0; k < 3; ++k) acc = fmaf(h2f(hin[k * SL_CONV_DIM + ch]), Y.conv_w[ch * 4 + k], acc);
          acc = fmaf(newest, Y.conv_w[ch * 4 + 3], acc);
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
          const float bP = ld_coh(P.proj + 12288 + hv), aP = ld_coh(P.proj + 12320 + hv);
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
          if (l32 == 0) st_co16(P.ycore + hv * 128 + dv, f2h(y));
          *reinterpret_cast<float4*>(Y.state[par ^ 1] + ((size_t)hv * 128 + dv) * 128 + 4 * l32) = make_float4(s[0], s[1], s[2], s[3]);
        }
        // history shift: rows 1,2 of the old history and the new sample
        if (ch >= 0 && (tid >= 256 || ((hv & 1) == 0 && dvb == 0))) {
          hout[ch] = hin[SL_CONV_DIM + ch];
          hout[SL_CONV_DIM + ch] = hin[2 * SL_CONV_DIM + ch];
          hout[2 * SL_CONV_DIM + ch] = f2h(newest);
        }
        __syncthreads();
      }
      if (wg >= 256 && !bar_wait(bar)) return;      // workgroups without a unit still pass the barrier
      bar_arrive(bar);
      // ================= stage 3: gated rmsnorm + out-projection (K = 4096) =================
      {
        size_t rows[1]; bool valid[1];
        deal_rows<1>(gw, NW, H, rows, valid);
        WRegs<2, 1> wr;
        wload<2, 1>(wr, Y.out_w, Y.out_sb, rows, valid, lane);
        if (!bar_wait(bar)) return;
        if (wave < 2) {
          const int b = wave;
          float xb[32], nw[32], z[32];
          ld_co_h32(P.ycore + b * 2048 + 32 * lane, xb);
          load32(Y.gdn_norm_w + 32 * (lane & 3), nw);
          float leaf[16];
#pragma unroll
          for (int j = 0; j < 16; ++j) leaf[j] = fmaf(xb[2 * j + 1], xb[2 * j + 1], fmaf(xb[2 * j], xb[2 * j], 0.0f));
#pragma unroll
          for (int st = 1; st < 16; st <<= 1)
#pragma unroll
            for (int j = 0; j < 16; j += 2 * st) leaf[j] = leaf[j] + leaf[j + st];
          const float ss = tree_sum<4>(leaf[0]);
          const float inv = 1.0f / sqrtf(ss / 128.0f + EPS);
          ld_co_h32(P.proj + 8192 + b * 2048 + 32 * lane, z);
#pragma unroll
          for (int i = 0; i < 32; ++i) {
            const float nrm = f16r(nw[i] * f16r(xb[i] * inv));
            xb[i] = f16r((z[i] * sigmoid32(z[i])) * nrm);
          }
          lds_put_x(L, b, lane, xb);
        }
        __syncthreads();
        float out[1];
        wdot<2, 1>(wr, L, lane, out);
        if (lane == 0 && valid[0]) st_co16(P.mix + rows[0], f2h(out[0]));
        bar_arrive(bar);
      }
    } else {
      // ================= attention stage 2: q/k prep, KV append, tile pass =================
      const int N = pos + 1, nt = (N + SDPA_TILE - 1) / SDPA_TILE;
      if (!bar_wait(bar)) return;
      for (int u = wg; u < nt * SL_ATT_KV; u += G) {
        const int tile = u >> 1, kvh = u & 1;
        const int j0 = tile * SDPA_TILE, nk = min(SDPA_TILE, N - j0);
        const bool has_new = (pos >= j0) && (pos < j0 + SDPA_TILE);
        // waves 0..7: query heads of the group; wave 8: the new key; wave 9: the new value
        if (wave < 9) {
          const bool isq = wave < 8;
          const uint16_t* src = P.proj + (isq ? (kvh * 8 + wave) * 512 : 8192 + kvh * 256);
          const uint16_t* nwp = isq ? Y.q_norm : Y.k_norm;
          float xv[4], wv[4];
          ld_co_h4(src + 4 * lane, xv);
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
          // partial rotary on the first 64 dims: lanes 0..15 hold dims 0..63, pairs (i, i+32) sit 8 lanes apart
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
          // all lanes of the wave have read dst before any lane overwrites it (same wave, lockstep)
#pragma unroll
          for (int i = 0; i < 4; ++i) dst[4 * lane + i] = isq ? 0.0625f * o[i] : o[i];
          if (!isq && has_new) st_co_h4(Y.kcache + ((size_t)kvh * P.max_seq + pos) * 256 + 4 * lane, o);
        } else if (wave == 9) {
          float vv[4];
          ld_co_h4(P.proj + 8192 + 512 + kvh * 256 + 4 * lane, vv);
#pragma unroll
          for (int i = 0; i < 4; ++i) L.vnew[4 * lane + i] = vv[i];
          if (has_new) st_co_h4(Y.vcache + ((size_t)kvh * P.max_seq + pos) * 256 + 4 * lane, vv);
        }
        // stage the tile's keys: 1024 threads x 16 bytes = 32 rows per pass
        const uint16_t* kbase = Y.kcache + ((size_t)kvh * P.max_seq + j0) * 256;
        for (int it = 0; it < 2; ++it) {
          const int row = it * 32 + (tid >> 5), c8 = (tid & 31) * 8;
          if (row < nk && j0 + row != pos) st16(&L.kt[row * KT_STRIDE + c8], ld16(kbase + (size_t)row * 256 + c8));
        }
        __syncthreads();
        if (has_new && tid < 64) {
          const int row = pos - j0;
          const uint2 pk = make_uint2(pack2(L.knew[4 * tid], L.knew[4 * tid + 1]), pack2(L.knew[4 * tid + 2], L.knew[4 * tid + 3]));
          *reinterpret_cast<uint2*>(&L.kt[row * KT_STRIDE + 4 * tid]) = pk;
        }
        __syncthreads();
        if (wave < 8) {
          // lane j scores key j for head `wave`: balanced tree over 64 leaves of 4 dims
          float stk[7];
          const uint16_t* kr = &L.kt[(lane < nk ? lane : 0) * KT_STRIDE];
          const float* qh = &L.sq[wave * 256];
#pragma unroll
          for (int leaf = 0; leaf < 64; ++leaf) {
            const uint2 kraw = *reinterpret_cast<const uint2*>(kr + 4 * leaf);
            float node = fmaf(qh[4 * leaf], lo_h(kraw.x), 0.0f);
            node = fmaf(qh[4 * leaf + 1], hi_h(kraw.x), node);
            node = fmaf(qh[4 * leaf + 2], lo_h(kraw.y), node);
            node = fmaf(qh[4 * leaf + 3], hi_h(kraw.y), node);
            int c = leaf, lvl = 0;
            while (c & 1) { node = stk[lvl] + node; c >>= 1; ++lvl; }
            stk[lvl] = node;
          }
          const float sc = (lane < nk) ? stk[6] : NEG;
          const float mx = tree_max<64>(sc);
          const float p = (lane < nk) ? exp_c(sc - mx) : 0.0f;
          const float l = tree_sum<64>(p);
          L.sm[wave * 64 + lane] = p;
          const int head = kvh * 8 + wave;
          if (lane == 0) { st_cof(P.pm + (size_t)head * P.max_tiles + tile, mx); st_cof(P.pl + (size_t)head * P.max_tiles + tile, l); }
          // o = fmaf chain over the tile's keys; V rows read coalesced, the new row from LDS
          float o[4] = {0.0f, 0.0f, 0.0f, 0.0f};
          const uint16_t* vbase = Y.vcache + ((size_t)kvh * P.max_seq + j0) * 256;
          for (int j = 0; j < nk; ++j) {
            float vf[4];
            if (j0 + j == pos) {
#pragma unroll
              for (int i = 0; i < 4; ++i) vf[i] = L.vnew[4 * lane + i];
            } else {
              const uint2 vraw = *reinterpret_cast<const uint2*>(vbase + (size_t)j * 256 + 4 * lane);
              vf[0] = lo_h(vraw.x); vf[1] = hi_h(vraw.x); vf[2] = lo_h(vraw.y); vf[3] = hi_h(vraw.y);
            }
            const float pj = L.sm[wave * 64 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i] = fmaf(pj, vf[i], o[i]);
          }
          float* po = P.po + ((size_t)head * P.max_tiles + tile) * 256 + 4 * lane;
#pragma unroll
          for (int i = 0; i < 4; ++i) st_cof(po + i, o[i]);
        }
        __syncthreads();
      }
      bar_arrive(bar);
      // ================= attention stage 3: merge tiles + output gate (workgroup 0) =================
      {
        size_t rows[1]; bool valid[1];
        deal_rows<1>(gw, NW, H, rows, valid);
        WRegs<2, 1> wr;
        wload<2, 1>(wr, Y.out_w, Y.out_sb, rows, valid, lane);      // o_proj weights for stage 4
        if (!bar_wait(bar)) return;
        if (wg == 0) {
          const int h = wave;
          const size_t base = (size_t)h * P.max_tiles;
          float Mx = NEG;
          for (int t = 0; t < nt; ++t) Mx = fmaxf(Mx, ld_cof(P.pm + base + t));
          float Ls = 0.0f, O[4] = {0.0f, 0.0f, 0.0f, 0.0f};
          for (int t = 0; t < nt; ++t) {
            const float f = exp_c(ld_cof(P.pm + base + t) - Mx);
            Ls = fmaf(ld_cof(P.pl + base + t), f, Ls);
            const float* po = P.po + (base + t) * 256 + 4 * lane;
#pragma unroll
            for (int i = 0; i < 4; ++i) O[i] = fmaf(ld_cof(po + i), f, O[i]);
          }
          float gt[4], r[4];
          ld_co_h4(P.proj + h * 512 + 256 + 4 * lane, gt);
#pragma unroll
          for (int i = 0; i < 4; ++i) r[i] = f16r(f16r(O[i] / Ls) * sigmoid16(gt[i]));
          st_co_h4(P.ycore + h * 256 + 4 * lane, r);
        }
        bar_arrive(bar);
        // ================= attention stage 4: o-projection (K = 4096) =================
        if (!bar_wait(bar)) return;
        if (wave < 2) {
          float xb[32];
          ld_co_h32(P.ycore + wave * 2048 + 32 * lane, xb);
          lds_put_x(L, wave, lane, xb);
        }
        __syncthreads();
        float out[1];
        wdot<2, 1>(wr, L, lane, out);
        if (lane == 0 && valid[0]) st_co16(P.mix + rows[0], f2h(out[0]));
        bar_arrive(bar);
      }
    }
    // ================= MoE stage A: post norm, shared gate/up + SwiGLU, router and shared-gate rows =================
    {
      const bool is_dense = gw <= P.E;                       // rows 0..E-1 router, row E shared gate
      const bool is_pair = gw >= 512 && gw < 1024;           // shared-expert pair gw-512
      float dw[32];
      WRegs<1, 2> wg_, wu_;
      size_t prow[2] = {0, 0}; bool pvalid[2] = {is_pair, is_pair};
      if (is_pair) { prow[0] = (size_t)(gw - 512); prow[1] = prow[0]; }
      {
        // one gate row and one up row per wave
        size_t r1[2] = {prow[0], 0}; bool v1[2] = {is_pair, false};
        wload<1, 2>(wg_, Y.shg_w, Y.shg_sb, r1, v1, lane);
        wload<1, 2>(wu_, Y.shu_w, Y.shu_sb, r1, v1, lane);
      }
      if (is_dense) load32((gw < P.E ? Y.router_w + (size_t)gw * H : Y.sgate_w) + 32 * lane, dw);
      if (!bar_wait(bar)) return;
      if (wave == 0) dec_hidden(L, P.hB, P.mix, Y.post_ln, P.hA, nullptr, wg == 0, lane, nullptr);
      __syncthreads();
      if (is_dense) {
        float x[32], sx[4];
        lds_get_x(L, 0, lane, x, sx);
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < 32; ++i) acc = fmaf(x[i], dw[i], acc);
        acc = tree_sum<64>(acc);
        if (lane == 0) { if (gw < P.E) st_co16(P.rlogits + gw, f2h(acc)); else st_co16(P.sgate, f2h(acc)); }
      }
      if (is_pair) {
        float g[2], u[2];
        wdot<1, 2>(wg_, L, lane, g);
        wdot<1, 2>(wu_, L, lane, u);
        if (lane == 0) st_co16(P.sh_act + prow[0], f2h(swiglu16(f16r(g[0]), f16r(u[0]))));
      }
      (void)pvalid;
      bar_arrive(bar);
    }
    // ================= MoE stage B: routing + routed gate/up + SwiGLU (xs still holds the post-normed row) =================
    {
      if (!bar_wait(bar)) return;
      if (wave == 0) {
        // logits through coherent loads into LDS, then the one-wave router
        uint16_t* lg = reinterpret_cast<uint16_t*>(L.red);      // 256 halves = 128 floats: red + ired
        const uint64_t v = ld_co64(P.rlogits + 4 * lane);
        *reinterpret_cast<uint64_t*>(lg + 4 * lane) = v;
        int inds[8]; float sc[8];
        route_wave(lg, P.E, lane, inds, sc);
        if (lane == 0) {
#pragma unroll
          for (int k = 0; k < 8; ++k) {
            L.inds[k] = inds[k]; L.scores[k] = sc[k];
            if (wg == 0) { Y.route_inds[k] = inds[k]; Y.route_scores[k] = f2h(sc[k]); }
          }
        }
      }
      __syncthreads();
      for (int p = gw; p < 8 * 512; p += NW) {
        const int k = p >> 9, i = p & 511;
        const size_t row = (size_t)L.inds[k] * 512 + i;
        size_t r1[2] = {row, 0}; bool v1[2] = {true, false};
        WRegs<1, 2> a, b;
        wload<1, 2>(a, Y.swg_w, Y.swg_sb, r1, v1, lane);
        wload<1, 2>(b, Y.swu_w, Y.swu_sb, r1, v1, lane);
        float g[2], u[2];
        wdot<1, 2>(a, L, lane, g);
        wdot<1, 2>(b, L, lane, u);
        if (lane == 0) st_co16(P.act + k * 512 + i, f2h(swiglu16(f16r(g[0]), f16r(u[0]))));
      }
      bar_arrive(bar);
    }
    // ================= MoE stage C: down-projections, half combine, gated shared add =================
    {
      const int sub = lane >> 4, li16 = lane & 15;
      const size_t shrow_base = 0;
      (void)shrow_base;
      // units (quad, slot): slot 0..7 routed expert k, slot 8 shared; 9 units per quad of 4 outputs
      const int nquads = H / 4;
      const int qpw = (nquads + G - 1) / G;                 // quads per workgroup (2 when G = 256)
      uint4 shw[2]; uint32_t shsb[2];
      // shared-expert rows do not depend on routing: prefetch them before the wait
#pragma unroll
      for (int qq = 0; qq < 2; ++qq) {
        const int un = wave + 16 * qq;                      // unit index within the workgroup
        const int ql = un / 9, slot = un % 9;
        const int quad = wg * qpw + ql;
        shw[qq] = make_uint4(0, 0, 0, 0); shsb[qq] = 0;
        if (ql < qpw && quad < nquads && slot == 8) {
          const size_t row = (size_t)quad * 4 + sub;
          shw[qq] = ld16(Y.shd_w + row * 64 + 4 * li16);
          shsb[qq] = Y.shd_sb[row * 8 + (li16 >> 1)];
        }
      }
      if (!bar_wait(bar)) return;
#pragma unroll
      for (int qq = 0; qq < 2; ++qq) {
        const int un = wave + 16 * qq;
        const int ql = un / 9, slot = un % 9;
        const int quad = wg * qpw + ql;
        if (ql < qpw && quad < nquads && ql < 2) {
          float x[32], sx[4];
          ld_co_h32((slot < 8 ? P.act + slot * 512 : P.sh_act) + 32 * li16, x);
          word_sums(x, sx);
          float d;
          if (slot < 8) {
            const size_t row = (size_t)L.inds[slot] * 2048 + (size_t)quad * 4 + sub;
            d = qdot512(Y.swd_w, Y.swd_sb, row, li16, x, sx);
          } else {
            d = tree_sum<16>(quad_term(shw[qq], shsb[qq], x, sx));
          }
          if (li16 == 0) L.dbuf[(ql * 9 + slot) * 4 + sub] = f16r(d);
        }
      }
      __syncthreads();
      if (tid < 8) {
        const int ql = tid >> 2, sb4 = tid & 3;
        const int quad = wg * qpw + ql;
        if (ql < qpw && quad < nquads) {
          float acc = 0.0f;
#pragma unroll
          for (int k = 0; k < 8; ++k) acc = f16r(acc + f16r(L.dbuf[(ql * 9 + k) * 4 + sb4] * L.scores[k]));
          const float s = sigmoid16(ld_coh(P.sgate));
          st_co16(P.moe_out + quad * 4 + sb4, f2h(f16r(acc + f16r(s * L.dbuf[(ql * 9 + 8) * 4 + sb4]))));
        }
      }
      bar_arrive(bar);
    }
  }
  // ================= head: final norm + lm_head + argmax =================
  {
    // each wave owns a contiguous chunk of 64 vocabulary rows, 4 at a time, one group prefetched ahead
    const int nchunks = (P.vocab + 63) / 64;
    float bv = NEG; int bi = 0x7fffffff;
    WRegs<1, 4> cur, nxt;
    size_t rows[4]; bool valid[4];
    const int c0 = gw;
    auto group_rows = [&](int chunk, int g4) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const long r = (long)chunk * 64 + g4 * 4 + j;
        valid[j] = chunk < nchunks && r < P.vocab;
        rows[j] = valid[j] ? (size_t)r : 0;
      }
    };
    group_rows(c0, 0);
    wload<1, 4>(cur, P.lm_w, P.lm_sb, rows, valid, lane);
    if (!bar_wait(bar)) return;
    if (wave == 0) dec_hidden(L, P.hA, P.moe_out, P.final_norm, P.hB, P.normed, wg == 0, lane, nullptr);
    __syncthreads();
    for (int chunk = c0; chunk < nchunks; chunk += NW) {
      for (int g4 = 0; g4 < 16; ++g4) {
        // prefetch the next group (possibly of the next chunk)
        int nchunk = chunk, ng = g4 + 1;
        if (ng == 16) { ng = 0; nchunk = chunk + NW; }
        group_rows(nchunk, ng);
        wload<1, 4>(nxt, P.lm_w, P.lm_sb, rows, valid, lane);
        float out[4];
        wdot<1, 4>(cur, L, lane, out);
        const long r0 = (long)chunk * 64 + g4 * 4;
        if (r0 < P.vocab) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float v = f16r(out[j]);
            if (v > bv) { bv = v; bi = (int)(r0 + j); }
          }
          if (lane == 0) *reinterpret_cast<uint2*>(P.logits + r0) = make_uint2(pack2(out[0], out[1]), pack2(out[2], out[3]));
        }
        cur = nxt;
      }
    }
    if (lane == 0) { L.red[wave] = bv; L.ired[wave] = bi; }
    __syncthreads();
    if (tid == 0) {
      for (int w = 1; w < DEC_WAVES; ++w)
        if (L.red[w] > bv || (L.red[w] == bv && L.ired[w] < bi)) { bv = L.red[w]; bi = L.ired[w]; }
      st_cof(P.cand_v + wg, bv);
      st_co32(P.cand_i + wg, (uint32_t)bi);
    }
    bar_arrive(bar);
    if (!bar_wait(bar)) return;
    if (wg == 0) {
      float v = NEG; int i = 0x7fffffff;
      if (tid < G) { v = ld_cof(P.cand_v + tid); i = (int)ld_co32(P.cand_i + tid); }
      // first maximum over up to 1024 candidates: wave butterflies, then wave 0 over the 16 wave results
#pragma unroll
      for (int msk = 1; msk < 64; msk <<= 1) {
        const float ov = __shfl_xor(v, msk, 64); const int oi = __shfl_xor(i, msk, 64);
        if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
      }
      if (lane == 0) { L.red[wave] = v; L.ired[wave] = i; }
      __syncthreads();
      if (tid == 0) {
        for (int w = 1; w < DEC_WAVES; ++w)
          if (L.red[w] > v || (L.red[w] == v && L.ired[w] < i)) { v = L.red[w]; i = L.ired[w]; }
        P.tok_out[out_off] = i;
        if (feed) P.tok_in[0] = i;
        P.st[0] = pos + 1;
        st_co32(P.bar, bar.ep);
      }
      for (int l = tid; l < P.n_layers; l += DEC_THREADS) P.st[1 + l] ^= 1;
    }
  }
}

}  // namespace sl
