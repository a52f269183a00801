// Shared pieces of the persistent single-token decode kernel for gfx950 (sl_flow.cuh): parameter blocks,
// coherent (sc1) buffer access, the workgroup's LDS layout, weight rows held in registers and the three dot
// shapes of a step.
//
// One launch runs a whole batch-1 step (all layers -> final norm -> lm_head -> argmax) on a grid of one
// 1024-thread workgroup per compute unit.  Values that cross workgroups go through raw buffer instructions
// with the sc1 cache policy, which are coherent across the 8 XCDs without cache maintenance.  Weights, KV rows
// of earlier tokens and the recurrent state are only read after a launch boundary and use plain loads.
//
// The arithmetic is that of sl_kernels.cuh (same helpers, same reduction order), so a step here equals a step
// of the multi-kernel path bit for bit.
#pragma once
#include "sl_kernels.cuh"

namespace sl {

constexpr int DEC_THREADS = 1024;
constexpr int DEC_WAVES = DEC_THREADS / 64;

struct LayerP {
  int is_linear;
  const uint16_t *input_ln, *post_ln;
  const uint32_t *in_w, *in_sb;          // GDN in_proj [12352,2048] or attention q|k|v [9216,2048]
  const uint32_t *out_w, *out_sb;        // GDN out_proj or attention o_proj [2048,4096]
  const float *conv_w, *a_log, *dt_bias;
  const float* gdn_norm_w;               // [128] fp32 (an fp16 checkpoint weight converted exactly)
  int gdn_norm_f32;                      // the checkpoint weight was fp32: gated norm without the half roundings
  uint16_t* hist[2];
  float* state[2];
  const uint16_t *q_norm, *k_norm;
  uint16_t *kcache, *vcache;
  const uint16_t *router_w, *sgate_w;    // with 8-bit gates: words [E+1, 512] (row E = shared gate) and {scale, bias} [E+1, 32]
  const uint32_t *swg_w, *swg_sb, *swu_w, *swu_sb, *swd_w, *swd_sb;
  const uint32_t *shg_w, *shg_sb, *shu_w, *shu_sb, *shd_w, *shd_sb;
  int32_t* route_inds;
  uint16_t* route_scores;
};

struct DecodeP {
  int n_layers, E, vocab, max_seq, max_tiles;
  const LayerP* layers;
  const uint32_t *lm_w, *lm_sb;
  const uint32_t *emb_w, *emb_sb;     // token embedding [vocab, 2048] 4-bit
  const uint16_t* final_norm;
  const float *rope_cos, *rope_sin;
  uint16_t *hA, *normed, *logits;     // (hA: unused by the step kernel) final-normed row and logits out
  int32_t *tok_in, *tok_out, *st;     // st: {position, parity of every layer's ping-pong caches}
  uint32_t* tstamp;             // diagnostic clock stamps of the stamping kernel variant: [workgroups][STAMP_WORDS]
  unsigned* bar;   // [16] stage-instance counter (advanced every launch), [32] abort flag
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

// ---- activation vector in LDS ------------------------------------------------------------------------
// Packed pair i (elements 2i, 2i+1) of lane l of block b lives at xs[(16*b + i)*64 + l]; the sum of the lane's share
// of 32 elements at sxs[64*b + l].
struct Lds {
  union {                                    // the staged key tile is only live while xs is not
    struct { uint32_t xs[2048]; float sxs[128]; };
    uint16_t kt[SDPA_TILE * KT_STRIDE];
  };
  float red[64];
  int ired[64];
  float q[128], k[128], v[32], gb[2];      // GDN head scratch
  int inds[8];
  float scores[8];
  float dbuf[2 * 9 * 4];
  int pf[4];                                // poll outcome slots (three in rotation) and the give-up flag
  uint32_t pub[64];                         // a stage's tagged outputs, gathered for the publishing wave
  alignas(16) float sq[8 * 256];            // attention: scaled queries of one kv group (read back 16 bytes at a time)
  float knew[256], vnew[256];
  alignas(16) float sm[8 * 64];             // attention: per head softmax weights of the tile (read back 16 bytes at a time)
  alignas(16) float part[16 * 64];          // router: logits and exps; attention merge: hand-over words
};
__shared__ Lds g_L;
extern __shared__ __align__(16) uint16_t g_vt[];   // dynamic: staged value tile [64][256] halves, then the softmax
                                                   // weights of up to SDPA_ROUND (tile, kv head) units [8 heads][64 keys]
constexpr int SDPA_ROUND = 12;
// Attention tile units use the dynamic LDS as: value tile 32 KB | softmax weights of a round's units | score partials
// [8 heads][8 chains of 32 dims][64 keys] fp32 (also the value sums of the keys' second half on their way to the first).
constexpr int SPART_OFF = SDPA_TILE * 256 * 2 + SDPA_ROUND * 8 * 64 * 4;            // bytes into g_vt
constexpr int DEC_DYN_LDS = 77824;               // what the rows parked ahead of their stage need (the larger of the two uses)
static_assert(SPART_OFF + 64 * 64 * 4 <= DEC_DYN_LDS, "score partials fit");

SL_DEV void lds_get_x(int b, int lane, uint32_t* xp, float& sx) {
#pragma unroll
  for (int i = 0; i < 16; ++i) xp[i] = g_L.xs[(16 * b + i) * 64 + lane];
  sx = g_L.sxs[64 * b + lane];
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
// Dot shapes of a step (arguments travel in registers): 2 rows x 2048, 1 row x 4096.
SL_DEV F2 dot_1x2_(uint4 w0, uint4 w1, uint32_t s0, uint32_t s1) {
  const int lane = threadIdx.x & 63;
  uint32_t x[16]; float sx;
  lds_get_x(0, lane, x, sx);
  F2 o;
  o.v[0] = tree_sum<64>(share_term(w0, s0, x, sx));
  o.v[1] = tree_sum<64>(share_term(w1, s1, x, sx));
  return o;
}
SL_DEV float dot_2x1_(uint4 w0, uint4 w1, uint32_t s0, uint32_t s1) {
  const int lane = threadIdx.x & 63;
  uint32_t x[16]; float sx;
  lds_get_x(0, lane, x, sx);
  float acc = share_term(w0, s0, x, sx);
  lds_get_x(1, lane, x, sx);
  acc = acc + share_term(w1, s1, x, sx);
  return tree_sum<64>(acc);
}
SL_DEV F2 dot_1x2(const WRegs<1, 2>& r) { return dot_1x2_(r.w[0][0], r.w[1][0], r.sb[0][0], r.sb[1][0]); }
SL_DEV float dot_2x1(const WRegs<2, 1>& r) { return dot_2x1_(r.w[0][0], r.w[0][1], r.sb[0][0], r.sb[0][1]); }

}  // namespace sl
