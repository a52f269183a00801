// TEST INFRASTRUCTURE — CPU oracle for the Seedless decode path.  Nothing outside tests/,
// __graft_entry__.smoke() and bench.py's cpu_baseline leg may use this directory.
//
// A CPU restatement of the reference's decode forward (embed -> 40 x [mixer, MoE] -> final norm
// -> lm_head -> argmax).  Op order and every fp16 rounding point follow the reference's composed
// forward and kernels, cited per function below (paths relative to swift/Sources/QwispCore/).
// What the reference leaves to Metal/MLX — the order of fp32 reductions and the last bit of
// exp/log/sin/cos — is fixed here ("canonical order"); the HIP kernels implement the same order,
// so indices, tokens, hidden states and caches compare bit-for-bit.
//
// Canonical reductions: a reduction over n values is a balanced binary tree over 64 (or fewer)
// "lane" partials, adjacent lanes paired first; what a lane partial is (fmaf chains over the
// elements the lane owns, or a sub-tree) is stated per function below.
//
// PARITY PINNING: the reference ships no golden vectors for this path (its tests derive inputs
// from MLXRandom at run time) and none of its code can be built here (Swift + MLX + Metal), so
// this oracle is pinned by closed forms, brute force and library cross-checks in
// tests/test_oracle_pins.py; against MLX's own CPU kernels it is "parity unpinned".
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../include/seedless_hip.h"
#include "orc_math.h"

namespace orc {

constexpr int H = SL_H, I = SL_MOE_I, TOPK = SL_TOPK;
constexpr int NH = SL_ATT_HEADS, NKV = SL_ATT_KV, HD = SL_ATT_D, ROPE = SL_ROPE_DIM;
constexpr int HK = SL_GDN_HK, HV = SL_GDN_HV, GD = SL_GDN_D, CK = SL_CONV_K, CD = SL_CONV_DIM;
constexpr int KEYDIM = HK * GD, VALDIM = HV * GD;
constexpr float EPS = 1e-6f;
constexpr int SDPA_TILE = 64;
constexpr int MERGE_BLOCK = 64;     // key tiles whose partial sums form one chain in the merge

// ------------------------------------------------------------------------------------------------
// 4-bit GEMV.  Reference: qmm4 (SeedlessMetalForward.swift:238-310): y[n] = sum_k x[k]*(s*q+b),
// evaluated as s*sum(x*q) + b*sum(x) per run of weights that share one (s, b), fp32 accumulate,
// fp16 result.
// Canonical order: a "share" is 32 consecutive elements (4 packed words, half a quantisation
// group, so one scale and one bias).  Its term is T = fmaf(s, dq, b*sx) with
//   dq = A + B, A = fmaf chain over the share's even-indexed elements in order, B = the same over
//        the odd-indexed ones (two chains: on the device the even and odd nibbles of a word are
//        isolated by different masks and meet only here),
//   sx = balanced binary tree over the 16 pair sums x[2i] + x[2i+1], adjacent pairs first.
// Lane l of L = min(64, K/32) owns share l of every block of L shares and adds its terms block
// after block; the lanes are tree-summed.
// ------------------------------------------------------------------------------------------------
struct XPrep {
  int K = 0, S = 0;
  std::vector<float> xe, xo;   // even / odd elements, xe[i*S + sh] = x[32 sh + 2i], xo[...] = x[32 sh + 2i + 1]
  std::vector<float> sx;       // per share
  void set(const float* x, int k) {
    K = k; S = k / 32;
    xe.resize((size_t)16 * S); xo.resize((size_t)16 * S); sx.resize(S);
    for (int sh = 0; sh < S; ++sh) {
      float ps[16];
      for (int i = 0; i < 16; ++i) {
        const float a = x[32 * sh + 2 * i], b = x[32 * sh + 2 * i + 1];
        xe[(size_t)i * S + sh] = a; xo[(size_t)i * S + sh] = b; ps[i] = a + b;
      }
      sx[sh] = tree_sum(ps, 16);
    }
  }
};

static float qdot(const XPrep& xp, const uint32_t* wrow, const uint16_t* srow, const uint16_t* brow) {
  const int S = xp.S;
  float t[128];
  for (int s0 = 0; s0 < S; s0 += 8) {          // eight shares at a time (the loops over j vectorise)
    const int nb = std::min(8, S - s0);
    float A[8], B[8];
    uint32_t wt[4][8];                         // word wd of share j
    for (int j = 0; j < 8; ++j) {
      A[j] = 0.0f; B[j] = 0.0f;
      for (int wd = 0; wd < 4; ++wd) wt[wd][j] = j < nb ? wrow[4 * (s0 + j) + wd] : 0u;
    }
    if (nb == 8) {
      for (int i = 0; i < 16; ++i) {           // pair i of a share: nibbles 2(i%4), 2(i%4)+1 of its word i/4
        const float* xe = &xp.xe[(size_t)i * S + s0];
        const float* xo = &xp.xo[(size_t)i * S + s0];
        const uint32_t* wv = wt[i >> 2];
        const int sh = 8 * (i & 3);
        for (int j = 0; j < 8; ++j) {
          A[j] = std::fmaf(xe[j], (float)((wv[j] >> sh) & 15u), A[j]);
          B[j] = std::fmaf(xo[j], (float)((wv[j] >> (sh + 4)) & 15u), B[j]);
        }
      }
    } else {
      for (int i = 0; i < 16; ++i)
        for (int j = 0; j < nb; ++j) {
          A[j] = std::fmaf(xp.xe[(size_t)i * S + s0 + j], (float)((wt[i >> 2][j] >> (8 * (i & 3))) & 15u), A[j]);
          B[j] = std::fmaf(xp.xo[(size_t)i * S + s0 + j], (float)((wt[i >> 2][j] >> (8 * (i & 3) + 4)) & 15u), B[j]);
        }
    }
    for (int j = 0; j < nb; ++j) {
      const float sc = h2f(srow[(s0 + j) / 2]), bi = h2f(brow[(s0 + j) / 2]);
      t[s0 + j] = std::fmaf(sc, A[j] + B[j], bi * xp.sx[s0 + j]);
    }
  }
  const int L = std::min(64, S), nblk = S / L;
  float p[64];
  for (int l = 0; l < L; ++l) {
    float acc = t[l];
    for (int blk = 1; blk < nblk; ++blk) acc = acc + t[blk * L + l];
    p[l] = acc;
  }
  return tree_sum(p, L);
}

// y[n] = f16(qdot) for n rows; x holds half values as floats.
static void qmv(const float* x, const sl_q4& q, int row0, int nrows, float* y) {
  XPrep xp; xp.set(x, q.k);
  const int W = q.k / 8, G = q.k / 64;
  if (q.k % 64 != 0 || q.k > 4096) { std::fprintf(stderr, "oracle qmv: K = %d is not a multiple of 64 up to 4096\n", q.k); std::abort(); }
#pragma omp parallel for schedule(static)
  for (int n = 0; n < nrows; ++n) {
    size_t r = (size_t)row0 + n;
    y[n] = f16r(qdot(xp, q.w + r * W, q.scales + r * G, q.biases + r * G));
  }
}

// Dense fp16 row dot (router gate, shared-expert gate): lane l of 64 owns K/64 contiguous elements.
static float dense_dot(const float* x, const uint16_t* wrow, int K) {
  const int per = K / 64;
  float p[64];
  for (int l = 0; l < 64; ++l) {
    float acc = 0.0f;
    for (int i = 0; i < per; ++i) acc = std::fmaf(x[l * per + i], h2f(wrow[l * per + i]), acc);
    p[l] = acc;
  }
  return tree_sum(p, 64);
}

// 8-bit affine row dot, group 64 (router gate and shared-expert gate of the released checkpoint; reference
// kernel qmm8, SeedlessMetalForward.swift:372-428: per 8 values `scale * sum(x*q) + bias * sum(x)`, the sum of x
// formed sequentially in fp32).  Lane l of 64 owns the 32 contiguous values 32l..32l+31, i.e. half a group and
// four terms of 8; a term is fmaf(s, chain of fmaf(x, q), b * sx), the lane's partial (t0+t1)+(t2+t3).
static float q8_dot(const float* x, const uint32_t* wrow, const uint16_t* srow, const uint16_t* brow, int K) {
  const uint8_t* q = reinterpret_cast<const uint8_t*>(wrow);   // little-endian: value j of a word in bits 8j..8j+7
  float p[64];
  for (int l = 0; l < 64; ++l) {
    const float s = h2f(srow[(32 * l) / 64]), b = h2f(brow[(32 * l) / 64]);
    float t[4];
    for (int j = 0; j < 4; ++j) {
      const int e0 = 32 * l + 8 * j;
      float dq = 0.0f, sx = 0.0f;
      for (int i = 0; i < 8; ++i) { dq = std::fmaf(x[e0 + i], (float)q[e0 + i], dq); sx = sx + x[e0 + i]; }
      t[j] = std::fmaf(s, dq, b * sx);
    }
    p[l] = (t[0] + t[1]) + (t[2] + t[3]);
  }
  (void)K;
  return tree_sum(p, 64);
}

// Sum of squares over D values (D/2 a power of two): pair terms fmaf(x1, x1, x0*x0), then a balanced binary tree
// over the D/2 pair terms, adjacent ones first.  (Any split of the vector into aligned power-of-two blocks reduces
// in this order: a lane that owns 32 elements, a wave of 64 pairs, 16 waves.)
static float sumsq(const float* x, int D) {
  std::vector<float> p((size_t)D / 2);
  for (int i = 0; i < D / 2; ++i) p[i] = std::fmaf(x[2 * i + 1], x[2 * i + 1], x[2 * i] * x[2 * i]);
  return tree_sum(p.data(), D / 2);
}
static inline float inv_rms(const float* x, int D) { return 1.0f / std::sqrt(sumsq(x, D) / (float)D + EPS); }

// rmsnorm (SeedlessMetalForward.swift:805-826): out = w * half(x * inv), both products in half.
// w == nullptr: weightless variant used for the GDN q/k norms, result scaled by half `scale`.
static void rmsnorm(const float* x, const uint16_t* w, int D, float* out) {
  const float inv = inv_rms(x, D);
  for (int i = 0; i < D; ++i) out[i] = f16r(h2f(w[i]) * f16r(x[i] * inv));
}

// ------------------------------------------------------------------------------------------------
struct GdnCache {
  std::vector<float> hist;    // [3][8192] half values, oldest first
  std::vector<float> state;   // [32][128][128] fp32, [hv][dv][dk]
  std::vector<float> hist_prev, state_prev;   // what one rollback restores
};
struct KvCache {
  std::vector<uint16_t> k, v; // [2][maxSeq][256]
};

struct Engine {
  sl_model_desc desc;
  std::vector<sl_layer_desc> layers;
  int maxM, maxSeq;
  int pos = 0;
  std::vector<GdnCache> gdn;
  std::vector<KvCache> kv;
  std::vector<float> ropeCos, ropeSin;        // [maxSeq][32]
  std::vector<float> hidden;                  // [M][H] last hidden rows
  std::vector<float> normed;                  // [M][H] last final-normed rows
  std::vector<float> logits;                  // [M][vocab]
  std::vector<int32_t> routeInds;             // [layer][maxM][8]
  std::vector<float> routeScores;
  std::string fault;
};

// ------------------------------------------------------------------------------------------------
// Embedding (SeedlessFusedVerify.swift:556-570): x = half(half(s*nib) + b).
static void embed_row(const Engine& e, int tok, float* h) {
  const sl_q4& q = e.desc.embed;
  const uint32_t* w = q.w + (size_t)tok * (H / 8);
  const uint16_t* s = q.scales + (size_t)tok * (H / 64);
  const uint16_t* b = q.biases + (size_t)tok * (H / 64);
  for (int j = 0; j < H; ++j) {
    float nib = (float)((w[j / 8] >> (4 * (j % 8))) & 15u);
    h[j] = f16r(f16r(h2f(s[j / 64]) * nib) + h2f(b[j / 64]));
  }
}

// ------------------------------------------------------------------------------------------------
// Router (SeedlessFusedVerify.swift:191-213): softmax over E half logits in fp32, gates rounded
// to half, 8 x arg-max of the raw logits with ties to the lower index, half renormalisation.
// Canonical: Z = tree over 64 lanes, lane l owning experts 4l..4l+3 (absent experts add +0).
static void route(const float* gl, int E, int32_t* inds, float* scores) {
  float m = -INFINITY;
  for (int i = 0; i < E; ++i) m = std::fmax(m, gl[i]);
  float ex[SL_MAX_EXPERTS], p[64];
  for (int i = 0; i < SL_MAX_EXPERTS; ++i) ex[i] = (i < E) ? exp_c(gl[i] - m) : 0.0f;
  for (int l = 0; l < 64; ++l) p[l] = ((ex[4 * l] + ex[4 * l + 1]) + ex[4 * l + 2]) + ex[4 * l + 3];
  const float Z = tree_sum(p, 64);
  float work[SL_MAX_EXPERTS];
  for (int i = 0; i < E; ++i) work[i] = gl[i];
  for (int k = 0; k < TOPK; ++k) {
    int bi = 0; float bv = work[0];
    for (int i = 1; i < E; ++i) if (work[i] > bv) { bv = work[i]; bi = i; }
    inds[k] = bi; scores[k] = f16r(ex[bi] / Z); work[bi] = -INFINITY;
  }
  float ss = 0.0f;
  for (int k = 0; k < TOPK; ++k) ss = f16r(ss + scores[k]);
  for (int k = 0; k < TOPK; ++k) scores[k] = f16r(scores[k] / ss);
}

// SwiGLU in half (SeedlessMetalForward.swift:982-991): h = (g * sigmoid16(g)) * u.
static inline float swiglu16(float g, float u) { return f16r(f16r(g * sigmoid16(g)) * u); }

// MoE block (SeedlessVerifyForward.swift:205-248; combine SeedlessFusedVerify.swift:462-470;
// shared gate + final combine :474-484).  x: normed rows; out: block output rows.
static void moe_block_rows(Engine& e, int li, const float* x, int M, float* out) {
  const sl_moe_w& w = e.layers[li].moe;
  const int E = e.desc.n_experts;
  std::vector<float> gl(E), g(I), u(I), act(I), d((size_t)TOPK * H), sg(I), su(I), sact(I), sy(H);
  for (int m = 0; m < M; ++m) {
    const float* xm = x + (size_t)m * H;
    for (int i = 0; i < E; ++i)
      gl[i] = w.router_w ? f16r(dense_dot(xm, w.router_w + (size_t)i * H, H))
                         : f16r(q8_dot(xm, w.router_q8.w + (size_t)i * (H / 4), w.router_q8.scales + (size_t)i * (H / 64),
                                       w.router_q8.biases + (size_t)i * (H / 64), H));
    int32_t* inds = &e.routeInds[((size_t)li * e.maxM + m) * TOPK];
    float* sc = &e.routeScores[((size_t)li * e.maxM + m) * TOPK];
    route(gl.data(), E, inds, sc);
    for (int k = 0; k < TOPK; ++k) {
      qmv(xm, w.sw_gate, inds[k] * I, I, g.data());
      qmv(xm, w.sw_up, inds[k] * I, I, u.data());
      for (int i = 0; i < I; ++i) act[i] = swiglu16(g[i], u[i]);
      qmv(act.data(), w.sw_down, inds[k] * H, H, &d[(size_t)k * H]);
    }
    qmv(xm, w.sh_gate, 0, I, sg.data());
    qmv(xm, w.sh_up, 0, I, su.data());
    for (int i = 0; i < I; ++i) sact[i] = swiglu16(sg[i], su[i]);
    qmv(sact.data(), w.sh_down, 0, H, sy.data());
    const float t = w.shared_gate_w ? f16r(dense_dot(xm, w.shared_gate_w, H))
                                    : f16r(q8_dot(xm, w.shared_gate_q8.w, w.shared_gate_q8.scales, w.shared_gate_q8.biases, H));
    const float s = sigmoid16(t);
    for (int n = 0; n < H; ++n) {
      float acc = 0.0f;
      for (int k = 0; k < TOPK; ++k) acc = f16r(acc + f16r(d[(size_t)k * H + n] * sc[k]));
      out[(size_t)m * H + n] = f16r(acc + f16r(s * sy[n]));
    }
  }
}

// One head of the gated delta rule (GatedDelta.swift:92-112): per state row dv,
// s *= g; kv = sum s*k; delta = (v - kv)*beta; s += k*delta; y = sum s*q.  Canonical order: 32
// lanes x 4 contiguous dk, fmaf chains, tree over the 32 lanes; y rounded to half.
static void delta_head_step(float* state, const float* qh, const float* kh, const float* v, float g, float beta, float* y) {
  for (int dv = 0; dv < GD; ++dv) {
    float* s = &state[(size_t)dv * GD];
    float p[32];
    for (int l = 0; l < 32; ++l) {
      float acc = 0.0f;
      for (int i = 0; i < 4; ++i) { s[4 * l + i] = s[4 * l + i] * g; acc = std::fmaf(s[4 * l + i], kh[4 * l + i], acc); }
      p[l] = acc;
    }
    const float kv = tree_sum(p, 32);
    const float delta = (v[dv] - kv) * beta;
    for (int l = 0; l < 32; ++l) {
      float acc = 0.0f;
      for (int i = 0; i < 4; ++i) { s[4 * l + i] = std::fmaf(kh[4 * l + i], delta, s[4 * l + i]); acc = std::fmaf(s[4 * l + i], qh[4 * l + i], acc); }
      p[l] = acc;
    }
    y[dv] = f16r(tree_sum(p, 32));
  }
}
static inline float gdn_beta(float b) { return sigmoid16(b); }
static inline float gdn_decay(float a, float a_log, float dt_bias) { return exp_c(-(exp_c(a_log) * softplus_c(a + dt_bias))); }
static inline float conv_silu(const float* win, const float* w) {
  float acc = 0.0f;
  for (int k = 0; k < CK; ++k) acc = std::fmaf(win[k], w[k], acc);
  return f16r(acc * sigmoid32(acc));
}

// ------------------------------------------------------------------------------------------------
// Gated-DeltaNet layer (SeedlessVerifyForward.swift:115-169).
//   conv + silu + history shift: SeedlessFusedVerify.swift:634-663 (fp32 taps, tap k multiplies
//     window row k, newest last);  q/k norm + scale, beta, g: :839-938;  recurrence:
//     GatedDelta.swift:63-124;  gated rmsnorm: SeedlessFusedVerify.swift:768-812.
static void gdn_layer_rows(Engine& e, int li, const float* x, int M, float* out) {
  const sl_gdn_w& w = e.layers[li].gdn;
  GdnCache& c = e.gdn[li];
  c.hist_prev = c.hist; c.state_prev = c.state;
  std::vector<float> cat((size_t)(CK - 1 + M) * CD), z((size_t)M * VALDIM), bP((size_t)M * HV), aP((size_t)M * HV);
  std::copy(c.hist.begin(), c.hist.end(), cat.begin());
  for (int m = 0; m < M; ++m) {
    const float* xm = x + (size_t)m * H;
    qmv(xm, w.in_proj_qkv, 0, CD, &cat[(size_t)(CK - 1 + m) * CD]);
    qmv(xm, w.in_proj_z, 0, VALDIM, &z[(size_t)m * VALDIM]);
    qmv(xm, w.in_proj_b, 0, HV, &bP[(size_t)m * HV]);
    qmv(xm, w.in_proj_a, 0, HV, &aP[(size_t)m * HV]);
  }
  std::vector<float> conv(CD), qn(KEYDIM), kn(KEYDIM), y(VALDIM), gated(VALDIM);
  const float qs = f16r(1.0f / 128.0f), ks = f16r(0.08838834764831845f);
  for (int m = 0; m < M; ++m) {
    for (int ch = 0; ch < CD; ++ch) {
      float win[CK];
      for (int k = 0; k < CK; ++k) win[k] = cat[(size_t)(m + k) * CD + ch];
      conv[ch] = conv_silu(win, &w.conv1d_w[ch * CK]);
    }
    for (int hk = 0; hk < HK; ++hk) {
      const float* q = &conv[hk * GD];
      const float* k = &conv[KEYDIM + hk * GD];
      const float qi = inv_rms(q, GD), ki = inv_rms(k, GD);
      for (int i = 0; i < GD; ++i) {
        qn[hk * GD + i] = f16r(qs * f16r(q[i] * qi));
        kn[hk * GD + i] = f16r(ks * f16r(k[i] * ki));
      }
    }
    const float* v = &conv[2 * KEYDIM];
#pragma omp parallel for schedule(static)
    for (int hv = 0; hv < HV; ++hv) {
      const float beta = gdn_beta(bP[(size_t)m * HV + hv]);
      const float g = gdn_decay(aP[(size_t)m * HV + hv], w.a_log[hv], w.dt_bias[hv]);
      const float* qh = &qn[(hv / (HV / HK)) * GD];
      const float* kh = &kn[(hv / (HV / HK)) * GD];
      delta_head_step(&c.state[(size_t)hv * GD * GD], qh, kh, &v[hv * GD], g, beta, &y[hv * GD]);
    }
    for (int hv = 0; hv < HV; ++hv) {
      const float inv = inv_rms(&y[hv * GD], GD);
      for (int i = 0; i < GD; ++i) {
        // fp32 weight: w * (y * inv) stays in fp32 (the reference's promote variant, SeedlessFusedVerify.swift:811)
        const float nrm = w.norm_w_f32 ? w.norm_w_f32[i] * (y[hv * GD + i] * inv) : f16r(h2f(w.norm_w[i]) * f16r(y[hv * GD + i] * inv));
        const float zf = z[(size_t)m * VALDIM + hv * GD + i];
        gated[hv * GD + i] = f16r((zf * sigmoid32(zf)) * nrm);
      }
    }
    qmv(gated.data(), w.out_proj, 0, H, out + (size_t)m * H);
  }
  std::copy(cat.begin() + (size_t)M * CD, cat.begin() + (size_t)(M + CK - 1) * CD, c.hist.begin());
}

// ------------------------------------------------------------------------------------------------
// Attention layer (SeedlessVerifyForward.swift:37-85).
//   q/k rmsnorm + partial RoPE: SeedlessFusedVerify.swift:1183-1260 (NeoX pairs (i, i+32), 64
//     rotary dims, theta 1e7, angle = float(pos)*freq);  decode attention:
//     SeedlessMetalForward.swift:4922-4989 (q pre-scaled by 1/16, fp32 softmax, fp16 out);
//     output gate: SeedlessMetalForward.swift:1012-1022.
// Canonical softmax order: keys in tiles of 64 aligned at absolute positions; per tile exact max,
// p = exp(s - max), l = tree over the 64 p, o = (fmaf chain over keys 0..31) + (fmaf chain over keys
// 32..63); tiles merged in order with the global max: L = sum l_t*f_t, O = sum o_t*f_t as fmaf
// chains, out = half(O/L).
static void build_rope(Engine& e) {
  e.ropeCos.resize((size_t)e.maxSeq * 32); e.ropeSin.resize((size_t)e.maxSeq * 32);
  for (int i = 0; i < 32; ++i) {
    const float freq = (float)std::exp(-2.0 * (double)i / (double)ROPE * std::log(1e7));
    for (int p = 0; p < e.maxSeq; ++p) {
      const float ang = (float)p * freq;
      e.ropeCos[(size_t)p * 32 + i] = (float)std::cos((double)ang);
      e.ropeSin[(size_t)p * 32 + i] = (float)std::sin((double)ang);
    }
  }
}
static void norm_rope(const Engine& e, const float* x, const uint16_t* w, int pos, float* out) {
  float nr[HD];
  rmsnorm(x, w, HD, nr);
  const float* c = &e.ropeCos[(size_t)pos * 32];
  const float* s = &e.ropeSin[(size_t)pos * 32];
  for (int d = 0; d < HD; ++d) {
    if (d >= ROPE) { out[d] = nr[d]; continue; }
    const int i = d % 32;
    const float x0 = nr[i], x1 = nr[i + 32];
    out[d] = (d < 32) ? f16r(std::fmaf(-x1, s[i], x0 * c[i])) : f16r(std::fmaf(x1, c[i], x0 * s[i]));
  }
}
// Score of one key: eight fmaf chains over 32 consecutive dims each, combined by a balanced tree (on the device a
// lane owns a key and a chain is the unit of work a wave can take).
static float dot256(const float* q, const uint16_t* k) {
  float c[8];
  for (int j = 0; j < 8; ++j) {
    float acc = 0.0f;
    for (int i = 0; i < 32; ++i) acc = std::fmaf(q[32 * j + i], h2f(k[32 * j + i]), acc);
    c[j] = acc;
  }
  return tree_sum(c, 8);
}
static void sdpa_row(const float* qrot /*[HD]*/, const uint16_t* kc, const uint16_t* vc, int N, float* out /*[HD]*/) {
  float q[HD];
  for (int d = 0; d < HD; ++d) q[d] = 0.0625f * qrot[d];
  const int nt = (N + SDPA_TILE - 1) / SDPA_TILE;
  std::vector<float> tm(nt), tl(nt), to((size_t)nt * HD);
  for (int t = 0; t < nt; ++t) {
    float s[SDPA_TILE], p[SDPA_TILE];
    const int j0 = t * SDPA_TILE, nk = std::min(SDPA_TILE, N - j0);
    float mx = -INFINITY;
    for (int j = 0; j < nk; ++j) { s[j] = dot256(q, kc + (size_t)(j0 + j) * HD); mx = std::fmax(mx, s[j]); }
    for (int j = 0; j < SDPA_TILE; ++j) p[j] = (j < nk) ? exp_c(s[j] - mx) : 0.0f;
    // weighted value sum of the tile: one fmaf chain over its first 32 keys, one over the other 32, added
    float* o = &to[(size_t)t * HD];
    float ob[HD];
    for (int d = 0; d < HD; ++d) { o[d] = 0.0f; ob[d] = 0.0f; }
    for (int j = 0; j < nk; ++j) {
      const uint16_t* vr = vc + (size_t)(j0 + j) * HD;
      float* dst = j < SDPA_TILE / 2 ? o : ob;
      for (int d = 0; d < HD; ++d) dst[d] = std::fmaf(p[j], h2f(vr[d]), dst[d]);
    }
    for (int d = 0; d < HD; ++d) o[d] = o[d] + ob[d];
    tm[t] = mx; tl[t] = tree_sum(p, SDPA_TILE);
  }
  float Mx = -INFINITY;
  for (int t = 0; t < nt; ++t) Mx = std::fmax(Mx, tm[t]);
  // Tiles are added up in blocks of 64: within a block one fmaf chain in tile order (from zero), the blocks' chains
  // added in block order.  (Up to 4096 keys that is a single chain over the tiles.)
  float Lsum = 0.0f, O[HD];
  for (int d = 0; d < HD; ++d) O[d] = 0.0f;
  for (int t0 = 0; t0 < nt; t0 += MERGE_BLOCK) {
    float Lb = 0.0f, Ob[HD];
    for (int d = 0; d < HD; ++d) Ob[d] = 0.0f;
    for (int t = t0; t < std::min(nt, t0 + MERGE_BLOCK); ++t) {
      const float f = exp_c(tm[t] - Mx);
      Lb = std::fmaf(tl[t], f, Lb);
      for (int d = 0; d < HD; ++d) Ob[d] = std::fmaf(to[(size_t)t * HD + d], f, Ob[d]);
    }
    Lsum = t0 == 0 ? Lb : Lsum + Lb;
    for (int d = 0; d < HD; ++d) O[d] = t0 == 0 ? Ob[d] : O[d] + Ob[d];
  }
  for (int d = 0; d < HD; ++d) out[d] = f16r(O[d] / Lsum);
}
static void attn_layer_rows(Engine& e, int li, const float* x, int M, int base, float* out) {
  const sl_attn_w& w = e.layers[li].attn;
  KvCache& c = e.kv[li];
  std::vector<float> qo((size_t)M * NH * 2 * HD), ko(NKV * HD), vo(NKV * HD), qrot((size_t)M * NH * HD), kr(HD);
  for (int m = 0; m < M; ++m) {
    const float* xm = x + (size_t)m * H;
    qmv(xm, w.q_proj, 0, NH * 2 * HD, &qo[(size_t)m * NH * 2 * HD]);
    qmv(xm, w.k_proj, 0, NKV * HD, ko.data());
    qmv(xm, w.v_proj, 0, NKV * HD, vo.data());
    const int pos = base + m;
    for (int h = 0; h < NH; ++h)
      norm_rope(e, &qo[((size_t)m * NH + h) * 2 * HD], w.q_norm, pos, &qrot[((size_t)m * NH + h) * HD]);
    for (int h = 0; h < NKV; ++h) {
      norm_rope(e, &ko[h * HD], w.k_norm, pos, kr.data());
      for (int d = 0; d < HD; ++d) {
        c.k[((size_t)h * e.maxSeq + pos) * HD + d] = f2h(kr[d]);
        c.v[((size_t)h * e.maxSeq + pos) * HD + d] = f2h(vo[h * HD + d]);
      }
    }
  }
  std::vector<float> gated((size_t)NH * HD);
  for (int m = 0; m < M; ++m) {
    const int N = base + m + 1;
#pragma omp parallel for schedule(static)
    for (int h = 0; h < NH; ++h) {
      const int kvh = h / (NH / NKV);
      float ao[HD];
      sdpa_row(&qrot[((size_t)m * NH + h) * HD], &c.k[(size_t)kvh * e.maxSeq * HD], &c.v[(size_t)kvh * e.maxSeq * HD], N, ao);
      const float* gate = &qo[((size_t)m * NH + h) * 2 * HD + HD];
      for (int d = 0; d < HD; ++d) gated[h * HD + d] = f16r(ao[d] * sigmoid16(gate[d]));
    }
    qmv(gated.data(), w.o_proj, 0, H, out + (size_t)m * H);
  }
}

// ------------------------------------------------------------------------------------------------
// Decoder stack (SeedlessVerifyForward.swift:284-309; residual adds in fp32 rounded to half,
// SeedlessFusedVerify.swift:969).  h: [M][H] in/out.
static void forward_layers(Engine& e, float* h, int M) {
  std::vector<float> nr((size_t)M * H), r((size_t)M * H);
  const int base = e.pos;
  for (int li = 0; li < e.desc.n_layers; ++li) {
    const sl_layer_desc& L = e.layers[li];
    for (int m = 0; m < M; ++m) rmsnorm(h + (size_t)m * H, L.input_ln, H, &nr[(size_t)m * H]);
    if (L.is_linear) gdn_layer_rows(e, li, nr.data(), M, r.data());
    else attn_layer_rows(e, li, nr.data(), M, base, r.data());
    for (size_t i = 0; i < (size_t)M * H; ++i) h[i] = f16r(h[i] + r[i]);
    for (int m = 0; m < M; ++m) rmsnorm(h + (size_t)m * H, L.post_ln, H, &nr[(size_t)m * H]);
    moe_block_rows(e, li, nr.data(), M, r.data());
    for (size_t i = 0; i < (size_t)M * H; ++i) h[i] = f16r(h[i] + r[i]);
  }
  e.pos = base + M;
}

// lm_head + first-index argmax (SeedlessFusedVerify.swift:3855-3876, 572-596).
static int head_argmax(Engine& e, const float* normed, float* logits) {
  qmv(normed, e.desc.lm_head, 0, e.desc.vocab, logits);
  int bi = 0; float bv = logits[0];
  for (int v = 1; v < e.desc.vocab; ++v) if (logits[v] > bv) { bv = logits[v]; bi = v; }
  return bi;
}

static bool check_rows(Engine* e, int M) {
  if (!e || M < 1 || M > e->maxM) return false;
  bool has_attn = false;
  for (auto& L : e->layers) has_attn |= !L.is_linear;
  if (has_attn && e->pos + M > e->maxSeq) return false;
  return true;
}

}  // namespace orc

using namespace orc;

extern "C" {

// ---- engine-level mirror of the C ABI in include/seedless_hip.h (host pointers only) -------------
Engine* orc_create(const sl_model_desc* d, int maxM, int maxSeq) {
  if (!d || d->location != SL_LOC_HOST || maxM < 1 || maxSeq < 1) return nullptr;
  Engine* e = new Engine();
  e->desc = *d;
  e->layers.assign(d->layers, d->layers + d->n_layers);
  e->desc.layers = e->layers.data();
  e->maxM = maxM; e->maxSeq = maxSeq;
  e->gdn.resize(d->n_layers); e->kv.resize(d->n_layers);
  for (int i = 0; i < d->n_layers; ++i) {
    if (e->layers[i].is_linear) {
      e->gdn[i].hist.assign((size_t)(CK - 1) * CD, 0.0f);
      e->gdn[i].state.assign((size_t)HV * GD * GD, 0.0f);
    } else {
      e->kv[i].k.assign((size_t)NKV * maxSeq * HD, 0);
      e->kv[i].v.assign((size_t)NKV * maxSeq * HD, 0);
    }
  }
  build_rope(*e);
  e->hidden.assign((size_t)maxM * H, 0.0f);
  e->normed.assign((size_t)maxM * H, 0.0f);
  if (d->lm_head.w) e->logits.assign((size_t)maxM * d->vocab, 0.0f);
  e->routeInds.assign((size_t)d->n_layers * maxM * TOPK, 0);
  e->routeScores.assign((size_t)d->n_layers * maxM * TOPK, 0.0f);
  return e;
}
void orc_destroy(Engine* e) { delete e; }
int orc_position(const Engine* e) { return e->pos; }

int orc_forward_rows(Engine* e, const uint16_t* x, int M, int final_norm, uint16_t* out) {
  if (!check_rows(e, M) || !x || !out) return SL_ERR_ARG;
  for (size_t i = 0; i < (size_t)M * H; ++i) e->hidden[i] = h2f(x[i]);
  forward_layers(*e, e->hidden.data(), M);
  const float* src = e->hidden.data();
  if (final_norm) {
    for (int m = 0; m < M; ++m) rmsnorm(&e->hidden[(size_t)m * H], e->desc.final_norm, H, &e->normed[(size_t)m * H]);
    src = e->normed.data();
  }
  for (size_t i = 0; i < (size_t)M * H; ++i) out[i] = f2h(src[i]);
  return SL_OK;
}
int orc_step_argmax(Engine* e, const int32_t* tok, int M, int32_t* out) {
  if (!check_rows(e, M) || !tok || !out || !e->desc.embed.w) return SL_ERR_ARG;
  for (int m = 0; m < M; ++m) {
    if (tok[m] < 0 || tok[m] >= e->desc.vocab) return SL_ERR_ARG;
    embed_row(*e, tok[m], &e->hidden[(size_t)m * H]);
  }
  forward_layers(*e, e->hidden.data(), M);
  for (int m = 0; m < M; ++m) {
    rmsnorm(&e->hidden[(size_t)m * H], e->desc.final_norm, H, &e->normed[(size_t)m * H]);
    out[m] = head_argmax(*e, &e->normed[(size_t)m * H], &e->logits[(size_t)m * e->desc.vocab]);
  }
  return SL_OK;
}
int orc_forward_tokens(Engine* e, const int32_t* tok, int M, uint16_t* out) {
  if (!check_rows(e, M) || !tok || !out || !e->desc.embed.w) return SL_ERR_ARG;
  for (int m = 0; m < M; ++m) embed_row(*e, tok[m], &e->hidden[(size_t)m * H]);
  forward_layers(*e, e->hidden.data(), M);
  for (int m = 0; m < M; ++m) rmsnorm(&e->hidden[(size_t)m * H], e->desc.final_norm, H, &e->normed[(size_t)m * H]);
  for (size_t i = 0; i < (size_t)M * H; ++i) out[i] = f2h(e->normed[i]);
  return SL_OK;
}
int orc_head_argmax(Engine* e, const uint16_t* normed, int M, int32_t* out) {
  if (!e || M < 1 || M > e->maxM || !e->desc.lm_head.w) return SL_ERR_ARG;
  std::vector<float> nr(H);
  for (int m = 0; m < M; ++m) {
    for (int i = 0; i < H; ++i) nr[i] = h2f(normed[(size_t)m * H + i]);
    out[m] = head_argmax(*e, nr.data(), &e->logits[(size_t)m * e->desc.vocab]);
  }
  return SL_OK;
}
int orc_chained_step_argmax(Engine* e, int32_t first, int K, int32_t* out) {
  int32_t t = first;
  for (int k = 0; k < K; ++k) { int r = orc_step_argmax(e, &t, 1, &out[k]); if (r) return r; t = out[k]; }
  return SL_OK;
}
int orc_greedy_generate(Engine* e, const int32_t* prompt, int nPrompt, int nNew, int32_t* out) {
  std::vector<uint16_t> nr((size_t)e->maxM * H);
  int done = 0, lastM = 0;
  while (done < nPrompt) {
    lastM = std::min(e->maxM, nPrompt - done);
    int r = orc_forward_tokens(e, prompt + done, lastM, nr.data()); if (r) return r;
    done += lastM;
  }
  if (nNew < 1) return SL_OK;
  int32_t t;
  int r = orc_head_argmax(e, &nr[(size_t)(lastM - 1) * H], 1, &t); if (r) return r;
  out[0] = t;
  for (int k = 1; k < nNew; ++k) { r = orc_step_argmax(e, &t, 1, &out[k]); if (r) return r; t = out[k]; }
  return SL_OK;
}
int orc_logits_row(Engine* e, int m, uint16_t* out) {
  if (!e || m < 0 || m >= e->maxM || e->logits.empty()) return SL_ERR_ARG;
  for (int v = 0; v < e->desc.vocab; ++v) out[v] = f2h(e->logits[(size_t)m * e->desc.vocab + v]);
  return SL_OK;
}
int orc_hidden_rows(Engine* e, int M, uint16_t* out) {
  if (!e || M < 1 || M > e->maxM) return SL_ERR_ARG;
  for (size_t i = 0; i < (size_t)M * H; ++i) out[i] = f2h(e->normed[i]);
  return SL_OK;
}
int orc_read_route(Engine* e, int layer, int M, int32_t* inds, uint16_t* scores) {
  if (!e || layer < 0 || layer >= e->desc.n_layers || M < 1 || M > e->maxM) return SL_ERR_ARG;
  for (int i = 0; i < M * TOPK; ++i) {
    inds[i] = e->routeInds[(size_t)layer * e->maxM * TOPK + i];
    scores[i] = f2h(e->routeScores[(size_t)layer * e->maxM * TOPK + i]);
  }
  return SL_OK;
}
int orc_read_layer_cache(Engine* e, int layer, void* a, void* b) {
  if (!e || layer < 0 || layer >= e->desc.n_layers) return SL_ERR_ARG;
  if (e->layers[layer].is_linear) {
    const GdnCache& c = e->gdn[layer];
    if (a) for (size_t i = 0; i < c.hist.size(); ++i) ((uint16_t*)a)[i] = f2h(c.hist[i]);
    if (b) std::memcpy(b, c.state.data(), c.state.size() * 4);
  } else {
    const KvCache& c = e->kv[layer];
    for (int h = 0; h < NKV; ++h) {
      if (a) std::memcpy((uint16_t*)a + (size_t)h * e->pos * HD, &c.k[(size_t)h * e->maxSeq * HD], (size_t)e->pos * HD * 2);
      if (b) std::memcpy((uint16_t*)b + (size_t)h * e->pos * HD, &c.v[(size_t)h * e->maxSeq * HD], (size_t)e->pos * HD * 2);
    }
  }
  return SL_OK;
}
int orc_load_layer_cache(Engine* e, int layer, const void* a, const void* b, int len) {
  if (!e || layer < 0 || layer >= e->desc.n_layers) return SL_ERR_ARG;
  if (e->layers[layer].is_linear) {
    GdnCache& c = e->gdn[layer];
    if (a) for (size_t i = 0; i < c.hist.size(); ++i) c.hist[i] = h2f(((const uint16_t*)a)[i]);
    if (b) std::memcpy(c.state.data(), b, c.state.size() * 4);
  } else {
    if (len < 0 || len > e->maxSeq) return SL_ERR_ARG;
    KvCache& c = e->kv[layer];
    for (int h = 0; h < NKV; ++h) {
      if (a) std::memcpy(&c.k[(size_t)h * e->maxSeq * HD], (const uint16_t*)a + (size_t)h * len * HD, (size_t)len * HD * 2);
      if (b) std::memcpy(&c.v[(size_t)h * e->maxSeq * HD], (const uint16_t*)b + (size_t)h * len * HD, (size_t)len * HD * 2);
    }
    e->pos = len;
  }
  return SL_OK;
}
// One-step rollback: KV by position, GDN from the copy taken before the last forward.
int orc_rollback_one_step(Engine* e, int pos_before) {
  e->pos = pos_before;
  for (int i = 0; i < e->desc.n_layers; ++i)
    if (e->layers[i].is_linear && !e->gdn[i].hist_prev.empty()) { e->gdn[i].hist = e->gdn[i].hist_prev; e->gdn[i].state = e->gdn[i].state_prev; }
  return SL_OK;
}

static void rows_in(const uint16_t* x, int M, std::vector<float>& v) { v.resize((size_t)M * H); for (size_t i = 0; i < v.size(); ++i) v[i] = h2f(x[i]); }
static void rows_out(const std::vector<float>& v, uint16_t* out) { for (size_t i = 0; i < v.size(); ++i) out[i] = f2h(v[i]); }
int orc_moe_block_rows(Engine* e, int layer, const uint16_t* x, int M, uint16_t* out) {
  if (!e || M < 1 || M > e->maxM) return SL_ERR_ARG;
  std::vector<float> xi, o((size_t)M * H); rows_in(x, M, xi);
  moe_block_rows(*e, layer, xi.data(), M, o.data()); rows_out(o, out); return SL_OK;
}
int orc_gdn_layer_rows(Engine* e, int layer, const uint16_t* x, int M, uint16_t* out) {
  if (!e || M < 1 || M > e->maxM || !e->layers[layer].is_linear) return SL_ERR_ARG;
  std::vector<float> xi, o((size_t)M * H); rows_in(x, M, xi);
  gdn_layer_rows(*e, layer, xi.data(), M, o.data()); rows_out(o, out); return SL_OK;
}
int orc_attn_layer_rows(Engine* e, int layer, const uint16_t* x, int M, uint16_t* out) {
  if (!check_rows(e, M) || e->layers[layer].is_linear) return SL_ERR_ARG;
  std::vector<float> xi, o((size_t)M * H); rows_in(x, M, xi);
  attn_layer_rows(*e, layer, xi.data(), M, e->pos, o.data()); e->pos += M; rows_out(o, out); return SL_OK;
}

// ---- primitives, exported so tests can pin each against closed forms ------------------------------
float orc_exp(float x) { return exp_c(x); }
float orc_log(float x) { return log_c(x); }
float orc_sigmoid32(float x) { return sigmoid32(x); }
float orc_sigmoid16(float x) { return sigmoid16(x); }
float orc_softplus(float x) { return softplus_c(x); }
float orc_ppnd7(float p) { return ppnd7(p); }
float orc_f16r(float x) { return f16r(x); }
uint16_t orc_f2h(float x) { return f2h(x); }
uint16_t orc_f2h_soft(float x) { return f2h_soft(x); }
float orc_h2f(uint16_t h) { return h2f(h); }
float orc_h2f_soft(uint16_t h) { return h2f_soft(h); }
uint64_t orc_hash64(uint64_t seed, uint64_t idx) { return hash64(seed, idx); }
float orc_normal01(uint64_t seed, uint64_t idx) { return normal01(seed, idx); }
void orc_exp_vec(const float* x, float* y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = exp_c(x[i]); }
void orc_log_vec(const float* x, float* y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = log_c(x[i]); }
// y[i] = op(x[i]); op numbering as in sl_selftest_math.
void orc_map_vec(int op, const float* x, float* y, int64_t n) {
  for (int64_t i = 0; i < n; ++i) {
    const float v = x[i];
    float r;
    switch (op) {
      case 0: r = exp_c(v); break;
      case 1: r = log_c(v); break;
      case 2: r = sigmoid32(v); break;
      case 3: r = sigmoid16(v); break;
      case 4: r = softplus_c(v); break;
      case 5: r = f16r(v); break;
      case 6: r = 1.0f / std::sqrt(v / 128.0f + EPS); break;
      case 7: r = f16r(v * sigmoid32(v)); break;
      default: r = ppnd7(v); break;
    }
    y[i] = r;
  }
}
void orc_ppnd7_vec(const float* x, float* y, int64_t n) { for (int64_t i = 0; i < n; ++i) y[i] = ppnd7(x[i]); }

void orc_qmv(const uint16_t* x, const uint32_t* w, const uint16_t* s, const uint16_t* b, int n, int k, uint16_t* y) {
  std::vector<float> xf(k), yf(n);
  for (int i = 0; i < k; ++i) xf[i] = h2f(x[i]);
  sl_q4 q{w, s, b, n, k};
  qmv(xf.data(), q, 0, n, yf.data());
  for (int i = 0; i < n; ++i) y[i] = f2h(yf[i]);
}
// The same dot without the final half rounding (for accuracy checks against float64).
void orc_qmv_f32(const uint16_t* x, const uint32_t* w, const uint16_t* s, const uint16_t* b, int n, int k, float* y) {
  std::vector<float> xf(k);
  for (int i = 0; i < k; ++i) xf[i] = h2f(x[i]);
  XPrep xp; xp.set(xf.data(), k);
  for (int r = 0; r < n; ++r) y[r] = qdot(xp, w + (size_t)r * (k / 8), s + (size_t)r * (k / 64), b + (size_t)r * (k / 64));
}
void orc_dense_f16(const uint16_t* x, const uint16_t* w, int n, int k, uint16_t* y) {
  std::vector<float> xf(k);
  for (int i = 0; i < k; ++i) xf[i] = h2f(x[i]);
  for (int r = 0; r < n; ++r) y[r] = f2h(dense_dot(xf.data(), w + (size_t)r * k, k));
}
// 8-bit rows (K = 2048): y = q8_dot before the half rounding, for checks against float64.
void orc_q8_f32(const uint16_t* x, const uint32_t* w, const uint16_t* s, const uint16_t* b, int n, int k, float* y) {
  std::vector<float> xf(k);
  for (int i = 0; i < k; ++i) xf[i] = h2f(x[i]);
  for (int r = 0; r < n; ++r) y[r] = q8_dot(xf.data(), w + (size_t)r * (k / 4), s + (size_t)r * (k / 64), b + (size_t)r * (k / 64), k);
}
void orc_rmsnorm(const uint16_t* x, const uint16_t* w, int D, uint16_t* y) {
  std::vector<float> xf(D), yf(D);
  for (int i = 0; i < D; ++i) xf[i] = h2f(x[i]);
  rmsnorm(xf.data(), w, D, yf.data());
  for (int i = 0; i < D; ++i) y[i] = f2h(yf[i]);
}
void orc_route(const uint16_t* logits, int E, int32_t* inds, uint16_t* scores) {
  float gl[SL_MAX_EXPERTS], sc[TOPK];
  for (int i = 0; i < E; ++i) gl[i] = h2f(logits[i]);
  route(gl, E, inds, sc);
  for (int k = 0; k < TOPK; ++k) scores[k] = f2h(sc[k]);
}
void orc_swiglu(const uint16_t* g, const uint16_t* u, int n, uint16_t* out) {
  for (int i = 0; i < n; ++i) out[i] = f2h(swiglu16(h2f(g[i]), h2f(u[i])));
}
// q: [256] half (post-RoPE, unscaled); k, v: [N, 256] half.
void orc_sdpa(const uint16_t* q, const uint16_t* k, const uint16_t* v, int N, uint16_t* out) {
  float qf[HD], of[HD];
  for (int d = 0; d < HD; ++d) qf[d] = h2f(q[d]);
  sdpa_row(qf, k, v, N, of);
  for (int d = 0; d < HD; ++d) out[d] = f2h(of[d]);
}
// Rotary table entry, as built at engine creation.
void orc_rope_entry(int pos, int i, float* c, float* s) {
  const float freq = (float)std::exp(-2.0 * (double)i / (double)ROPE * std::log(1e7));
  const float ang = (float)pos * freq;
  *c = (float)std::cos((double)ang); *s = (float)std::sin((double)ang);
}
void orc_norm_rope(const uint16_t* x, const uint16_t* w, int pos, uint16_t* out) {
  Engine e; e.maxSeq = pos + 1; build_rope(e);
  float xf[HD], of[HD];
  for (int d = 0; d < HD; ++d) xf[d] = h2f(x[d]);
  norm_rope(e, xf, w, pos, of);
  for (int d = 0; d < HD; ++d) out[d] = f2h(of[d]);
}

// Gated delta rule on nhv value heads sharing nhk key heads; q, k: [nhk,128] half values as
// float, v: [nhv,128], state: [nhv,128,128] updated in place, y: [nhv,128].
void orc_delta_step(float* state, const float* q, const float* k, const float* v, const float* g, const float* beta,
                    int nhk, int nhv, float* y) {
  for (int hv = 0; hv < nhv; ++hv)
    delta_head_step(state + (size_t)hv * GD * GD, q + (hv / (nhv / nhk)) * GD, k + (hv / (nhv / nhk)) * GD,
                    v + hv * GD, g[hv], beta[hv], y + hv * GD);
}
float orc_gdn_beta(float b) { return gdn_beta(b); }
float orc_gdn_decay(float a, float a_log, float dt_bias) { return gdn_decay(a, a_log, dt_bias); }
float orc_conv_silu(const float* win, const float* w) { return conv_silu(win, w); }

// ---- synthetic tensors: the host statement of sl_synth_q4 / sl_synth_f16 / sl_synth_f32 -----------
// MLX affine quantisation rule, group 64 (as published for mlx.core.quantize, mode "affine").
void orc_synth_q4(uint32_t* w, uint16_t* sc, uint16_t* bi, int64_t n, int32_t k, uint64_t seed, float sigma) {
  const int G = k / 64;
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < n; ++r) {
    for (int g = 0; g < G; ++g) {
      float v[64];
      float mn = INFINITY, mx = -INFINITY;
      for (int i = 0; i < 64; ++i) {
        v[i] = sigma * normal01(seed, (uint64_t)r * (uint64_t)k + (uint64_t)(g * 64 + i));
        mn = std::fmin(mn, v[i]); mx = std::fmax(mx, v[i]);
      }
      const bool mask = std::fabs(mn) > std::fabs(mx);
      float scale = std::fmax((mx - mn) / 15.0f, 1e-7f);
      scale = mask ? scale : -scale;
      const float edge = mask ? mn : mx;
      const float q0 = std::rint(edge / scale);
      float bias = 0.0f;
      if (q0 != 0.0f) { scale = edge / q0; bias = edge; }
      sc[r * G + g] = f2h(scale); bi[r * G + g] = f2h(bias);
      for (int wd = 0; wd < 8; ++wd) {
        uint32_t pack = 0;
        for (int i = 0; i < 8; ++i) {
          float q = std::rint((v[wd * 8 + i] - bias) / scale);
          q = std::fmin(std::fmax(q, 0.0f), 15.0f);
          pack |= (uint32_t)q << (4 * i);
        }
        w[(r * G + g) * 8 + wd] = pack;
      }
    }
  }
}
void orc_synth_f16(uint16_t* dst, int64_t count, uint64_t seed, float mean, float sigma) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < count; ++i) dst[i] = f2h(mean + sigma * normal01(seed, (uint64_t)i));
}
void orc_synth_f32(float* dst, int64_t count, uint64_t seed, float mean, float sigma) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < count; ++i) dst[i] = mean + sigma * normal01(seed, (uint64_t)i);
}

}  // extern "C"
