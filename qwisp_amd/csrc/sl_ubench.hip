// Micro-benchmarks of the three machine limits that bound the Seedless kernels on gfx950.  They are measurement
// hooks of the library (no counterpart in the reference); bench.py --microbench runs them and prints their figures.
//
//  * sl_ubench_exchange: the dependent hand-over between the 256 resident workgroups of a persistent launch.  Every
//    round each workgroup publishes a few tagged words (one wave, coherent stores), polls the words of its peers with
//    coherent loads until all tags are the round's, and only then can form what it publishes next.
//  * sl_ubench_gemv_stream: 4-bit rows streamed back to back through the step kernel's own dot code with no stage
//    boundary in between: what the weight stream of a stage could reach if it never had to wait.
//  * sl_ubench_mfma_issue: v_mfma_f32_32x32x16_f16 with vector instructions (the in-register 4-bit unpacking of the
//    matrix-core GEMMs) and LDS operand reads mixed in: the issue cost of everything that is not a matrix instruction.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <vector>

#include "sl_device.cuh"
#include "../../include/seedless_hip.h"

namespace sl {
namespace {

typedef uint32_t ub_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t ub_u32x2 __attribute__((ext_vector_type(2)));
SL_DEV __amdgpu_buffer_rsrc_t ub_rsrc(const void* p) { return __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, 0x7fffffff, 0x00020000); }
constexpr int UB_SC1 = 16;                       // agent-coherent cache policy of the polls and stores
constexpr unsigned UB_SPINS = 200000;            // every wait is bounded: a workgroup that gives up raises `fail` and leaves

__shared__ unsigned ub_flag[4];

// mode 0: all-gather of 2048 words, the first eight waves poll 16 bytes per thread, one barrier per polling round
// mode 1: the same, every wave repeats its own share until it is complete, one barrier per hand-over
// mode 2: every thread polls the pair of words it owns (8 bytes), one barrier per hand-over (the step kernel's shape)
// mode 3: 256 words among the 32 workgroups of one XCD (workgroup n runs on XCD n % 8)
// mode 4: 256 words among 32 workgroups spread over all XCDs
__global__ __launch_bounds__(1024) void k_ub_exchange(uint32_t* buf, int mode, int rounds, unsigned long long* times, unsigned* fail) {
  const int tid = threadIdx.x, wg = blockIdx.x, wave = tid >> 6, lane = tid & 63;
  if (tid < 4) ub_flag[tid] = 0;
  __syncthreads();
  unsigned acc = 0;
  unsigned long long t0 = 0;
  for (int r = 0; r < rounds; ++r) {
    const unsigned tag = (unsigned)(r + 1) & 0xffffu;
    uint32_t* b = buf + (r & 1) * 2048;
    if (r == 8 && tid == 0) t0 = wall_clock64();
    if (wave == 15 && lane < 8) {                 // publish this workgroup's 8 words (their value depends on the round before)
      const unsigned v = ((acc + wg * 8 + lane) & 0xffffu) | (tag << 16);
      __builtin_amdgcn_raw_buffer_store_b32(v, ub_rsrc(b), 4 * (wg * 8 + lane), 0, UB_SC1);
    }
    const auto rr = ub_rsrc(b);
    bool gave_up = false;
    if (mode == 0 || mode >= 3) {
      const int pollers = mode == 0 ? 512 : 64;
      bool ok = tid >= pollers, done = false;
      unsigned spins = 0;
      for (; spins < UB_SPINS && !done; ++spins) {
        if (!ok) {
          int word = 4 * tid;
          if (mode >= 3) {                        // members of the group: same XCD (wg % 8 + 8 j) or neighbours (32 (wg / 32) + j)
            const int member = mode == 3 ? (wg & 7) + 8 * (tid >> 1) : (wg & ~31) + (tid >> 1);
            word = member * 8 + 4 * (tid & 1);
          }
          const ub_u32x4 q = __builtin_amdgcn_raw_buffer_load_b128(rr, 4 * word, 0, UB_SC1);
          ok = (q.x >> 16) == tag && (q.y >> 16) == tag && (q.z >> 16) == tag && (q.w >> 16) == tag;
          if (ok) acc += (q.x + q.y + q.z + q.w) & 0xffffu;
        }
        const unsigned slot = spins % 3u;
        if (!__all(ok ? 1 : 0) && lane == 0) ub_flag[slot] = 1;
        lds_barrier();
        const unsigned failed = ub_flag[slot];
        if (tid == 0) ub_flag[(spins + 2u) % 3u] = 0;
        done = !failed;
      }
      gave_up = !done;
    } else {
      bool ok = false;
      unsigned spins = 0;
      const bool polls = mode == 2 || wave < 8;
      for (; polls && spins < UB_SPINS; ++spins) {
        if (!ok) {
          if (mode == 1) {
            const ub_u32x4 q = __builtin_amdgcn_raw_buffer_load_b128(rr, 16 * tid, 0, UB_SC1);
            ok = (q.x >> 16) == tag && (q.y >> 16) == tag && (q.z >> 16) == tag && (q.w >> 16) == tag;
            if (ok) acc += (q.x + q.y + q.z + q.w) & 0xffffu;
          } else {
            const ub_u32x2 q = __builtin_amdgcn_raw_buffer_load_b64(rr, 8 * tid, 0, UB_SC1);
            ok = (q.x >> 16) == tag && (q.y >> 16) == tag;
            if (ok) acc += (q.x + q.y) & 0xffffu;
          }
        }
        if (__all(ok ? 1 : 0)) break;
      }
      if (polls && spins >= UB_SPINS && lane == 0) ub_flag[3] = 1;
      lds_barrier();
      gave_up = ub_flag[3] != 0;
    }
    if (gave_up) { if (tid == 0) fail[0] = 1; return; }
    acc = __shfl(acc, 0);
  }
  if (tid == 0) { times[wg * 2] = t0; times[wg * 2 + 1] = wall_clock64(); }
}

// Wave gw takes chunks of 64 consecutive rows of 2048 weights, four rows per iteration, the next four in flight.
// mode 0: loads only; 1: with the dots (share_term); 2: with the dots and the 64-lane reduction per row.
template <int MODE>
__global__ __launch_bounds__(1024) void k_ub_gemv(const uint32_t* __restrict__ W, const uint32_t* __restrict__ SB, long nrows, float* out) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long NW = (long)gridDim.x * 16, gw = (long)blockIdx.x * 16 + wave;
  uint32_t xp[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) xp[i] = 0x3c003c00u ^ (uint32_t)(lane * 7 + i);
  const float sx = 1.0f + lane;
  float acc = 0.0f;
  uint32_t xacc = 0;
  const long nchunks = nrows / 64;
  for (long chunk = gw; chunk < nchunks; chunk += NW) {
    uint4 cur[4], nxt[4];
    uint32_t csb[4], nsb[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) { const long r = chunk * 64 + j; cur[j] = ld16(W + r * 256 + 4 * lane); csb[j] = SB[r * 32 + (lane >> 1)]; }
    for (int g = 0; g < 16; ++g) {
      const int ng = (g + 1) & 15;
      const long nc = (g == 15) ? chunk + NW : chunk;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const long r = min(nc, nchunks - 1) * 64 + ng * 4 + j;
        nxt[j] = ld16(W + r * 256 + 4 * lane); nsb[j] = SB[r * 32 + (lane >> 1)];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (MODE == 0) {
          xacc ^= cur[j].x ^ cur[j].y ^ cur[j].z ^ cur[j].w ^ csb[j];
        } else {
          float t = share_term(cur[j], csb[j], xp, sx);
          if (MODE == 2) t = tree_sum<64>(t);
          acc += t;
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) { cur[j] = nxt[j]; csb[j] = nsb[j]; }
    }
  }
  if (acc == 12345.678f || xacc == 0xdeadbeefu) out[0] = acc + (float)xacc;   // (keeps the work alive)
}

typedef float ub_f16v __attribute__((ext_vector_type(16)));
typedef _Float16 ub_h8 __attribute__((ext_vector_type(8)));
// Four accumulator tiles per wave; per matrix instruction VALU unpacking steps (mask-and-or, subtract, fused
// multiply-add on a half pair: 3 vector instructions each) and optionally one 16-byte LDS operand read.
template <int VALU, int LDSR>
__global__ __launch_bounds__(256) void k_ub_mfma(float* out, int iters, uint32_t seed) {
  __shared__ __align__(16) uint16_t lds[16384];
  for (int i = threadIdx.x; i < 16384; i += 256) lds[i] = (uint16_t)(0x3c00 + (i & 7));
  __syncthreads();
  constexpr int NACC = 4;
  ub_f16v acc[NACC];
#pragma unroll
  for (int t = 0; t < NACC; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[t][r] = 0.0f;
  ub_h8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) { a[i] = (_Float16)(0.001f * (threadIdx.x + i)); b[i] = (_Float16)(0.002f * i); }
  uint32_t w = seed + threadIdx.x;
  const h2_t s2 = {(_Float16)0.01f, (_Float16)0.01f}, b2 = {(_Float16)-0.07f, (_Float16)-0.07f};
  const int lane = threadIdx.x & 63;
  uint32_t k1024 = 0x64006400u;
  asm volatile("" : "+v"(k1024));
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int t = 0; t < NACC; ++t) {
      if (LDSR) a = *reinterpret_cast<const ub_h8*>(&lds[((lane & 31) * 136 + (lane >> 5) * 32 + ((it * NACC + t) & 7) * 8) & 16383 & ~7]);
      acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[t], 0, 0, 0);
#pragma unroll
      for (int v = 0; v < VALU; ++v) {
        const h2_t f1024 = {(_Float16)1024.0f, (_Float16)1024.0f};
        const h2_t q = as_h2(((w >> (4 * (v & 3))) & 0x000F000Fu) | k1024) - f1024;
        const h2_t r = __builtin_elementwise_fma(q, s2, b2);
        b[(2 * v) & 7] = r[0]; b[(2 * v + 1) & 7] = r[1];
        w += 0x01010101u;
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  float sum = 0.0f;
#pragma unroll
  for (int t = 0; t < NACC; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) sum += acc[t][r];
  out[blockIdx.x * 256 + threadIdx.x] = sum;
}

template <typename T>
struct DevBuf {
  T* p = nullptr;
  explicit DevBuf(size_t n, int fill = 0) { if (hipMalloc(&p, n * sizeof(T)) != hipSuccess) p = nullptr; else (void)hipMemset(p, fill, n * sizeof(T)); }
  ~DevBuf() { if (p) (void)hipFree(p); }
};

}  // namespace
}  // namespace sl

using namespace sl;

extern "C" {

int sl_ubench_exchange(int mode, int rounds, float* us_per_round) {
  if (mode < 0 || mode > 4 || rounds < 16 || rounds > 100000 || !us_per_round) return SL_ERR_ARG;
  int per_cu = 0, dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return SL_ERR_DEVICE;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)k_ub_exchange, 1024, 0) != hipSuccess) return SL_ERR_DEVICE;
  if (per_cu < 1 || prop.multiProcessorCount < 256) return SL_ERR_UNSUPPORTED;     // all 256 workgroups must be resident at once
  DevBuf<uint32_t> buf(2 * 2048);
  DevBuf<unsigned long long> times(512);
  DevBuf<unsigned> fail(1);
  if (!buf.p || !times.p || !fail.p) return SL_ERR_DEVICE;
  hipLaunchKernelGGL(k_ub_exchange, dim3(256), dim3(1024), 0, 0, buf.p, mode, rounds, times.p, fail.p);
  if (hipDeviceSynchronize() != hipSuccess) return SL_ERR_DEVICE;
  std::vector<unsigned long long> t(512);
  unsigned f = 0;
  if (hipMemcpy(t.data(), times.p, 512 * 8, hipMemcpyDeviceToHost) != hipSuccess || hipMemcpy(&f, fail.p, 4, hipMemcpyDeviceToHost) != hipSuccess)
    return SL_ERR_DEVICE;
  if (f) return SL_ERR_DEVICE;
  unsigned long long lo = ~0ull, hi = 0;
  for (int w = 0; w < 256; ++w) { if (t[2 * w] && t[2 * w] < lo) lo = t[2 * w]; if (t[2 * w + 1] > hi) hi = t[2 * w + 1]; }
  *us_per_round = (float)((double)(hi - lo) * 0.01 / (double)(rounds - 8));      // the wall clock counts at 100 MHz
  return SL_OK;
}

int sl_ubench_gemv_stream(int mode, int grid, float* tb_per_s) {
  if (mode < 0 || mode > 2 || grid < 1 || grid > 4096 || !tb_per_s) return SL_ERR_ARG;
  const long nrows = 1L << 21;                    // 2 M rows of 1024 + 128 bytes = 2.4 GB
  DevBuf<uint32_t> W((size_t)nrows * 256, 0x35), SB((size_t)nrows * 32, 0x21);
  DevBuf<float> out(16);
  if (!W.p || !SB.p || !out.p) return SL_ERR_DEVICE;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return SL_ERR_DEVICE;
  float ms = 0.0f;
  for (int rep = 0; rep < 2; ++rep) {
    (void)hipEventRecord(e0, 0);
    if (mode == 0) hipLaunchKernelGGL(k_ub_gemv<0>, dim3(grid), dim3(1024), 0, 0, W.p, SB.p, nrows, out.p);
    if (mode == 1) hipLaunchKernelGGL(k_ub_gemv<1>, dim3(grid), dim3(1024), 0, 0, W.p, SB.p, nrows, out.p);
    if (mode == 2) hipLaunchKernelGGL(k_ub_gemv<2>, dim3(grid), dim3(1024), 0, 0, W.p, SB.p, nrows, out.p);
    (void)hipEventRecord(e1, 0);
    if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) { ms = 0.0f; break; }
  }
  (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
  if (ms <= 0.0f) return SL_ERR_DEVICE;
  *tb_per_s = (float)((double)nrows * 1152.0 / (double)ms / 1e9);
  return SL_OK;
}

int sl_ubench_mfma_issue(int valu_steps, int lds_read, int waves_per_simd, float* tflops, float* ns_per_mfma) {
  if (valu_steps < 0 || valu_steps > 8 || waves_per_simd < 1 || waves_per_simd > 2 || !tflops || !ns_per_mfma) return SL_ERR_ARG;
  const int wgs = 256 * waves_per_simd, iters = 4096;
  DevBuf<float> out((size_t)wgs * 256);
  if (!out.p) return SL_ERR_DEVICE;
  auto launch = [&](int n) {
#define UB_CASE(V, L) if (valu_steps == V && (lds_read != 0) == (L != 0)) hipLaunchKernelGGL((k_ub_mfma<V, L>), dim3(wgs), dim3(256), 0, 0, out.p, n, 1u)
    UB_CASE(0, 0); UB_CASE(1, 0); UB_CASE(2, 0); UB_CASE(3, 0); UB_CASE(4, 0); UB_CASE(5, 0); UB_CASE(6, 0); UB_CASE(7, 0); UB_CASE(8, 0);
    UB_CASE(0, 1); UB_CASE(1, 1); UB_CASE(2, 1); UB_CASE(3, 1); UB_CASE(4, 1); UB_CASE(5, 1); UB_CASE(6, 1); UB_CASE(7, 1); UB_CASE(8, 1);
#undef UB_CASE
  };
  launch(16);
  if (hipDeviceSynchronize() != hipSuccess) return SL_ERR_DEVICE;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return SL_ERR_DEVICE;
  (void)hipEventRecord(e0, 0);
  launch(iters);
  (void)hipEventRecord(e1, 0);
  float ms = 0.0f;
  const bool ok = hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&ms, e0, e1) == hipSuccess && ms > 0.0f;
  (void)hipEventDestroy(e0); (void)hipEventDestroy(e1);
  if (!ok) return SL_ERR_DEVICE;
  const double mfmas = (double)wgs * 4.0 * iters * 4.0;             // workgroups x waves x iterations x tiles
  *tflops = (float)(mfmas * 32768.0 / ((double)ms * 1e-3) / 1e12);  // 32 x 32 x 16 multiply-adds = 32768 flop
  *ns_per_mfma = (float)((double)ms * 1e6 / ((double)iters * 4.0 * waves_per_simd));   // per SIMD: wall time per matrix instruction issued
  return SL_OK;
}

}  // extern "C"
