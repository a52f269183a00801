// Synthetic checkpoint generator: seeded N(0, sigma) tensors and their MLX-affine 4-bit
// quantisation (group 64), produced directly in HBM.  Element i of a tensor is a pure function of
// (seed, i); one thread owns one quantisation group.
#include "sl_device.cuh"
#include "../../include/seedless_hip.h"

using namespace sl;

__global__ __launch_bounds__(256) void k_synth_q4(uint32_t* __restrict__ w, uint16_t* __restrict__ sc,
                                                  uint16_t* __restrict__ bi, int64_t ngroups, uint64_t seed,
                                                  float sigma) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= ngroups) return;
  float v[64];
  float mn = __int_as_float(0x7f800000), mx = -mn;
#pragma unroll
  for (int i = 0; i < 64; ++i) {
    v[i] = sigma * normal01(seed, (uint64_t)g * 64ull + (uint64_t)i);
    mn = fminf(mn, v[i]);
    mx = fmaxf(mx, v[i]);
  }
  const bool mask = fabsf(mn) > fabsf(mx);
  float scale = fmaxf((mx - mn) / 15.0f, 1e-7f);
  scale = mask ? scale : -scale;
  const float edge = mask ? mn : mx;
  const float q0 = rintf(edge / scale);
  float bias = 0.0f;
  if (q0 != 0.0f) { scale = edge / q0; bias = edge; }
  sc[g] = f2h(scale);
  bi[g] = f2h(bias);
#pragma unroll
  for (int wd = 0; wd < 8; ++wd) {
    uint32_t pack = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      float q = rintf((v[wd * 8 + i] - bias) / scale);
      q = fminf(fmaxf(q, 0.0f), 15.0f);
      pack |= (uint32_t)q << (4 * i);
    }
    w[g * 8 + wd] = pack;
  }
}

__global__ __launch_bounds__(256) void k_synth_f16(uint16_t* __restrict__ dst, int64_t n, uint64_t seed, float mean,
                                                   float sigma) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = f2h(mean + sigma * normal01(seed, (uint64_t)i));
}
__global__ __launch_bounds__(256) void k_synth_f32(float* __restrict__ dst, int64_t n, uint64_t seed, float mean,
                                                   float sigma) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = mean + sigma * normal01(seed, (uint64_t)i);
}

// Applies one scalar routine of sl_device.cuh to an array (self-test of the device arithmetic).
__global__ __launch_bounds__(256) void k_math(int op, const float* __restrict__ x, float* __restrict__ y, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float v = x[i];
  float r;
  switch (op) {
    case 0: r = exp_c(v); break;
    case 1: r = log_c(v); break;
    case 2: r = sigmoid32(v); break;
    case 3: r = sigmoid16(v); break;
    case 4: r = softplus_c(v); break;
    case 5: r = f16r(v); break;
    case 6: r = 1.0f / sqrtf(v / 128.0f + 1e-6f); break;
    case 7: r = f16r(v * sigmoid32(v)); break;
    default: r = ppnd7(v); break;
  }
  y[i] = r;
}

static int launch_status() { return hipGetLastError() == hipSuccess ? SL_OK : SL_ERR_DEVICE; }

extern "C" int sl_synth_q4(uint32_t* w, uint16_t* s, uint16_t* b, int64_t n, int32_t k, uint64_t seed, float sigma,
                           void* stream) {
  if (!w || !s || !b || n < 1 || k < 64 || (k % 64) != 0) return SL_ERR_ARG;
  const int64_t groups = n * (int64_t)(k / 64);
  const int64_t blocks = (groups + 255) / 256;
  if (blocks > 0x7fffffffLL) return SL_ERR_ARG;
  hipLaunchKernelGGL(k_synth_q4, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, w, s, b, groups, seed, sigma);
  return launch_status();
}
extern "C" int sl_synth_f16(uint16_t* dst, int64_t count, uint64_t seed, float mean, float sigma, void* stream) {
  if (!dst || count < 1) return SL_ERR_ARG;
  hipLaunchKernelGGL(k_synth_f16, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, (hipStream_t)stream, dst, count,
                     seed, mean, sigma);
  return launch_status();
}
extern "C" int sl_synth_f32(float* dst, int64_t count, uint64_t seed, float mean, float sigma, void* stream) {
  if (!dst || count < 1) return SL_ERR_ARG;
  hipLaunchKernelGGL(k_synth_f32, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, (hipStream_t)stream, dst, count,
                     seed, mean, sigma);
  return launch_status();
}

extern "C" int sl_selftest_math(int op, const float* x_host, float* y_host, int64_t n) {
  if (!x_host || !y_host || n < 1) return SL_ERR_ARG;
  float *dx = nullptr, *dy = nullptr;
  if (hipMalloc((void**)&dx, n * 4) != hipSuccess) return SL_ERR_DEVICE;
  if (hipMalloc((void**)&dy, n * 4) != hipSuccess) { (void)hipFree(dx); return SL_ERR_DEVICE; }
  int rc = SL_ERR_DEVICE;
  if (hipMemcpy(dx, x_host, n * 4, hipMemcpyHostToDevice) == hipSuccess) {
    hipLaunchKernelGGL(k_math, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, nullptr, op, dx, dy, n);
    if (hipGetLastError() == hipSuccess && hipMemcpy(y_host, dy, n * 4, hipMemcpyDeviceToHost) == hipSuccess) rc = SL_OK;
  }
  (void)hipFree(dx); (void)hipFree(dy);
  return rc;
}

