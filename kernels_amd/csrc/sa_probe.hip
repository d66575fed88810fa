// Measurement support for bench.py (not part of the operator): what the matrix pipe of this GPU
// sustains on a bare stream of v_mfma_f32_32x32x16_bf16, and what a plain copy moves through HBM.
// Built into its own small library (libsa_probe.so) so that the operator's C ABI stays clean.
//
//   sa_probe_mfma_bf16(random, iters, waves_per_simd, &tflops)
//       every wave issues 8 independent accumulator chains; operands are either one constant
//       fragment (no switching activity in the multipliers) or 8 fragments of N(0,1)-like random
//       bf16 values rotated between the MFMAs (the data-dependent power draw of real inputs).
//   sa_probe_copy(bytes, iters, &gbs)
//       device-to-device copy of `bytes` with 16-byte accesses.
// Both time their own launches with HIP events on the null stream and return 0 or a hipError_t.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {

__device__ __forceinline__ uint32_t lcg(uint32_t& s) { return s = s * 1664525u + 1013904223u; }
// roughly N(0,1): sum of four uniforms, centred and scaled
__device__ __forceinline__ float gaussish(uint32_t& s) {
  float a = 0.0f;
  for (int i = 0; i < 4; ++i) a += (float)(lcg(s) >> 8) * (1.0f / 16777216.0f);
  return (a - 2.0f) * 1.7320508f;
}

template <bool RANDOM>
__global__ __launch_bounds__(256) void mfma_kernel(float* out, int iters) {
  uint32_t seed = 1234567u + threadIdx.x * 7919u + blockIdx.x * 104729u;
  bf16x8 a[8], b[8];
#pragma unroll
  for (int g = 0; g < 8; ++g)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      a[g][e] = (__bf16)(RANDOM ? gaussish(seed) : 1.0f);
      b[g][e] = (__bf16)(RANDOM ? gaussish(seed) : 0.5f);
    }
  f32x16 c[8];
#pragma unroll
  for (int g = 0; g < 8; ++g)
#pragma unroll
    for (int i = 0; i < 16; ++i) c[g][i] = 0.0f;
  // 64 MFMAs per iteration: chain g takes the second operand (g + r) % 8 in round r
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 8; ++r)
#pragma unroll
      for (int g = 0; g < 8; ++g)
        c[g] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[RANDOM ? g : 0], b[RANDOM ? (g + r) & 7 : 0], c[g], 0, 0, 0);
  }
  float s = 0.0f;
#pragma unroll
  for (int g = 0; g < 8; ++g)
#pragma unroll
    for (int i = 0; i < 16; ++i) s += c[g][i];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

__global__ __launch_bounds__(256) void copy_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, size_t n) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

}  // namespace

extern "C" {

int sa_probe_mfma_bf16(int random, int iters, int waves_per_simd, double* tflops) {
  if (!tflops || iters < 1 || waves_per_simd < 1 || waves_per_simd > 2) return (int)hipErrorInvalidValue;
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
  if (hipError_t e = hipGetDeviceProperties(&prop, dev); e != hipSuccess) return (int)e;
  const int blocks = prop.multiProcessorCount * waves_per_simd;   // 4 waves per block: one per SIMD
  float* out = nullptr;
  if (hipError_t e = hipMalloc(&out, (size_t)blocks * 256 * sizeof(float)); e != hipSuccess) return (int)e;
  hipEvent_t e0, e1;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  auto launch = [&](int n) {
    if (random) hipLaunchKernelGGL(mfma_kernel<true>, dim3(blocks), dim3(256), 0, nullptr, out, n);
    else hipLaunchKernelGGL(mfma_kernel<false>, dim3(blocks), dim3(256), 0, nullptr, out, n);
  };
  launch(16);
  (void)hipEventRecord(e0, nullptr);
  launch(iters);
  (void)hipEventRecord(e1, nullptr);
  hipError_t err = hipEventSynchronize(e1);
  float ms = 0.0f;
  if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
  if (err == hipSuccess) err = hipGetLastError();
  // per MFMA: 32 x 32 x 16 multiply-adds
  if (err == hipSuccess) *tflops = (double)blocks * 4.0 * iters * 64.0 * 32768.0 / ((double)ms * 1e-3) / 1e12;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipFree(out);
  return (int)err;
}

int sa_probe_copy(size_t bytes, int iters, double* gbs) {
  if (!gbs || iters < 1 || bytes < 16 || bytes % 16) return (int)hipErrorInvalidValue;
  void *src = nullptr, *dst = nullptr;
  if (hipError_t e = hipMalloc(&src, bytes); e != hipSuccess) return (int)e;
  if (hipError_t e = hipMalloc(&dst, bytes); e != hipSuccess) {
    (void)hipFree(src);
    return (int)e;
  }
  (void)hipMemsetAsync(src, 1, bytes, nullptr);
  hipEvent_t e0, e1;
  (void)hipEventCreate(&e0);
  (void)hipEventCreate(&e1);
  const size_t n = bytes / 16;
  auto launch = [&] {
    hipLaunchKernelGGL(copy_kernel, dim3(8192), dim3(256), 0, nullptr, (const u32x4*)src, (u32x4*)dst, n);
  };
  launch();
  (void)hipEventRecord(e0, nullptr);
  for (int i = 0; i < iters; ++i) launch();
  (void)hipEventRecord(e1, nullptr);
  hipError_t err = hipEventSynchronize(e1);
  float ms = 0.0f;
  if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
  if (err == hipSuccess) err = hipGetLastError();
  if (err == hipSuccess) *gbs = 2.0 * (double)bytes * iters / ((double)ms * 1e-3) / 1e9;   // read + written
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  (void)hipFree(src);
  (void)hipFree(dst);
  return (int)err;
}

}  // extern "C"
