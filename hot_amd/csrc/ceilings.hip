// Achievable ceilings of the box the library runs on, measured with two plain kernels: a device copy
// (HBM read + write) and a loop of independent INT8 MFMAs.  bench.py quotes them beside the published
// peaks (8 TB/s, 5.0 POP/s) that the roofline fractions are priced against.  The reference has no
// counterpart; this is a measurement hook like hot_linear_backward_kernels.
#include "hot_device.h"
#include "hot_host.h"

namespace hot {

__global__ void __launch_bounds__(256) ceiling_copy_kernel(const v4i* __restrict__ src, v4i* __restrict__ dst, int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// 16 independent 32x32x32 INT8 MFMAs per iteration and wave (256 accumulator registers), one wave per SIMD
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
ceiling_mfma_kernel(int iters, int32_t* sink) {
  v16i acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0;
  v4i a = {(int)threadIdx.x, 1, 2, 3}, b = {4, 5, 6, (int)blockIdx.x};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[i], 0, 0, 0);
  }
  int32_t s = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += acc[i][0];
  if (s == 0x7fffffff) sink[0] = s;   // keeps the loop alive; never true for these operands
}

}  // namespace hot

using namespace hot;

extern "C" int hot_measure_ceilings(void* scratch, size_t scratch_bytes, float* copy_gbs, float* mfma_tops, void* hip_stream) {
  const char* who = "hot_measure_ceilings";
  if (!scratch || !copy_gbs || !mfma_tops) return fail(HOT_ERR_INVALID, "%s: null pointer", who);
  if (scratch_bytes < (size_t)(64u << 20) || ((uintptr_t)scratch & 15)) return fail(HOT_ERR_INVALID, "%s: a 16-byte aligned scratch buffer of at least 64 MiB", who);
  hipStream_t st = (hipStream_t)hip_stream;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  int rc = check_hip(hipEventCreate(&e0), "hipEventCreate");
  if (!rc) rc = check_hip(hipEventCreate(&e1), "hipEventCreate");
  float ms = 0.f;
  if (!rc) {
    const size_t half = (scratch_bytes / 2) & ~(size_t)15;
    const int64_t n16 = (int64_t)(half / 16);
    const v4i* src = (const v4i*)scratch;
    v4i* dst = (v4i*)((uint8_t*)scratch + half);
    const int reps = 10;
    hipLaunchKernelGGL(ceiling_copy_kernel, dim3(256 * 16), dim3(256), 0, st, src, dst, n16);
    (void)hipEventRecord(e0, st);
    for (int r = 0; r < reps; ++r) hipLaunchKernelGGL(ceiling_copy_kernel, dim3(256 * 16), dim3(256), 0, st, src, dst, n16);
    (void)hipEventRecord(e1, st);
    rc = check_hip(hipEventSynchronize(e1), "hipEventSynchronize");
    if (!rc) rc = check_hip(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
    if (!rc) *copy_gbs = (float)(2.0 * (double)half * reps / ((double)ms * 1e-3) / 1e9);   // bytes read + bytes written
  }
  if (!rc) {
    const int iters = 4000, wgs = 512;
    hipLaunchKernelGGL(ceiling_mfma_kernel, dim3(wgs), dim3(256), 0, st, 100, (int32_t*)scratch);
    (void)hipEventRecord(e0, st);
    hipLaunchKernelGGL(ceiling_mfma_kernel, dim3(wgs), dim3(256), 0, st, iters, (int32_t*)scratch);
    (void)hipEventRecord(e1, st);
    rc = check_hip(hipEventSynchronize(e1), "hipEventSynchronize");
    if (!rc) rc = check_hip(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
    if (!rc) *mfma_tops = (float)((double)wgs * 4 * iters * 16 * 65536.0 / ((double)ms * 1e-3) / 1e12);
  }
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  return rc ? rc : check_launch(who);
}
