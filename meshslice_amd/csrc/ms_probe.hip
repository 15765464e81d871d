// libmeshslice_hip.so — measurement aid: the rate of a bare MFMA stream on this device (declaration:
// include/meshslice_hip.h).
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstring>

#include "ms_common.hip.inc"

namespace msk {

typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));

constexpr int PROBE_MFMA_PER_ITER = 64;  // 4 k-chunks x (4 x 4) accumulator tiles

// One wave per SIMD: 16 accumulator tiles of 32x32 (256 registers), 4 + 4 operand fragments held in
// registers for the whole run, nothing but v_mfma_f32_32x32x16_bf16 in the loop (each accumulator is
// touched every 16th instruction, far beyond the dependent-issue distance).
__global__ __launch_bounds__(256) void mfma_stream_kernel(const probe_bf16x8 *ops, float *sink, int iters) {
  const int lane = threadIdx.x & 63;
  probe_bf16x8 a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    a[i] = ops[i * 64 + lane];
    b[i] = ops[(4 + i) * 64 + lane];
  }
  probe_f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int kk = 0; kk < 4; kk++)
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[j], a[i], acc[i][j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) s += acc[i][j][v];
  sink[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace msk

MS_API int ms_probe_mfma_stream(const void *operands, float *sink, int iters, int warmup, int reps,
                                float *ms_out, double *flops_per_launch, void *stream) {
  using msi::fail;
  const char *fn = "ms_probe_mfma_stream";
  if (!operands || !sink || !ms_out || !flops_per_launch) return fail(MS_ERR_ARG, "%s: null pointer", fn);
  if (reinterpret_cast<uintptr_t>(operands) & 15) return fail(MS_ERR_ARG, "%s: operands must be 16-byte aligned", fn);
  if (iters < 1 || warmup < 0 || reps < 1) return fail(MS_ERR_ARG, "%s: need iters >= 1, warmup >= 0, reps >= 1", fn);
  int dev = 0;
  MS_HIP(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  MS_HIP(hipGetDeviceProperties(&prop, dev));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return fail(MS_ERR_UNSUPPORTED, "%s: needs a gfx950 device", fn);
  const int cus = prop.multiProcessorCount;
  hipStream_t st = (hipStream_t)stream;
  auto launch = [&]() {
    hipLaunchKernelGGL(msk::mfma_stream_kernel, dim3(cus), dim3(256), 0, st,
                       reinterpret_cast<const msk::probe_bf16x8 *>(operands), sink, iters);
  };
  for (int i = 0; i < warmup; i++) launch();
  MS_HIP(hipGetLastError());
  hipEvent_t e0, e1;
  MS_HIP(hipEventCreate(&e0));
  MS_HIP(hipEventCreate(&e1));
  (void)hipEventRecord(e0, st);
  for (int i = 0; i < reps; i++) launch();
  (void)hipEventRecord(e1, st);
  int rc = MS_OK;
  float ms = 0.f;
  if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) rc = fail(MS_ERR_HIP, "%s: event timing failed", fn);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc != MS_OK) return rc;
  MS_HIP(hipGetLastError());
  *ms_out = ms / reps;
  // 4 waves per CU, each MFMA = 32 x 32 x 16 multiply-adds
  *flops_per_launch = (double)cus * 4.0 * iters * msk::PROBE_MFMA_PER_ITER * (2.0 * 32 * 32 * 16);
  return MS_OK;
}
