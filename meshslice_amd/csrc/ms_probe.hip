// libmeshslice_hip.so — measurement aid: the rate of a bare MFMA stream on this device (declarations:
// include/meshslice_hip.h).
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstring>
#include <type_traits>

#include "ms_common.hip.inc"

namespace msk {

typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));
typedef float probe_f32x4 __attribute__((ext_vector_type(4)));

constexpr int PROBE_MFMA_PER_ITER = 64;   // MFMA instructions per wave and loop trip, every kernel below

// Nothing but MFMAs in the loop: operand fragments and accumulators stay in registers for the whole run, and
// each accumulator is touched once per TA x TB instructions, far beyond the dependent-issue distance.
//   MF = 32: v_mfma_f32_32x32x16_bf16 (8 passes), accumulator tile = 16 registers
//   MF = 16: v_mfma_f32_16x16x32_bf16 (4 passes), accumulator tile =  4 registers
// WPS waves per SIMD (workgroup = 4 x WPS waves); the accumulators of a wave fill 256 / WPS registers.
template <int MF, int WPS>
__global__ __launch_bounds__(256 * WPS) void mfma_stream_kernel(const probe_bf16x8 *ops, float *sink, int iters) {
  constexpr int TILES = 256 / WPS / (MF == 32 ? 16 : 4);         // accumulator tiles per wave
  constexpr int TA = MF == 32 ? 4 : 8, TB = TILES / TA;          // 4 x 4 | 4 x 2 | 8 x 8 | 8 x 4
  static_assert(PROBE_MFMA_PER_ITER % TILES == 0, "a loop trip is a whole number of sweeps over the tiles");
  typedef typename std::conditional<MF == 32, probe_f32x16, probe_f32x4>::type Acc;
  const int lane = threadIdx.x & 63;
  probe_bf16x8 a[TA], b[TB];
#pragma unroll
  for (int i = 0; i < TA; i++) a[i] = ops[i * 64 + lane];
#pragma unroll
  for (int j = 0; j < TB; j++) b[j] = ops[(TA + j) * 64 + lane];
  Acc acc[TA][TB];
#pragma unroll
  for (int i = 0; i < TA; i++)
#pragma unroll
    for (int j = 0; j < TB; j++) acc[i][j] = Acc(0.f);
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int kk = 0; kk < PROBE_MFMA_PER_ITER / TILES; kk++)
#pragma unroll
      for (int i = 0; i < TA; i++)
#pragma unroll
        for (int j = 0; j < TB; j++) {
          if constexpr (MF == 32) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[j], a[i], acc[i][j], 0, 0, 0);
          else acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[j], a[i], acc[i][j], 0, 0, 0);
        }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < TA; i++)
#pragma unroll
    for (int j = 0; j < TB; j++)
#pragma unroll
      for (int v = 0; v < (MF == 32 ? 16 : 4); v++) s += acc[i][j][v];
  sink[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

}  // namespace msk

MS_API int ms_probe_mfma_stream_ex(const void *operands, float *sink, int shape, int waves_per_simd, int iters,
                                   int warmup, int reps, float *ms_out, double *flops_per_launch, void *stream) {
  using msi::fail;
  const char *fn = "ms_probe_mfma_stream_ex";
  if (!operands || !sink || !ms_out || !flops_per_launch) return fail(MS_ERR_ARG, "%s: null pointer", fn);
  if (reinterpret_cast<uintptr_t>(operands) & 15) return fail(MS_ERR_ARG, "%s: operands must be 16-byte aligned", fn);
  if (iters < 1 || warmup < 0 || reps < 1) return fail(MS_ERR_ARG, "%s: need iters >= 1, warmup >= 0, reps >= 1", fn);
  if (shape != MS_MFMA_32X32X16 && shape != MS_MFMA_16X16X32) return fail(MS_ERR_ARG, "%s: unknown instruction shape %d", fn, shape);
  if (waves_per_simd != 1 && waves_per_simd != 2) return fail(MS_ERR_ARG, "%s: waves_per_simd must be 1 or 2, got %d", fn, waves_per_simd);
  int dev = 0;
  MS_HIP(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  MS_HIP(hipGetDeviceProperties(&prop, dev));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return fail(MS_ERR_UNSUPPORTED, "%s: needs a gfx950 device", fn);
  const int cus = prop.multiProcessorCount;
  hipStream_t st = (hipStream_t)stream;
  const msk::probe_bf16x8 *ops = reinterpret_cast<const msk::probe_bf16x8 *>(operands);
  auto launch = [&]() {
    const dim3 gd(cus), bd(256 * waves_per_simd);
    if (shape == MS_MFMA_32X32X16) {
      if (waves_per_simd == 1) hipLaunchKernelGGL((msk::mfma_stream_kernel<32, 1>), gd, bd, 0, st, ops, sink, iters);
      else hipLaunchKernelGGL((msk::mfma_stream_kernel<32, 2>), gd, bd, 0, st, ops, sink, iters);
    } else {
      if (waves_per_simd == 1) hipLaunchKernelGGL((msk::mfma_stream_kernel<16, 1>), gd, bd, 0, st, ops, sink, iters);
      else hipLaunchKernelGGL((msk::mfma_stream_kernel<16, 2>), gd, bd, 0, st, ops, sink, iters);
    }
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
  // multiply-adds of one instruction: 16384 (32x32x16) or 8192 (16x16x32)
  const double macs = shape == MS_MFMA_32X32X16 ? 32.0 * 32 * 16 : 16.0 * 16 * 32;
  *flops_per_launch = (double)cus * 4.0 * waves_per_simd * iters * msk::PROBE_MFMA_PER_ITER * 2.0 * macs;
  return MS_OK;
}

MS_API int ms_probe_mfma_stream(const void *operands, float *sink, int iters, int warmup, int reps,
                                float *ms_out, double *flops_per_launch, void *stream) {
  return ms_probe_mfma_stream_ex(operands, sink, MS_MFMA_32X32X16, 1, iters, warmup, reps, ms_out, flops_per_launch, stream);
}
