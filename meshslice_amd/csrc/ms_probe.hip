// libmeshslice_hip.so — measurement aids (declarations: include/meshslice_hip.h): the rate of a bare MFMA stream on
// this device, the rate of a bare L2 -> LDS load stream, and the output-stationary 16x16x32 kernel with parts of its K
// loop left out.  None of this is on the path of a product.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstring>
#include <type_traits>

#include "ms_common.hip.inc"

#include "ms_gemm_bf16.hip.inc"
#include "ms_gemm_bf16_x16.hip.inc"

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

// ---------------------------------------------------------------------------------------------
// The output-stationary 16x16x32 kernel (bf16 in, bf16 out) with parts of its K loop left out
// ---------------------------------------------------------------------------------------------
#define MS_INSTANTIATE_SKIP(SKIP) template __global__ void msk::gemm_bf16_x16_kernel<true, false, true, false, SKIP>(const msk::GemmArgs);
MS_INSTANTIATE_SKIP(1) MS_INSTANTIATE_SKIP(2) MS_INSTANTIATE_SKIP(3) MS_INSTANTIATE_SKIP(4) MS_INSTANTIATE_SKIP(8) MS_INSTANTIATE_SKIP(16)
MS_INSTANTIATE_SKIP(24)
#undef MS_INSTANTIATE_SKIP

MS_API int ms_probe_os_parts(int skip, const void *const *A_slices, const void *const *B_slices, int S, int m, int n, int k_slice,
                             int lda, int ldb, void *C, int ldc, int warmup, int reps, float *ms_out, void *stream) {
  using msi::fail;
  const char *fn = "ms_probe_os_parts";
  if (!A_slices || !B_slices || !C || !ms_out) return fail(MS_ERR_ARG, "%s: null pointer", fn);
  if (S < 1 || S > MS_MAX_SLICES || m <= 0 || n <= 0 || k_slice <= 0) return fail(MS_ERR_ARG, "%s: bad extents (S=%d m=%d n=%d k=%d)", fn, S, m, n, k_slice);
  if (k_slice % 8 || n % 8 || lda % 8 || ldb % 8 || ldc % 8 || lda < k_slice || ldb < n || ldc < n)
    return fail(MS_ERR_ARG, "%s: extents and leading dimensions must be multiples of 8 and cover their rows", fn);
  if ((long long)m * lda * 2 > 0x7FFFFFFFLL || (long long)k_slice * ldb * 2 > 0x7FFFFFFFLL) return fail(MS_ERR_UNSUPPORTED, "%s: an operand slice spans 2 GiB or more", fn);
  if (warmup < 0 || reps < 1) return fail(MS_ERR_ARG, "%s: need warmup >= 0 and reps >= 1", fn);
  for (int s = 0; s < S; s++)
    if (!A_slices[s] || !B_slices[s] || ((reinterpret_cast<uintptr_t>(A_slices[s]) | reinterpret_cast<uintptr_t>(B_slices[s])) & 15))
      return fail(MS_ERR_ARG, "%s: slice pointer %d null or not 16-byte aligned", fn, s);
  if (reinterpret_cast<uintptr_t>(C) & 15) return fail(MS_ERR_ARG, "%s: C not 16-byte aligned", fn);
  int dev = 0;
  MS_HIP(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  MS_HIP(hipGetDeviceProperties(&prop, dev));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return fail(MS_ERR_UNSUPPORTED, "%s: needs a gfx950 device", fn);
  msk::GemmArgs g;
  memset(&g, 0, sizeof(g));
  for (int s = 0; s < S; s++) { g.a[s] = A_slices[s]; g.b[s] = B_slices[s]; }
  g.c[0] = C;
  g.nchunks = 1; g.nkslices = S;
  g.M = m; g.N = n; g.K = k_slice; g.lda = lda; g.ldb = ldb; g.ldc = ldc;
  g.tiles_m = (m + 255) / 256; g.tiles_n = (n + 383) / 384;
  g.total_tiles = g.tiles_m * g.tiles_n;
  g.group_m = 8; g.splits = 1;
  const dim3 gd(msi::balanced_grid(g.total_tiles, prop.multiProcessorCount)), bd(256);
  hipStream_t st = (hipStream_t)stream;
  auto launch = [&]() -> bool {
    switch (skip) {
      case 0: msk::gemm_bf16_x16_kernel<true, false, true, false, 0><<<gd, bd, 0, st>>>(g); return true;
      case 1: msk::gemm_bf16_x16_kernel<true, false, true, false, 1><<<gd, bd, 0, st>>>(g); return true;
      case 2: msk::gemm_bf16_x16_kernel<true, false, true, false, 2><<<gd, bd, 0, st>>>(g); return true;
      case 3: msk::gemm_bf16_x16_kernel<true, false, true, false, 3><<<gd, bd, 0, st>>>(g); return true;
      case 4: msk::gemm_bf16_x16_kernel<true, false, true, false, 4><<<gd, bd, 0, st>>>(g); return true;
      case 8: msk::gemm_bf16_x16_kernel<true, false, true, false, 8><<<gd, bd, 0, st>>>(g); return true;
      case 16: msk::gemm_bf16_x16_kernel<true, false, true, false, 16><<<gd, bd, 0, st>>>(g); return true;
      case 24: msk::gemm_bf16_x16_kernel<true, false, true, false, 24><<<gd, bd, 0, st>>>(g); return true;
      default: return false;
    }
  };
  if (!launch()) return fail(MS_ERR_ARG, "%s: no kernel was built for skip = %d (0, 1, 2, 3, 4, 8, 16, 24)", fn, skip);
  for (int i = 1; i < warmup; i++) launch();
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
  return MS_OK;
}

// ---------------------------------------------------------------------------------------------
// A bare L2 -> LDS stream: four waves per compute unit, twenty 128-bit direct-to-LDS loads per wave and step (80 KB per
// workgroup and step, the stage size of the 256x384x64 kernels), nothing else in the loop.  The workgroups that share an
// XCD (blockIdx % 8) walk the same region of `region_steps` x 80 KB round and round, so with a region inside the 4 MB
// of an L2 every load after the first round hits there.  A wave waits until at most `IN_FLIGHT` of its loads are
// outstanding before it issues the next step's.
// ---------------------------------------------------------------------------------------------
namespace msk {
template <int IN_FLIGHT>
__global__ __launch_bounds__(256) void l2_lds_stream_kernel(const char *base, int steps, int region_steps, float *sink) {
  constexpr int NW = 4, NI = 20;
  __shared__ __attribute__((aligned(1024))) char lds[NW * NI * 1024];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const char *p0 = base + (size_t)(blockIdx.x % 8) * region_steps * (NW * NI * 1024);
  unsigned voff[NI];
#pragma unroll
  for (int i = 0; i < NI; i++) voff[i] = (unsigned)((i * NW + wave) * 1024 + lane * 16);
  const int wb = (int)(unsigned)(size_t)MS_LDS(lds) + wave * 1024;
  int t2 = 0;
  for (int t = 0; t < steps; t++) {
    const unsigned long long p = (unsigned long long)(p0 + (size_t)t2 * (NW * NI * 1024));
    if (++t2 == region_steps) t2 = 0;
    const i32x4 rs = {(int)(unsigned)p, (int)(unsigned)(p >> 32), NW * NI * 1024, 0x00020000};
    static_for<0, NI>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      dma16<i * NW * 1024, 0>(voff[i], rs, wb);
    });
    wait_vmcnt<IN_FLIGHT>();
  }
  wait_vmcnt<0>();
  __syncthreads();
  const float x = *(const float *)(lds + lane * 4);
  if (x == 12345.678f) sink[0] = x;      // keeps the loads alive; never true for the buffer the host fills
}
}  // namespace msk

MS_API int ms_probe_l2_lds_stream(const void *buffer, size_t buffer_bytes, int region_steps, int in_flight_steps, int steps,
                                  int warmup, int reps, float *sink, float *ms_out, double *bytes_per_launch, void *stream) {
  using msi::fail;
  const char *fn = "ms_probe_l2_lds_stream";
  constexpr size_t STEP_BYTES = 4 * 20 * 1024;
  if (!buffer || !sink || !ms_out || !bytes_per_launch) return fail(MS_ERR_ARG, "%s: null pointer", fn);
  if (reinterpret_cast<uintptr_t>(buffer) & 255) return fail(MS_ERR_ARG, "%s: buffer must be 256-byte aligned", fn);
  if (region_steps < 1 || steps < 1 || warmup < 0 || reps < 1) return fail(MS_ERR_ARG, "%s: need region_steps, steps, reps >= 1 and warmup >= 0", fn);
  if (in_flight_steps < 1 || in_flight_steps > 3) return fail(MS_ERR_ARG, "%s: in_flight_steps must be 1, 2 or 3", fn);
  if (buffer_bytes < 8 * (size_t)region_steps * STEP_BYTES) return fail(MS_ERR_ARG, "%s: the buffer must hold 8 regions of %d x %zu bytes", fn, region_steps, STEP_BYTES);
  int dev = 0;
  MS_HIP(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  MS_HIP(hipGetDeviceProperties(&prop, dev));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) return fail(MS_ERR_UNSUPPORTED, "%s: needs a gfx950 device", fn);
  const int cus = prop.multiProcessorCount;
  hipStream_t st = (hipStream_t)stream;
  const char *base = static_cast<const char *>(buffer);
  auto launch = [&]() {
    const dim3 gd(cus), bd(256);
    if (in_flight_steps == 1) msk::l2_lds_stream_kernel<0><<<gd, bd, 0, st>>>(base, steps, region_steps, sink);
    else if (in_flight_steps == 2) msk::l2_lds_stream_kernel<20><<<gd, bd, 0, st>>>(base, steps, region_steps, sink);
    else msk::l2_lds_stream_kernel<40><<<gd, bd, 0, st>>>(base, steps, region_steps, sink);
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
  *bytes_per_launch = (double)cus * steps * STEP_BYTES;
  return MS_OK;
}
