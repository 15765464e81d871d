// libmeshslice_hip.so — C ABI over the gfx950 GEMM kernels (declarations: include/meshslice_hip.h).
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "ms_common.hip.inc"

#include "ms_gemm_bf16.hip.inc"
#include "ms_gemm_bf16_big.hip.inc"
#include "ms_gemm_bf16_x16.hip.inc"
#include "ms_gemm_f32.hip.inc"

// Every kernel variant is instantiated explicitly: with implicit instantiation alone the host
// compiler leaves some of the launch stubs undefined.
#define MS_INSTANTIATE_RING(BM, BN, BK, NS, WGM, WGN)                                                                         \
  template __global__ void msk::gemm_bf16_ring_kernel<BM, BN, BK, NS, WGM, WGN, true, false, true, false>(const msk::GemmArgs);   \
  template __global__ void msk::gemm_bf16_ring_kernel<BM, BN, BK, NS, WGM, WGN, true, false, false, false>(const msk::GemmArgs);  \
  template __global__ void msk::gemm_bf16_ring_kernel<BM, BN, BK, NS, WGM, WGN, true, false, true, true>(const msk::GemmArgs);    \
  template __global__ void msk::gemm_bf16_ring_kernel<BM, BN, BK, NS, WGM, WGN, true, false, false, true>(const msk::GemmArgs);   \
  template __global__ void msk::gemm_bf16_ring_kernel<BM, BN, BK, NS, WGM, WGN, true, true, false, false>(const msk::GemmArgs);   \
  template __global__ void msk::gemm_bf16_ring_kernel<BM, BN, BK, NS, WGM, WGN, true, true, true, false>(const msk::GemmArgs);    \
  template __global__ void msk::gemm_bf16_ring_kernel<BM, BN, BK, NS, WGM, WGN, false, false, false, false>(const msk::GemmArgs); \
  template __global__ void msk::gemm_bf16_ring_kernel<BM, BN, BK, NS, WGM, WGN, false, false, true, false>(const msk::GemmArgs);
MS_INSTANTIATE_RING(256, 256, 64, 2, 2, 2)
MS_INSTANTIATE_RING(256, 256, 32, 4, 2, 4)
MS_INSTANTIATE_RING(128, 128, 64, 2, 2, 2)
MS_INSTANTIATE_RING(256, 256, 32, 4, 2, 2)
MS_INSTANTIATE_RING(256, 192, 32, 4, 2, 2)
MS_INSTANTIATE_RING(192, 256, 32, 4, 2, 2)
MS_INSTANTIATE_RING(256, 256, 64, 2, 2, 4)
MS_INSTANTIATE_RING(256, 192, 64, 2, 2, 2)
MS_INSTANTIATE_RING(192, 256, 64, 2, 2, 2)
MS_INSTANTIATE_RING(128, 128, 64, 3, 2, 2)
#undef MS_INSTANTIATE_RING
#define MS_INSTANTIATE_BIG(TM, TN)                                                                             \
  template __global__ void msk::gemm_bf16_big_kernel<TM, TN, true, false, true, false>(const msk::GemmArgs);   \
  template __global__ void msk::gemm_bf16_big_kernel<TM, TN, true, false, false, false>(const msk::GemmArgs);  \
  template __global__ void msk::gemm_bf16_big_kernel<TM, TN, true, false, true, true>(const msk::GemmArgs);    \
  template __global__ void msk::gemm_bf16_big_kernel<TM, TN, true, false, false, true>(const msk::GemmArgs);   \
  template __global__ void msk::gemm_bf16_big_kernel<TM, TN, true, true, false, false>(const msk::GemmArgs);   \
  template __global__ void msk::gemm_bf16_big_kernel<TM, TN, true, true, true, false>(const msk::GemmArgs);    \
  template __global__ void msk::gemm_bf16_big_kernel<TM, TN, false, false, false, false>(const msk::GemmArgs); \
  template __global__ void msk::gemm_bf16_big_kernel<TM, TN, false, false, true, false>(const msk::GemmArgs);
MS_INSTANTIATE_BIG(4, 6)
MS_INSTANTIATE_BIG(6, 3)
#undef MS_INSTANTIATE_BIG
#define MS_INSTANTIATE_X16(BN)                                                                                  \
  template __global__ void msk::gemm_bf16_x16_kernel<true, false, true, false, 0, BN>(const msk::GemmArgs);    \
  template __global__ void msk::gemm_bf16_x16_kernel<true, false, false, false, 0, BN>(const msk::GemmArgs);   \
  template __global__ void msk::gemm_bf16_x16_kernel<true, false, true, true, 0, BN>(const msk::GemmArgs);     \
  template __global__ void msk::gemm_bf16_x16_kernel<true, false, false, true, 0, BN>(const msk::GemmArgs);    \
  template __global__ void msk::gemm_bf16_x16_kernel<true, true, false, false, 0, BN>(const msk::GemmArgs);    \
  template __global__ void msk::gemm_bf16_x16_kernel<true, true, true, false, 0, BN>(const msk::GemmArgs);     \
  template __global__ void msk::gemm_bf16_x16_kernel<false, false, false, false, 0, BN>(const msk::GemmArgs);  \
  template __global__ void msk::gemm_bf16_x16_kernel<false, false, true, false, 0, BN>(const msk::GemmArgs);
MS_INSTANTIATE_X16(384)
MS_INSTANTIATE_X16(256)
#undef MS_INSTANTIATE_X16
#define MS_INSTANTIATE_F32(WGM, WGN, TM, TN)                                                                          \
  template __global__ void msk::gemm_f32_tile_kernel<WGM, WGN, TM, TN, true, false, true>(const msk::GemmArgs);     \
  template __global__ void msk::gemm_f32_tile_kernel<WGM, WGN, TM, TN, true, false, false>(const msk::GemmArgs);    \
  template __global__ void msk::gemm_f32_tile_kernel<WGM, WGN, TM, TN, true, true, true>(const msk::GemmArgs);      \
  template __global__ void msk::gemm_f32_tile_kernel<WGM, WGN, TM, TN, true, true, false>(const msk::GemmArgs);     \
  template __global__ void msk::gemm_f32_tile_kernel<WGM, WGN, TM, TN, false, false, true>(const msk::GemmArgs);    \
  template __global__ void msk::gemm_f32_tile_kernel<WGM, WGN, TM, TN, false, false, false>(const msk::GemmArgs);
MS_INSTANTIATE_F32(4, 2, 2, 2)
MS_INSTANTIATE_F32(4, 2, 1, 3)
MS_INSTANTIATE_F32(2, 2, 2, 2)
MS_INSTANTIATE_F32(2, 2, 1, 1)
MS_INSTANTIATE_F32(2, 2, 3, 3)
#undef MS_INSTANTIATE_F32

namespace {
thread_local char g_err[512] = "";
}

int msi::fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

namespace {

thread_local int g_variant = 0;
thread_local int g_splits = 0;    // forced split count of the contraction (0 = library default)
thread_local int g_launches = 0;   // kernels launched by the last GEMM call of this thread
thread_local int g_last_variant = 0;   // kernel variant of that call's first launch (bf16 tiles 1..VARIANTS, fp32 tiles F32_FIRST..F32_LAST)
thread_local int g_last_splits = 1;    // and the number of ways it split the contraction
thread_local int g_last_grid = 0;      // and its workgroup count
thread_local int g_reserved_cus = 0;   // compute units the GEMM launches of this thread leave free (ms_set_reserved_cus)
thread_local int g_last_tiles_per_chunk = 0;   // output tiles per chunk (per output, for OS) of that call's last launch

using msi::fail;

struct DevFacts {
  int cus = 0, clock_khz = 0, gfx950 = 0, lds = 0;
};
struct DevInfo : DevFacts {
  std::once_flag once;
  hipError_t err = hipSuccess;
};
DevInfo g_dev[64];

// Facts about the calling thread's current device, read from the runtime once per ordinal (call_once: concurrent
// first calls from several host threads wait for the one that fills the entry).
int dev_info(DevInfo **out) {
  int d = 0;
  MS_HIP(hipGetDevice(&d));
  if (d < 0 || d >= 64) return fail(MS_ERR_HIP, "device ordinal %d out of range", d);
  DevInfo &di = g_dev[d];
  std::call_once(di.once, [&di, d]() {
    hipDeviceProp_t p;
    di.err = hipGetDeviceProperties(&p, d);
    if (di.err != hipSuccess) return;
    di.cus = p.multiProcessorCount;
    di.clock_khz = p.clockRate;
    di.gfx950 = strncmp(p.gcnArchName, "gfx950", 6) == 0;
    di.lds = (int)p.sharedMemPerBlock;
  });
  if (di.err != hipSuccess) return fail(MS_ERR_HIP, "hipGetDeviceProperties failed: %s", hipGetErrorString(di.err));
  *out = &di;
  return MS_OK;
}

enum Flow { OS = 0, LS = 1, RS = 2 };

// One local contraction, in kernel terms.
struct Problem {
  Flow flow;
  const void *const *a;  // nkslices (OS) or nchunks (RS) or 1 pointers
  const void *const *b;
  void *const *c;
  int na, nb, nc;
  int S;
  int M, N, K;           // per-chunk rows/cols, per-slice contraction
  int lda, ldb, ldc;
  int in_dtype, out_dtype;
  // fused OS epilogue (all zero / null = plain product)
  int act = 0;
  const void *res = nullptr;
  int ldr = 0;
  float *row_sum = nullptr;
  float *row_sumsq = nullptr;
  // workspace for split contractions (null / 0: none, the contraction is never split)
  void *ws = nullptr;
  size_t ws_bytes = 0;
  // LS / RS: per-chunk completion counters (null: none)
  unsigned *chunk_done = nullptr;
  // OS: per-slice input gate (null: none) and the longest wait for one slice, in ticks of the 100 MHz wall clock
  unsigned *slice_ready = nullptr;
  unsigned long long gate_ticks = 0;
};

// Layout of a split-contraction workspace: SPLIT_MAX_BANDS arrival counters per output tile, then one fp32 partial tile
// per work item.
constexpr size_t WS_HEADER_BYTES = 4096;
constexpr int WS_COUNTERS = (int)(WS_HEADER_BYTES / sizeof(int));
constexpr int WS_MAX_TILES = WS_COUNTERS / msk::SPLIT_MAX_BANDS;     // output tiles of a split product

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int validate(const Problem &p) {
  static const char *names[] = {"ms_gemm_os", "ms_gemm_ls", "ms_gemm_rs"};
  const char *fn = names[p.flow];
  if (p.S < 1 || p.S > MS_MAX_SLICES) return fail(MS_ERR_ARG, "%s: S = %d outside [1, %d]", fn, p.S, MS_MAX_SLICES);
  if (p.M <= 0 || p.N <= 0 || p.K <= 0) return fail(MS_ERR_ARG, "%s: non-positive extent (m=%d n=%d k=%d)", fn, p.M, p.N, p.K);
  if (p.in_dtype != MS_DTYPE_F32 && p.in_dtype != MS_DTYPE_BF16) return fail(MS_ERR_UNSUPPORTED, "%s: unknown in_dtype %d", fn, p.in_dtype);
  if (p.out_dtype != MS_DTYPE_F32 && p.out_dtype != MS_DTYPE_BF16) return fail(MS_ERR_UNSUPPORTED, "%s: unknown out_dtype %d", fn, p.out_dtype);
  if (!p.a || !p.b || !p.c) return fail(MS_ERR_ARG, "%s: null pointer table", fn);
  const int q = p.in_dtype == MS_DTYPE_BF16 ? 8 : 4;  // elements per 16 bytes
  // contiguous extent of each operand, and minimum leading dimension
  const int a_cont = p.flow == RS ? p.M : p.K;
  const int b_cont = p.flow == LS ? p.K : p.N;
  if (a_cont % q || b_cont % q) return fail(MS_ERR_ARG, "%s: contiguous extents (%d, %d) must be multiples of %d", fn, a_cont, b_cont, q);
  if (p.lda < a_cont || p.ldb < b_cont || p.ldc < p.N) return fail(MS_ERR_ARG, "%s: leading dimension smaller than the row length", fn);
  if (p.lda % q || p.ldb % q) return fail(MS_ERR_ARG, "%s: operand leading dimensions must be multiples of %d", fn, q);
  {
    // the kernels address an operand slice with 32-bit byte offsets, the upper half reserved for "out of range"
    const long long a_rows = p.flow == RS ? p.K : p.M, b_rows = p.flow == LS ? p.N : p.K;
    const long long es = p.in_dtype == MS_DTYPE_BF16 ? 2 : 4;
    if (a_rows * p.lda * es > 0x7FFFFFFFLL || b_rows * p.ldb * es > 0x7FFFFFFFLL)
      return fail(MS_ERR_UNSUPPORTED, "%s: an operand slice spans 2 GiB or more", fn);
  }
  const int qo = p.out_dtype == MS_DTYPE_BF16 ? 8 : 4;
  if (p.N % qo || p.ldc % qo) return fail(MS_ERR_ARG, "%s: output columns / leading dimension must be multiples of %d", fn, qo);
  if (p.act != MS_ACT_NONE && p.act != MS_ACT_GELU) return fail(MS_ERR_ARG, "%s: unknown activation %d", fn, p.act);
  if (p.res) {
    if (!aligned16(p.res)) return fail(MS_ERR_ARG, "%s: residual pointer not 16-byte aligned", fn);
    if (p.ldr < p.N || p.ldr % qo) return fail(MS_ERR_ARG, "%s: residual leading dimension %d must be >= n and a multiple of %d", fn, p.ldr, qo);
  }
  if (p.ws && ((reinterpret_cast<uintptr_t>(p.ws) & 255) || p.ws_bytes < WS_HEADER_BYTES))
    return fail(MS_ERR_ARG, "%s: a workspace must be 256-byte aligned and hold at least %zu bytes", fn, WS_HEADER_BYTES);
  if ((reinterpret_cast<uintptr_t>(p.row_sum) | reinterpret_cast<uintptr_t>(p.row_sumsq)) & 3) return fail(MS_ERR_ARG, "%s: row-moment pointers must be 4-byte aligned", fn);
  if ((p.act || p.res || p.row_sum || p.row_sumsq) && (p.flow != OS || p.in_dtype != MS_DTYPE_BF16))
    return fail(MS_ERR_UNSUPPORTED, "%s: the fused epilogue exists for the output-stationary bf16 kernel only", fn);
  for (int i = 0; i < p.na; i++) if (!p.a[i] || !aligned16(p.a[i])) return fail(MS_ERR_ARG, "%s: operand pointer %d null or not 16-byte aligned", fn, i);
  for (int i = 0; i < p.nb; i++) if (!p.b[i] || !aligned16(p.b[i])) return fail(MS_ERR_ARG, "%s: operand pointer %d null or not 16-byte aligned", fn, i);
  for (int i = 0; i < p.nc; i++) if (!p.c[i] || !aligned16(p.c[i])) return fail(MS_ERR_ARG, "%s: output pointer %d null or not 16-byte aligned", fn, i);
  return MS_OK;
}

// KIND 0: gemm_bf16_ring_kernel<BM, BN, ...>; 1: gemm_bf16_big_kernel (32x32x16 MFMA, 2x2 waves, two 64-deep stages);
// 2: gemm_bf16_x16_kernel (256x384x64 or 256x256x64 on the 16x16x32 MFMA)
template <int KIND, int BM, int BN, int BK_, int NS, int WGM, int WGN, bool AK, bool BKM, bool OBF, bool EPI>
void launch_one(dim3 gd, dim3 bd, hipStream_t stream, const msk::GemmArgs &g) {
  if constexpr (KIND == 0) {
    msk::gemm_bf16_ring_kernel<BM, BN, BK_, NS, WGM, WGN, AK, BKM, OBF, EPI><<<gd, bd, 0, stream>>>(g);
  } else if constexpr (KIND == 1) {
    static_assert(BM % 64 == 0 && BN % 64 == 0 && BK_ == 64 && NS == 2 && WGM == 2 && WGN == 2, "the big-tile kernels are 2 x 2 waves on two 64-deep stages");
    msk::gemm_bf16_big_kernel<BM / 64, BN / 64, AK, BKM, OBF, EPI><<<gd, bd, 0, stream>>>(g);
  } else {
    static_assert(BM == 256 && (BN == 384 || BN == 256) && BK_ == 64 && NS == 2 && WGM == 2 && WGN == 2, "the 16x16x32 kernel has two shapes");
    msk::gemm_bf16_x16_kernel<AK, BKM, OBF, EPI, 0, BN><<<gd, bd, 0, stream>>>(g);
  }
}

using msi::balanced_grid;
constexpr double PARTIAL_ROUND_LOSS = 0.6;

// Two workgroups of the 128x128 kernel fit one compute unit (64 KB of LDS and at most 220 registers per lane each) and
// hide each other's barriers and load latencies: 4096^3 on 1024 such tiles 0.165 -> 0.129 ms, 1536 x 4096 x 2048 0.044 ->
// 0.029 ms.  Every other kernel takes the unit's registers or LDS for itself.  With units reserved the 128x128 kernel
// goes back to one workgroup per unit: the dispatcher would spread a larger grid over the reserved units as well.
int workgroups_per_unit(int variant) { return variant == 3 && g_reserved_cus == 0 ? 2 : 1; }

extern const char *const SPLIT_REFUSALS[];
int split_refused(const Problem &p, const DevFacts &dev, int variant, int splits);

// tile BM x BN, WGM x WGN waves, NS ring stages of BK_ k-elements; contraction split `splits` ways
template <int BM, int BN, int WGM, int WGN, int BK_, int NS, int KIND = 0>
int launch_bf16_tile(const Problem &p, const DevFacts &dev, hipStream_t stream, int variant, int splits) {
  msk::GemmArgs g;
  memset(&g, 0, sizeof(g));
  for (int i = 0; i < p.na; i++) g.a[i] = p.a[i];
  for (int i = 0; i < p.nb; i++) g.b[i] = p.b[i];
  for (int i = 0; i < p.nc; i++) g.c[i] = p.c[i];
  g.nchunks = p.flow == OS ? 1 : p.S;
  g.nkslices = p.flow == OS ? p.S : 1;
  g.a_by_chunk = p.flow == RS;
  g.b_by_chunk = p.flow == LS;
  g.M = p.M; g.N = p.N; g.K = p.K;
  g.lda = p.lda; g.ldb = p.ldb; g.ldc = p.ldc;
  g.tiles_m = (p.M + BM - 1) / BM;
  g.tiles_n = (p.N + BN - 1) / BN;
  const long total = (long)g.tiles_m * g.tiles_n * g.nchunks;
  if (total > 0x7FFFFFFF) return fail(MS_ERR_ARG, "problem has too many tiles");
  g.total_tiles = (int)total;
  g.group_m = 8;
  g.splits = 1;
  g.chunk_done = p.chunk_done;
  g.slice_ready = p.slice_ready; g.gate_ticks = p.gate_ticks;
  g_last_tiles_per_chunk = g.tiles_m * g.tiles_n;
  if (splits > 1) {
    const int why = split_refused(p, dev, variant, splits);
    if (why) return fail(MS_ERR_ARG, "contraction cannot be split %d ways here: %s", splits, SPLIT_REFUSALS[why]);
    g.splits = splits;
    g.ws_count = static_cast<int *>(p.ws);
    g.ws_tiles = static_cast<char *>(p.ws) + WS_HEADER_BYTES;
  }
  const long items = total * g.splits;
  const int grid = balanced_grid(items, workgroups_per_unit(variant) * dev.cus);
  dim3 gd(grid), bd(WGM * WGN * 64);
  const bool obf = p.out_dtype == MS_DTYPE_BF16;
  g.act = p.act; g.res = p.res; g.ldr = p.ldr; g.row_sum = p.row_sum; g.row_sumsq = p.row_sumsq;
  const bool epi = p.act != 0 || p.res || p.row_sum || p.row_sumsq;
  if (p.flow == OS) {
    if (epi) {
      if (obf) launch_one<KIND, BM, BN, BK_, NS, WGM, WGN, true, false, true, true>(gd, bd, stream, g);
      else launch_one<KIND, BM, BN, BK_, NS, WGM, WGN, true, false, false, true>(gd, bd, stream, g);
    } else {
      if (obf) launch_one<KIND, BM, BN, BK_, NS, WGM, WGN, true, false, true, false>(gd, bd, stream, g);
      else launch_one<KIND, BM, BN, BK_, NS, WGM, WGN, true, false, false, false>(gd, bd, stream, g);
    }
  } else if (p.flow == LS) {
    if (obf) launch_one<KIND, BM, BN, BK_, NS, WGM, WGN, true, true, true, false>(gd, bd, stream, g);
    else launch_one<KIND, BM, BN, BK_, NS, WGM, WGN, true, true, false, false>(gd, bd, stream, g);
  } else {
    if (obf) launch_one<KIND, BM, BN, BK_, NS, WGM, WGN, false, false, true, false>(gd, bd, stream, g);
    else launch_one<KIND, BM, BN, BK_, NS, WGM, WGN, false, false, false, false>(gd, bd, stream, g);
  }
  if (g_launches == 0) g_last_grid = grid;
  g_launches++;
  MS_HIP(hipGetLastError());
  return MS_OK;
}

// Kernel variants (tile, waves, ring stages x k-elements per stage):
//   1: 256x256, 4 waves, 2 x 64     2: 256x256, 8 waves, 4 x 32     3: 128x128, 4 waves, 2 x 64
//   4: 256x256, 4 waves, 4 x 32     5: 256x192, 4 waves, 4 x 32     6: 192x256, 4 waves, 4 x 32
//   7: 256x256, 8 waves, 2 x 64     8: 256x192, 4 waves, 2 x 64     9: 192x256, 4 waves, 2 x 64
//  10: 256x384, 4 waves, 2 x 64 (gemm_bf16_big_kernel<4, 6>)     11: 384x192, 4 waves, 2 x 64 (gemm_bf16_big_kernel<6, 3>)
//  12: 256x384, 4 waves, 2 x 64 on the 16x16x32 MFMA (gemm_bf16_x16_kernel)     13: 256x256, the same kernel
//  14: 128x128, 4 waves, 3 x 64 (one workgroup per unit: for products of at most one round of such tiles, where a third
//      stage covers the load latency that two 64-deep stages do not: 2048^3 in 20.7 us against 26.3 us, 1536^3 14.7 against 18.8)
// The default picks the tile shape that wastes the least of the machine: a launch runs in
// ceil(work items / CUs) rounds of one item per CU (a partly filled last round is charged in part, see
// balanced_grid), so the estimate is rounds x tile area / relative tile
// efficiency (measured on the GPT-3-sized products, per flop, 256x256 = 1: the 256x384 tile, on the 16x16x32 kernel
// that every such pick runs on, reaches 1.15 (OS) / 1.20 (LS) with a k-contiguous A and 1.16 without, the 384x192 tile 1.04,
// 192-wide ring tiles about 0.93, 128x128 tiles about 0.55, or 0.42 per workgroup with two of them on a unit).  The ring-kernel defaults use four waves over two 64-deep stages when an operand is
// k-contiguous: whole 128-byte lines per request, half as many barriers as 32-deep stages.
//
// An output-stationary product with fewer tiles than compute units may split its contraction (work items = tiles x
// splits, see split_k_exchange): a split item costs 1 / splits of the tile, and the whole launch pays for the exchange
// of partial tiles, which is bound by memory bandwidth (splits x m x n fp32 values written through to memory and read
// back: about 2.8 TB/s) plus a fixed few microseconds.  In the estimate's units (tile area x share of the contraction,
// one compute unit doing about 5.7 TFLOP/s) that is (SPLIT_FIX + splits x m x n x SPLIT_PER_ELEMENT) / K.  Measured on
// 2048 x 1536 x 12288 (64 tiles of 256x192): 170 us unsplit, 100 / 85 / 88 us with 2 / 3 / 4 splits.
struct Pick { int v, splits; double cost; };

constexpr int VARIANTS = 14;
constexpr int F32_FIRST = 21, F32_LAST = 25;      // ids of the fp32 kernel's tiles (ms_set_variant, MS_QUERY_LAST_VARIANT)
struct TileShape { int bm, bn; };
constexpr TileShape TILE_OF[VARIANTS + 1] = {{0, 0},     {256, 256}, {256, 256}, {128, 128}, {256, 256}, {256, 192},
                                             {192, 256}, {256, 256}, {256, 192}, {192, 256}, {256, 384}, {384, 192},
                                             {256, 384}, {256, 256}, {128, 128}};
// unsplit 256x256: the 16x16x32 kernel (variant 13) against the eight-wave ring kernel (variant 7); with two m/n-contiguous
// operands (RS) it gains 0-6 % only, and beyond some 6000 contraction elements per chunk it loses (10240 x 2560 x 12288 in
// two chunks: 0.622 against 0.555 ms), so there the ring kernel stays
constexpr double X16_OVER_RING_256 = 1.10, X16_OVER_RING_256_LS = 1.13, X16_OVER_RING_256_RS = 1.03;
constexpr int X16_RS_MAX_K = 6144;
constexpr int SPLIT_CHOICES[] = {1, 2, 3, 4, 6, 8};
constexpr int SPLIT_MAX = 8;
constexpr long SPLIT_MIN_K = 512;            // contraction elements per split item, at least
constexpr double SPLIT_FIX = 1.4e7;          // fixed cost of an exchange (about 5 us)
constexpr double SPLIT_PER_ELEMENT = 8.2;    // per split and output element (8 bytes through memory)

const char *const SPLIT_REFUSALS[] = {"", "only output-stationary products split their contraction", "no workspace was given",
                                      "more work items than compute units", "too many output tiles for the workspace's counters",
                                      "the partial tiles do not fit the workspace", "too few contraction steps per split",
                                      "split count outside [2, 8]", "this tile variant has no split path",
                                      "products with a fused epilogue are not split"};

// 0 if problem p can run on tile variant v with its contraction split `splits` ways, else an index into SPLIT_REFUSALS
int split_refused(const Problem &p, const DevFacts &dev, int v, int splits) {
  const int bm = TILE_OF[v].bm, bn = TILE_OF[v].bn;
  if (splits < 2 || splits > SPLIT_MAX) return 7;
  if (v == 1 || v == 4 || v == 12 || v == 13) return 8;     // 256x256 on four waves: see ring_can_split; the 16x16x32 kernels have none
  if (p.act || p.res || p.row_sum || p.row_sumsq) return 9;   // see ring_can_split, big_can_split
  if (p.flow != OS) return 1;
  if (!p.ws) return 2;
  const long tiles = (long)((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn);
  if (tiles * splits > dev.cus) return 3;
  if (tiles > WS_MAX_TILES) return 4;
  if ((size_t)(tiles * splits) * bm * bn * sizeof(float) + WS_HEADER_BYTES > p.ws_bytes) return 5;
  if (((long)(p.K + 63) / 64) * p.S < splits) return 6;     // every part needs at least one 64-deep K step
  return 0;
}

// the tile shape and split count with the lowest estimated cost for the whole problem
Pick pick_variant(const Problem &p, const DevFacts &dev) {
  struct Cand { int v; double eff; };
  // with two m/n-contiguous operands (RS) the hand-scheduled tiles gain less over the 256x256 ring than with a
  // k-contiguous operand, and the 192-wide ring tiles do best on four 32-deep stages
  // (256x256 runs on eight waves, two per SIMD: 1-3 % faster than four waves, 10-15 % on short contractions, where
  // prologue and write-out weigh most, and the one of the two that can split its contraction: 2048 x 2048 x 16384 in
  // 0.125 ms on 64 tiles x 4 splits, 0.165 ms on 256 tiles of 128x128; four waves stay selectable as variant 1)
  const bool rs = p.flow == RS, ls = p.flow == LS;
  const Cand cands[] = {{7, 1.0}, {10, rs ? 1.16 : ls ? 1.20 : 1.15}, {11, 1.04}, {rs ? 5 : 8, rs ? 0.95 : 0.93}, {rs ? 6 : 9, rs ? 0.95 : 0.93}, {3, workgroups_per_unit(3) == 2 ? 0.42 : 0.55}, {14, 0.66}};
  const long chunks = p.flow == OS ? 1 : p.S;
  const double total_k = p.flow == OS ? (double)p.K * p.S : (double)p.K;
  Pick best = {0, 1, 0};
  for (const Cand &c : cands) {
    const int bm = TILE_OF[c.v].bm, bn = TILE_OF[c.v].bn;
    const long tiles = (long)((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) * chunks;
    for (int splits : SPLIT_CHOICES) {
      if (g_splits != 0 && splits != g_splits) continue;
      if (splits > 1 && (split_refused(p, dev, c.v, splits) || (g_splits == 0 && total_k / splits < SPLIT_MIN_K))) continue;
      // rounds the launch is charged: whole ones, or with the last round partly filled (see balanced_grid) its filled
      // share plus PARTIAL_ROUND_LOSS of the rest
      const long slots = (long)dev.cus * (splits == 1 ? workgroups_per_unit(c.v) : 1);     // (a split launch is one item per unit)
      const double exact = (double)(tiles * splits) / slots;
      const double whole = (double)((tiles * splits + slots - 1) / slots);
      // (the 128x128 kernels do not reach the power limit: their units gain no clock from idle neighbours)
      const bool small_tile = c.v == 3 || c.v == 14;
      const double loss = small_tile ? 1.0 : PARTIAL_ROUND_LOSS;
      // (a launch of less than one round is charged the same way, down to 0.7 of a round: the idle units' power lets the
      // busy ones clock up to 1.4 times higher)
      const double part = exact + loss * (1.0 - exact);
      const double rounds = exact <= 1.0 ? (part > 0.7 ? part : 0.7) : exact + loss * (whole - exact);
      const double exchange = splits == 1 ? 0.0 : (SPLIT_FIX + (double)splits * p.M * p.N * SPLIT_PER_ELEMENT) / total_k;
      // (a split 256x384 product stays on the 32x32x16 kernel, which carries the exchange and is about 5 % slower; an
      // unsplit 256x256 one runs on the 16x16x32 kernel, 7-14 % faster than the eight-wave ring kernel that carries the split)
      // (two 128x128 workgroups share a unit only where there are more tiles than units: 0.55 alone, 0.42 each when every
      // unit holds two)
      const double shared = c.v == 3 && workgroups_per_unit(3) == 2 ? (tiles * splits <= dev.cus ? 0.0 : tiles * splits >= 2L * dev.cus ? 1.0 : (double)(tiles * splits - dev.cus) / dev.cus) : 0.0;
      const double eff = c.v == 3 && workgroups_per_unit(3) == 2 ? 0.55 - 0.13 * shared : c.v == 10 && splits > 1 ? c.eff / 1.05 : c.v == 7 && splits == 1 ? c.eff * (ls ? X16_OVER_RING_256_LS : !rs ? X16_OVER_RING_256 : p.K <= X16_RS_MAX_K ? X16_OVER_RING_256_RS : 1.0) : c.eff;
      const double cost = rounds * bm * bn / eff / splits + exchange;
      if (best.v == 0 || cost < best.cost) best = {c.v, splits, cost};
    }
  }
  // An unsplit 256x384 product runs on the 16x16x32 kernel: 4-8 % faster than the 32x32x16 one, which stays selectable
  // as variant 10 and carries the split contraction.
  if (best.splits == 1 && best.v == 10) best.v = 12;
  // Likewise an unsplit 256x256 product (4096^3 in 0.093-0.095 ms against 0.106 ms on the ring kernel, 4096 x 4096 x 14336 in
  // 0.302-0.309 against 0.344 ms); the eight-wave ring kernel stays selectable as variant 7 and carries the split contraction.
  // (not where an LS chunk is a single tile column: every XCD then streams all of A, the product is bound by the fabric, and
  // two waves per SIMD ride that out better: 8192 x 256 x 8192 in eight chunks 0.217 against 0.262 ms)
  const bool one_column_chunks = ls && p.N <= 256;
  if (best.splits == 1 && best.v == 7 && !(rs && p.K > X16_RS_MAX_K) && !one_column_chunks) best.v = 13;
  return best;
}

int launch_variant(int v, int splits, const Problem &p, const DevFacts &dev, hipStream_t stream) {
  if (p.slice_ready && (v == 1 || v == 4)) return fail(MS_ERR_UNSUPPORTED, "tile variant %d has no input gate (256x256 on four waves of the ring kernel)", v);
  if (g_launches == 0) { g_last_variant = v; g_last_splits = splits; }
  switch (v) {
    case 1: return launch_bf16_tile<256, 256, 2, 2, 64, 2>(p, dev, stream, 1, splits);
    case 2: return launch_bf16_tile<256, 256, 2, 4, 32, 4>(p, dev, stream, 2, splits);
    case 3: return launch_bf16_tile<128, 128, 2, 2, 64, 2>(p, dev, stream, 3, splits);
    case 4: return launch_bf16_tile<256, 256, 2, 2, 32, 4>(p, dev, stream, 4, splits);
    case 5: return launch_bf16_tile<256, 192, 2, 2, 32, 4>(p, dev, stream, 5, splits);
    case 6: return launch_bf16_tile<192, 256, 2, 2, 32, 4>(p, dev, stream, 6, splits);
    case 7: return launch_bf16_tile<256, 256, 2, 4, 64, 2>(p, dev, stream, 7, splits);
    case 8: return launch_bf16_tile<256, 192, 2, 2, 64, 2>(p, dev, stream, 8, splits);
    case 9: return launch_bf16_tile<192, 256, 2, 2, 64, 2>(p, dev, stream, 9, splits);
    case 10: return launch_bf16_tile<256, 384, 2, 2, 64, 2, 1>(p, dev, stream, 10, splits);
    case 11: return launch_bf16_tile<384, 192, 2, 2, 64, 2, 1>(p, dev, stream, 11, splits);
    case 12: return launch_bf16_tile<256, 384, 2, 2, 64, 2, 2>(p, dev, stream, 12, splits);
    case 13: return launch_bf16_tile<256, 256, 2, 2, 64, 2, 2>(p, dev, stream, 13, splits);
    case 14: return launch_bf16_tile<128, 128, 2, 2, 64, 3>(p, dev, stream, 14, splits);
    default: return fail(MS_ERR_ARG, "unknown kernel variant %d", v);
  }
}

// An output-stationary product whose best single tile shape leaves much of its last round idle is done in two
// launches: the 256x384 tile on as many leading tile columns of C as fill whole rounds, the best shape for what
// is left on the remaining columns (4096x9216x12288: 256 tiles of 256x384 plus 256 tiles of 256x192, 0.67 ms,
// instead of 768 tiles of 256x192 in three rounds, 0.76 ms).  The second launch costs about a hundredth of a
// millisecond (launch gap, one more prologue), which the estimate charges as tile area.  LS / RS are not split:
// their chunks are promised in slice order.
int launch_bf16(const Problem &p, const DevFacts &dev, hipStream_t stream) {
  if (!dev.gfx950) return fail(MS_ERR_UNSUPPORTED, "the bf16 kernels need a gfx950 device");
  if (g_variant >= 1 && g_variant <= VARIANTS) return launch_variant(g_variant, g_splits > 1 ? g_splits : 1, p, dev, stream);
  const Pick single = pick_variant(p, dev);
  // (a gated product stays one launch: a second one would stand in the stream behind the first while that waits for slices)
  if (p.flow == OS && single.splits == 1 && g_splits == 0 && !p.slice_ready) {
    constexpr int BM = 256, BN = 384;
    constexpr double EFF = 1.15;
    const long tiles_m = (p.M + BM - 1) / BM;
    const long total_k = (long)p.K * p.S;
    // whole rounds of the big tile: the largest count of leading tile columns whose tiles are a multiple of the CUs
    long nb1 = p.N / BN;
    while (nb1 > 0 && (tiles_m * nb1) % dev.cus != 0) nb1--;
    const long n1 = nb1 * BN;
    if (nb1 > 0 && n1 < p.N) {
      Problem rest = p;
      rest.N = p.N - (int)n1;
      rest.ws = nullptr;   // the second launch is not split: the first may still be using the workspace's counters
      const Pick tail = pick_variant(rest, dev);
      const double second_launch = 3.4e7 / (double)total_k;      // ~12 us at the rate one CU computes tile area x K
      const double cost = (double)(tiles_m * nb1 / dev.cus) * BM * BN / EFF + tail.cost + second_launch;
      if (cost < 0.97 * single.cost) {
        const int es_in = 2, es_out = p.out_dtype == MS_DTYPE_BF16 ? 2 : 4;
        Problem head = p;
        head.N = (int)n1;
        int rc = launch_variant(12, 1, head, dev, stream);   // (see pick_variant)
        if (rc != MS_OK) return rc;
        const void *b2[MS_MAX_SLICES];
        void *c2[1] = {static_cast<char *>(p.c[0]) + n1 * es_out};
        for (int s = 0; s < p.nb; s++) b2[s] = static_cast<const char *>(p.b[s]) + n1 * es_in;
        rest.b = b2;
        rest.c = c2;
        if (p.res) rest.res = static_cast<const char *>(p.res) + n1 * es_out;
        return launch_variant(tail.v, 1, rest, dev, stream);
      }
    }
  }
  return launch_variant(single.v, single.splits, p, dev, stream);
}

// fp32 operands: gemm_f32_tile_kernel on one of its five tiles (ids F32_FIRST ..: 256 x 128 and 128 x 192 on eight
// waves, 128 x 128, 64 x 64 and 192 x 192 on four); `share`: two workgroups of the 128 x 128 or 64 x 64 tile per compute unit
int f32_split_refused(const Problem &p, const DevFacts &dev, int bm, int bn, int splits);

template <int WGM, int WGN, int TM, int TN>
int launch_f32_tile(const Problem &p, const DevFacts &dev, hipStream_t stream, int id, bool share, int splits) {
  constexpr int BM = 32 * TM * WGM, BN = 32 * TN * WGN;
  msk::GemmArgs g;
  memset(&g, 0, sizeof(g));
  for (int i = 0; i < p.na; i++) g.a[i] = p.a[i];
  for (int i = 0; i < p.nb; i++) g.b[i] = p.b[i];
  for (int i = 0; i < p.nc; i++) g.c[i] = p.c[i];
  g.nchunks = p.flow == OS ? 1 : p.S;
  g.nkslices = p.flow == OS ? p.S : 1;
  g.a_by_chunk = p.flow == RS;
  g.b_by_chunk = p.flow == LS;
  g.M = p.M; g.N = p.N; g.K = p.K;
  g.lda = p.lda; g.ldb = p.ldb; g.ldc = p.ldc;
  g.tiles_m = (p.M + BM - 1) / BM;
  g.tiles_n = (p.N + BN - 1) / BN;
  const long total = (long)g.tiles_m * g.tiles_n * g.nchunks;
  if (total > 0x7FFFFFFF) return fail(MS_ERR_ARG, "problem has too many tiles");
  g.total_tiles = (int)total;
  g.group_m = 8;
  g.splits = 1;
  g.chunk_done = p.chunk_done;
  g.slice_ready = p.slice_ready; g.gate_ticks = p.gate_ticks;
  g_last_tiles_per_chunk = g.tiles_m * g.tiles_n;
  if (splits > 1) {
    const int why = f32_split_refused(p, dev, BM, BN, splits);
    if (why) return fail(MS_ERR_ARG, "contraction cannot be split %d ways here: %s", splits, SPLIT_REFUSALS[why]);
    g.splits = splits;
    g.ws_count = static_cast<int *>(p.ws);
    g.ws_tiles = static_cast<char *>(p.ws) + WS_HEADER_BYTES;
  }
  const long items = total * g.splits;
  const int grid = !(share && WGM * WGN == 4) ? balanced_grid(items, dev.cus) : items <= 2L * dev.cus ? (int)items : balanced_grid(items, 2 * dev.cus);
  dim3 gd(grid), bd(WGM * WGN * 64);
  const bool obf = p.out_dtype == MS_DTYPE_BF16;
  if (p.flow == OS) {
    if (obf) msk::gemm_f32_tile_kernel<WGM, WGN, TM, TN, true, false, true><<<gd, bd, 0, stream>>>(g);
    else msk::gemm_f32_tile_kernel<WGM, WGN, TM, TN, true, false, false><<<gd, bd, 0, stream>>>(g);
  } else if (p.flow == LS) {
    if (obf) msk::gemm_f32_tile_kernel<WGM, WGN, TM, TN, true, true, true><<<gd, bd, 0, stream>>>(g);
    else msk::gemm_f32_tile_kernel<WGM, WGN, TM, TN, true, true, false><<<gd, bd, 0, stream>>>(g);
  } else {
    if (obf) msk::gemm_f32_tile_kernel<WGM, WGN, TM, TN, false, false, true><<<gd, bd, 0, stream>>>(g);
    else msk::gemm_f32_tile_kernel<WGM, WGN, TM, TN, false, false, false><<<gd, bd, 0, stream>>>(g);
  }
  if (g_launches == 0) { g_last_grid = (int)gd.x; g_last_variant = id; g_last_splits = g.splits; }
  g_launches++;
  MS_HIP(hipGetLastError());
  return MS_OK;
}

// 0 if the fp32 product p can run on a bm x bn tile with its contraction split `splits` ways, else an index into SPLIT_REFUSALS
int f32_split_refused(const Problem &p, const DevFacts &dev, int bm, int bn, int splits) {
  if (splits < 2 || splits > SPLIT_MAX) return 7;
  if (p.flow != OS) return 1;
  if (!p.ws) return 2;
  const long tiles = (long)((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn);
  if (tiles * splits > dev.cus) return 3;
  if (tiles > WS_MAX_TILES) return 4;
  if ((size_t)(tiles * splits) * bm * bn * sizeof(float) + WS_HEADER_BYTES > p.ws_bytes) return 5;
  if (((long)(p.K + 31) / 32) * p.S < splits) return 6;     // every part needs at least one K step
  return 0;
}

// The fp32 tiles as the chooser prices them: time per output element and contraction step relative to the 256 x 128
// tile's, for a unit that holds one workgroup, and the factor by which a unit that holds two four-wave workgroups takes
// longer over the pair.  Fitted to ten products from 512^2 x 1024 to 4096^3 (one round of 256 tiles of 128 x 192 on
// 4096 contraction elements 363 us, of 256 x 128 468 us, of 128 x 128 on 8192 elements 510 us; 512 tiles of 64 x 64
// shared 133 us, alone in two rounds 150 us; 1024 tiles of 128 x 128 shared 957 us; one round of 256 tiles of 192 x 192,
// four waves of 3 x 3 tiles each, 567 us).  Unlike the bf16 kernels this one
// does not sit on the power limit: a partly filled round costs a whole one.
struct F32Tile { int id, bm, bn; bool pairs; double cost, shared; };      // pairs: two such workgroups fit a compute unit
constexpr F32Tile F32_TILES[] = {{F32_FIRST, 256, 128, false, 1.0, 0.0}, {F32_FIRST + 1, 128, 192, false, 1.0 / 0.967, 0.0},
                                 {F32_FIRST + 2, 128, 128, true, 1.0 / 0.918, 1.88}, {F32_FIRST + 3, 64, 64, true, 1.0 / 0.78, 1.78},
                                 {F32_FIRST + 4, 192, 192, false, 1.0 / 0.93, 0.0}};

int launch_f32_id(int id, bool share, int splits, const Problem &p, const DevFacts &dev, hipStream_t stream) {
  switch (id) {
    case F32_FIRST: return launch_f32_tile<4, 2, 2, 2>(p, dev, stream, id, false, splits);
    case F32_FIRST + 1: return launch_f32_tile<4, 2, 1, 3>(p, dev, stream, id, false, splits);
    case F32_FIRST + 2: return launch_f32_tile<2, 2, 2, 2>(p, dev, stream, id, share, splits);
    case F32_FIRST + 3: return launch_f32_tile<2, 2, 1, 1>(p, dev, stream, id, share, splits);
    default: return launch_f32_tile<2, 2, 3, 3>(p, dev, stream, id, false, splits);
  }
}

// An output-stationary fp32 product whose tiles leave compute units idle may split its contraction like the bf16 ones
// (work items = tiles x splits, see split_k_exchange).  The exchange of the partial tiles is priced, in the chooser's
// unit (the 256 x 128 tile's time per output element and contraction step, 3.5e-6 us), at
// (F32_SPLIT_FIX + splits x m x n x F32_SPLIT_PER_ELEMENT) / K: about 5 us plus 2 us per million partial elements,
// fitted to 2048 x 2048 x 8192 (128 tiles of 256 x 128 in two parts: 484 us against 513 us unsplit on 128 x 128) and
// 1536 x 1536 x 4096 (72 tiles in three parts: 179 us against 224 us on 64 x 64 tiles in three rounds).
constexpr double F32_SPLIT_FIX = 1.43e6, F32_SPLIT_PER_ELEMENT = 0.6;
constexpr long F32_SPLIT_MIN_K = 256;      // contraction elements per split item, at least

// the fp32 tile, whether its workgroups pair up on the units, and the split count with the lowest estimated cost (id 0: a
// forced tile and split count that cannot be)
struct F32Pick { int id, splits; bool share; };
F32Pick pick_f32(const Problem &p, const DevFacts &dev) {
  const long chunks = p.flow == OS ? 1 : p.S;
  const long total_k = (long)p.K * (p.flow == OS ? p.S : 1);
  const bool forced_tile = g_variant >= F32_FIRST;
  F32Pick best = {0, 1, false};
  double best_cost = 0.0;
  for (const F32Tile &t : F32_TILES) {
    if (forced_tile && g_variant != t.id) continue;
    const long tiles = (long)((p.M + t.bm - 1) / t.bm) * ((p.N + t.bn - 1) / t.bn) * chunks;
    const double area = (double)t.bm * t.bn * t.cost;
    for (int splits = 1; splits <= SPLIT_MAX; splits++) {
      if (forced_tile && g_splits != 0 && splits != g_splits) continue;
      if (!forced_tile && g_splits != 0) { if (splits > 1) break; }      // (a split forced for the bf16 tiles says nothing here)
      if (splits > 1 && (f32_split_refused(p, dev, t.bm, t.bn, splits) || (!(forced_tile && g_splits != 0) && total_k / splits < F32_SPLIT_MIN_K))) continue;
      const long items = tiles * splits;
      double cost = (double)((items + dev.cus - 1) / dev.cus) * area / splits;
      bool share = false;
      if (t.pairs && g_reserved_cus == 0 && items > dev.cus) {
        const double both = (double)((items + 2L * dev.cus - 1) / (2L * dev.cus)) * area * t.shared / splits;
        if (both < cost) { cost = both; share = true; }
      }
      if (splits > 1) cost += (F32_SPLIT_FIX + (double)splits * p.M * p.N * F32_SPLIT_PER_ELEMENT) / total_k;
      if (best.id == 0 || cost < best_cost) { best = {t.id, splits, share}; best_cost = cost; }
    }
  }
  return best;
}

int launch_f32(const Problem &p, const DevFacts &dev, hipStream_t stream) {
  const F32Pick best = pick_f32(p, dev);
  if (best.id == 0) return fail(MS_ERR_ARG, "contraction cannot be split %d ways on fp32 tile %d here", g_splits, g_variant);
  return launch_f32_id(best.id, best.share, best.splits, p, dev, stream);
}

// the device as this thread's launches may use it: without the compute units it has been told to leave free
DevFacts usable(const DevInfo &dev) {
  DevFacts f = dev;
  f.cus = f.cus - g_reserved_cus > 0 ? f.cus - g_reserved_cus : 1;
  return f;
}

int run(const Problem &p, void *stream) {
  int rc = validate(p);
  if (rc) return rc;
  DevInfo *dev = nullptr;
  rc = dev_info(&dev);
  if (rc) return rc;
  hipStream_t st = (hipStream_t)stream;
  g_launches = 0;
  g_last_variant = 0;
  g_last_splits = 1;
  // the kernels are persistent, one workgroup per compute unit: with units reserved they run on the rest, and the
  // tile choice plans for that many
  const DevFacts facts = usable(*dev);
  return p.in_dtype == MS_DTYPE_BF16 ? launch_bf16(p, facts, st) : launch_f32(p, facts, st);
}

int timed(const Problem &p, void *stream, int warmup, int reps, float *ms_out) {
  if (warmup < 0 || reps < 1 || !ms_out) return fail(MS_ERR_ARG, "timing: need warmup >= 0, reps >= 1 and an output array");
  hipStream_t st = (hipStream_t)stream;
  for (int i = 0; i < warmup; i++) {
    int rc = run(p, stream);
    if (rc) return rc;
  }
  hipEvent_t e0, e1;
  MS_HIP(hipEventCreate(&e0));
  MS_HIP(hipEventCreate(&e1));
  int rc = MS_OK;
  for (int r = 0; r < reps && rc == MS_OK; r++) {
    (void)hipEventRecord(e0, st);
    rc = run(p, stream);
    (void)hipEventRecord(e1, st);
    if (hipEventSynchronize(e1) != hipSuccess) rc = fail(MS_ERR_HIP, "hipEventSynchronize failed");
    float ms = 0.f;
    if (rc == MS_OK && hipEventElapsedTime(&ms, e0, e1) != hipSuccess) rc = fail(MS_ERR_HIP, "hipEventElapsedTime failed");
    ms_out[r] = ms;
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc == MS_OK) MS_HIP(hipStreamSynchronize(st));
  return rc;
}

Problem make_problem(Flow flow, const void *const *a, const void *const *b, void *const *c, int na, int nb, int nc, int S,
                     int m, int n, int k, int lda, int ldb, int ldc, int in_dtype, int out_dtype) {
  Problem p;
  p.flow = flow; p.a = a; p.b = b; p.c = c; p.na = na; p.nb = nb; p.nc = nc; p.S = S;
  p.M = m; p.N = n; p.K = k; p.lda = lda; p.ldb = ldb; p.ldc = ldc; p.in_dtype = in_dtype; p.out_dtype = out_dtype;
  if (S < 1 || S > MS_MAX_SLICES) p.na = p.nb = p.nc = 0;   // the pointer tables are not read for a bad S
  return p;
}
Problem make_os(const void *const *A, const void *const *B, int S, int m, int n, int k, int lda, int ldb,
                void *const *C, int ldc, int in_dtype, int out_dtype) {
  return make_problem(OS, A, B, C, S, S, 1, S, m, n, k, lda, ldb, ldc, in_dtype, out_dtype);
}
Problem make_ls(const void *const *A, int lda, const void *const *W, int ldw, int S, int m, int n, int k,
                void *const *Y, int ldy, int in_dtype, int out_dtype = MS_DTYPE_F32) {
  return make_problem(LS, A, W, Y, 1, S, S, S, m, n, k, lda, ldw, ldy, in_dtype, out_dtype);
}
Problem make_rs(const void *const *X, int ldx, const void *const *W, int ldw, int S, int m, int n, int k,
                void *const *Y, int ldy, int in_dtype, int out_dtype = MS_DTYPE_F32) {
  return make_problem(RS, X, W, Y, S, 1, S, S, m, n, k, ldx, ldw, ldy, in_dtype, out_dtype);
}

}  // namespace

MS_API int ms_version(void) { return 100; }

MS_API const char *ms_last_error(void) { return g_err; }

MS_API long ms_query(int what) {
  if (what == MS_QUERY_MAX_SLICES) return MS_MAX_SLICES;
  if (what == MS_QUERY_LAST_LAUNCHES) return g_launches;
  if (what == MS_QUERY_LAST_VARIANT) return g_last_variant;
  if (what == MS_QUERY_LAST_SPLITS) return g_last_splits;
  if (what == MS_QUERY_LAST_GRID) return g_last_grid;
  DevInfo *d = nullptr;
  if (dev_info(&d) != MS_OK) return -1;
  switch (what) {
    case MS_QUERY_CU_COUNT: return d->cus;
    case MS_QUERY_CLOCK_KHZ: return d->clock_khz;
    case MS_QUERY_IS_GFX950: return d->gfx950;
    case MS_QUERY_LDS_BYTES: return d->lds;
    default: fail(MS_ERR_ARG, "ms_query: unknown selector %d", what); return -1;
  }
}

MS_API int ms_set_variant(int variant) {
  const int v = variant % 100, splits = variant / 100;
  const bool known = v <= VARIANTS || (v >= F32_FIRST && v <= F32_LAST);
  if (variant < 0 || !known || splits == 1 || splits > SPLIT_MAX) return fail(MS_ERR_ARG, "ms_set_variant: unknown variant %d", variant);
  g_variant = v;
  g_splits = splits;
  return MS_OK;
}

MS_API int ms_set_reserved_cus(int n) {
  if (n < 0 || n > 1024) return fail(MS_ERR_ARG, "ms_set_reserved_cus: %d out of range", n);
  g_reserved_cus = n;
  return MS_OK;
}

// Scratch of the entry point that allocates nothing (ms_gemm_os_noalloc): a split-contraction workspace that lives in
// the code object.  Every device the library runs on holds its own copy, at its own address, until the process ends; the
// name below is only a handle for hipGetSymbolAddress, host code never passes it to a kernel.
constexpr size_t NOALLOC_SCRATCH_BYTES = WS_HEADER_BYTES + (size_t)256 * 256 * 192 * sizeof(float);   // 256 partial tiles of 256 x 192
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];

namespace {
struct ScratchAddr {
  std::mutex lock;
  void *ptr = nullptr;             // device address of `scratch` on this device, once looked up
  hipStream_t last_stream = nullptr;
  bool used = false;               // a call has used the scratch on last_stream
};
ScratchAddr g_scratch[64];

// The scratch entry of the calling thread's current device; its address is looked up with that device current on the
// first call that gets an answer (a failed look-up is reported and tried again by the next call).
int scratch_address(ScratchAddr **entry) {
  int d = 0;
  MS_HIP(hipGetDevice(&d));
  if (d < 0 || d >= 64) return fail(MS_ERR_HIP, "device ordinal %d out of range", d);
  ScratchAddr &sa = g_scratch[d];
  std::lock_guard<std::mutex> hold(sa.lock);
  if (!sa.ptr) {
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return fail(MS_ERR_HIP, "hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
    sa.ptr = p;
  }
  *entry = &sa;
  return MS_OK;
}

__global__ void ws_clear_kernel(int *counters, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) counters[i] = 0;
}
}  // namespace

MS_API size_t ms_workspace_bytes(void) {
  DevInfo *d = nullptr;
  if (dev_info(&d) != MS_OK) return 0;
  // one partial tile of the largest shape (256 x 384 fp32) per compute unit
  return WS_HEADER_BYTES + (size_t)d->cus * 256 * 384 * sizeof(float);
}

MS_API int ms_workspace_init(void *workspace, size_t bytes, void *stream) {
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255) || bytes < WS_HEADER_BYTES)
    return fail(MS_ERR_ARG, "ms_workspace_init: a workspace must be 256-byte aligned and hold at least %zu bytes", WS_HEADER_BYTES);
  // a fill kernel, not hipMemsetAsync, so that the call may be captured into a HIP graph
  hipLaunchKernelGGL(ws_clear_kernel, dim3(WS_COUNTERS / 256), dim3(256), 0, (hipStream_t)stream, static_cast<int *>(workspace), WS_COUNTERS);
  MS_HIP(hipGetLastError());
  return MS_OK;
}

MS_API int ms_gemm_os(const void *const *A_slices, const void *const *B_slices, int S, int m, int n, int k_slice,
                      int lda, int ldb, void *C, int ldc, int in_dtype, int out_dtype, void *stream) {
  void *c1[1] = {C};
  return run(make_os(A_slices, B_slices, S, m, n, k_slice, lda, ldb, c1, ldc, in_dtype, out_dtype), stream);
}

MS_API int ms_gemm_os_fused(const void *const *A_slices, const void *const *B_slices, int S, int m, int n, int k_slice,
                            int lda, int ldb, void *C, int ldc, int in_dtype, int out_dtype, int activation,
                            const void *residual, int ldr, float *row_sum, float *row_sumsq, void *stream) {
  void *c1[1] = {C};
  Problem p = make_os(A_slices, B_slices, S, m, n, k_slice, lda, ldb, c1, ldc, in_dtype, out_dtype);
  p.act = activation; p.res = residual; p.ldr = ldr; p.row_sum = row_sum; p.row_sumsq = row_sumsq;
  return run(p, stream);
}

MS_API int ms_gemm_os_ws(const void *const *A_slices, const void *const *B_slices, int S, int m, int n, int k_slice,
                         int lda, int ldb, void *C, int ldc, int in_dtype, int out_dtype, int activation,
                         const void *residual, int ldr, float *row_sum, float *row_sumsq,
                         void *workspace, size_t workspace_bytes, void *stream) {
  void *c1[1] = {C};
  Problem p = make_os(A_slices, B_slices, S, m, n, k_slice, lda, ldb, c1, ldc, in_dtype, out_dtype);
  p.act = activation; p.res = residual; p.ldr = ldr; p.row_sum = row_sum; p.row_sumsq = row_sumsq;
  p.ws = workspace; p.ws_bytes = workspace ? workspace_bytes : 0;
  return run(p, stream);
}

__global__ void signal_set_kernel(unsigned *flag, unsigned value) {
  // everything enqueued on the stream before this kernel has ended; the release makes it visible to whoever then reads the flag
  __hip_atomic_store(flag, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// the gate's half of a Problem: the flags, and the longest wait for one of them in ticks of wall_clock64()
namespace {
int set_gate(Problem &p, unsigned *slice_ready, unsigned timeout_ms, const char *fn) {
  if (!slice_ready || (reinterpret_cast<uintptr_t>(slice_ready) & 3))
    return fail(MS_ERR_ARG, "%s: slice_ready must be a 4-byte aligned device pointer to S + 1 words", fn);
  if (timeout_ms == 0 || timeout_ms > 60000) return fail(MS_ERR_ARG, "%s: timeout_ms %u outside [1, 60000]", fn, timeout_ms);
  p.slice_ready = slice_ready;
  int device = 0, wall_khz = 0;
  MS_HIP(hipGetDevice(&device));
  MS_HIP(hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, device));
  p.gate_ticks = (unsigned long long)timeout_ms * (unsigned long long)(wall_khz > 0 ? wall_khz : 100000);
  return MS_OK;
}
}  // namespace

MS_API int ms_gemm_os_gated(const void *const *A_slices, const void *const *B_slices, int S, int m, int n, int k_slice,
                            int lda, int ldb, void *C, int ldc, int in_dtype, int out_dtype,
                            void *workspace, size_t workspace_bytes, unsigned *slice_ready, unsigned timeout_ms, void *stream) {
  void *c1[1] = {C};
  Problem p = make_os(A_slices, B_slices, S, m, n, k_slice, lda, ldb, c1, ldc, in_dtype, out_dtype);
  p.ws = workspace; p.ws_bytes = workspace ? workspace_bytes : 0;
  const int rc = set_gate(p, slice_ready, timeout_ms, "ms_gemm_os_gated");
  return rc ? rc : run(p, stream);
}

MS_API int ms_signal_set(unsigned *flag, unsigned value, void *stream) {
  if (!flag || (reinterpret_cast<uintptr_t>(flag) & 3)) return fail(MS_ERR_ARG, "ms_signal_set: flag must be a 4-byte aligned device pointer");
  hipLaunchKernelGGL(signal_set_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, flag, value);
  MS_HIP(hipGetLastError());
  return MS_OK;
}

MS_API int ms_gemm_os_noalloc(const void *const *A_slices, const void *const *B_slices, int S, int m, int n, int k_slice,
                              int lda, int ldb, void *C, int ldc, int in_dtype, int out_dtype, void *stream) {
  void *c1[1] = {C};
  Problem p = make_os(A_slices, B_slices, S, m, n, k_slice, lda, ldb, c1, ldc, in_dtype, out_dtype);
  int rc = validate(p);
  if (rc) return rc;
  DevInfo *dev = nullptr;
  rc = dev_info(&dev);
  if (rc) return rc;
  // what the library would do with room to spare decides whether the built-in scratch is needed, and whether it is enough
  p.ws = reinterpret_cast<void *>(uintptr_t(256));    // stands for "a workspace": only its size is looked at here
  p.ws_bytes = ~size_t(0);
  int splits = 1, bm = 0, bn = 0;
  if (in_dtype == MS_DTYPE_BF16) {
    const Pick want = g_variant >= 1 && g_variant <= VARIANTS ? Pick{g_variant, g_splits > 1 ? g_splits : 1, 0.0} : pick_variant(p, usable(*dev));
    splits = want.splits; bm = TILE_OF[want.v].bm; bn = TILE_OF[want.v].bn;
  } else {
    const F32Pick want = pick_f32(p, usable(*dev));
    splits = want.id ? want.splits : 1;
    for (const F32Tile &t : F32_TILES) if (t.id == want.id) { bm = t.bm; bn = t.bn; }
  }
  if (splits <= 1) {
    // an unsplit product exchanges nothing (without a workspace the library makes the same choice: splits are only ever added)
    p.ws = nullptr;
    p.ws_bytes = 0;
    return run(p, stream);
  }
  const size_t tiles = (size_t)((m + bm - 1) / bm) * ((n + bn - 1) / bn);
  const size_t need = WS_HEADER_BYTES + tiles * splits * bm * bn * sizeof(float);
  if (need > NOALLOC_SCRATCH_BYTES)
    return fail(MS_ERR_UNSUPPORTED, "ms_gemm_os_noalloc: this product (m=%d n=%d k=%d x %d slices) would exchange %zu bytes of partial "
                "tiles, the built-in scratch holds %zu; use ms_gemm_os_ws with a workspace of ms_workspace_bytes()",
                m, n, k_slice, S, need, NOALLOC_SCRATCH_BYTES);
  ScratchAddr *sa = nullptr;
  rc = scratch_address(&sa);
  if (rc) return rc;
  // A product that splits leaves counters and partial tiles in the one array of its device, so two such calls must not
  // overlap.  Calls on one stream never do.  A call that comes on ANOTHER stream than the array's previous user first
  // waits for the device to go idle (hipDeviceSynchronize: allocates nothing), and the entry stays locked until this
  // call's kernels are queued, so eager calls from several streams or host threads cannot meet in the array.  A stream
  // under capture launches nothing now and cannot be waited for: how replays of such a graph are ordered against the
  // array's other users is the caller's business.
  std::lock_guard<std::mutex> hold(sa->lock);
  hipStream_t st = (hipStream_t)stream;
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  MS_HIP(hipStreamIsCapturing(st, &capturing));
  if (capturing == hipStreamCaptureStatusNone) {
    if (sa->used && sa->last_stream != st) MS_HIP(hipDeviceSynchronize());
    sa->last_stream = st;
    sa->used = true;
  }
  p.ws = sa->ptr;
  p.ws_bytes = NOALLOC_SCRATCH_BYTES;
  // the array keeps what the last call left: the counters must start at zero (a fill kernel, so that the call can be captured)
  hipLaunchKernelGGL(ws_clear_kernel, dim3(WS_COUNTERS / 256), dim3(256), 0, st, static_cast<int *>(sa->ptr), WS_COUNTERS);
  MS_HIP(hipGetLastError());
  return run(p, stream);
}

MS_API int ms_gemm_ls(const void *A, int lda, const void *const *W_slices, int ldw, int S, int m, int n_slice, int k,
                      float *const *Y_chunks, int ldy, int in_dtype, void *stream) {
  const void *a1[1] = {A};
  return run(make_ls(a1, lda, W_slices, ldw, S, m, n_slice, k, (void *const *)Y_chunks, ldy, in_dtype), stream);
}

MS_API int ms_gemm_rs(const void *const *X_slices, int ldx, const void *W, int ldw, int S, int m_slice, int n, int k,
                      float *const *Y_chunks, int ldy, int in_dtype, void *stream) {
  const void *w1[1] = {W};
  return run(make_rs(X_slices, ldx, w1, ldw, S, m_slice, n, k, (void *const *)Y_chunks, ldy, in_dtype), stream);
}

MS_API int ms_gemm_ls_ex(const void *A, int lda, const void *const *W_slices, int ldw, int S, int m, int n_slice, int k,
                         void *const *Y_chunks, int ldy, int in_dtype, int out_dtype, void *stream) {
  const void *a1[1] = {A};
  return run(make_ls(a1, lda, W_slices, ldw, S, m, n_slice, k, Y_chunks, ldy, in_dtype, out_dtype), stream);
}

MS_API int ms_gemm_rs_ex(const void *const *X_slices, int ldx, const void *W, int ldw, int S, int m_slice, int n, int k,
                         void *const *Y_chunks, int ldy, int in_dtype, int out_dtype, void *stream) {
  const void *w1[1] = {W};
  return run(make_rs(X_slices, ldx, w1, ldw, S, m_slice, n, k, Y_chunks, ldy, in_dtype, out_dtype), stream);
}

// the chunk-producing calls with completion counters
namespace {
int run_signal(Problem p, unsigned *chunk_done, int *tiles_per_chunk, void *stream, const char *fn) {
  if (!chunk_done || !tiles_per_chunk) return fail(MS_ERR_ARG, "%s: null chunk_done / tiles_per_chunk", fn);
  if (reinterpret_cast<uintptr_t>(chunk_done) & 3) return fail(MS_ERR_ARG, "%s: chunk_done must be 4-byte aligned", fn);
  p.chunk_done = chunk_done;
  const int rc = run(p, stream);
  if (rc == MS_OK) *tiles_per_chunk = g_last_tiles_per_chunk;
  return rc;
}
}  // namespace

MS_API int ms_gemm_ls_signal(const void *A, int lda, const void *const *W_slices, int ldw, int S, int m, int n_slice, int k,
                             void *const *Y_chunks, int ldy, int in_dtype, int out_dtype,
                             unsigned *chunk_done, int *tiles_per_chunk, void *stream) {
  const void *a1[1] = {A};
  return run_signal(make_ls(a1, lda, W_slices, ldw, S, m, n_slice, k, Y_chunks, ldy, in_dtype, out_dtype), chunk_done, tiles_per_chunk, stream, "ms_gemm_ls_signal");
}

MS_API int ms_gemm_rs_signal(const void *const *X_slices, int ldx, const void *W, int ldw, int S, int m_slice, int n, int k,
                             void *const *Y_chunks, int ldy, int in_dtype, int out_dtype,
                             unsigned *chunk_done, int *tiles_per_chunk, void *stream) {
  const void *w1[1] = {W};
  return run_signal(make_rs(X_slices, ldx, w1, ldw, S, m_slice, n, k, Y_chunks, ldy, in_dtype, out_dtype), chunk_done, tiles_per_chunk, stream, "ms_gemm_rs_signal");
}

// the chunk-producing calls behind the input gate; the completion counters are optional here
namespace {
int run_chunks_gated(Problem p, unsigned *chunk_done, int *tiles_per_chunk, unsigned *slice_ready, unsigned timeout_ms, void *stream, const char *fn) {
  if ((chunk_done == nullptr) != (tiles_per_chunk == nullptr)) return fail(MS_ERR_ARG, "%s: chunk_done and tiles_per_chunk come together or not at all", fn);
  const int rc = set_gate(p, slice_ready, timeout_ms, fn);
  if (rc) return rc;
  return chunk_done ? run_signal(p, chunk_done, tiles_per_chunk, stream, fn) : run(p, stream);
}
}  // namespace

MS_API int ms_gemm_ls_gated(const void *A, int lda, const void *const *W_slices, int ldw, int S, int m, int n_slice, int k,
                            void *const *Y_chunks, int ldy, int in_dtype, int out_dtype,
                            unsigned *chunk_done, int *tiles_per_chunk, unsigned *slice_ready, unsigned timeout_ms, void *stream) {
  const void *a1[1] = {A};
  return run_chunks_gated(make_ls(a1, lda, W_slices, ldw, S, m, n_slice, k, Y_chunks, ldy, in_dtype, out_dtype), chunk_done, tiles_per_chunk,
                          slice_ready, timeout_ms, stream, "ms_gemm_ls_gated");
}

MS_API int ms_gemm_rs_gated(const void *const *X_slices, int ldx, const void *W, int ldw, int S, int m_slice, int n, int k,
                            void *const *Y_chunks, int ldy, int in_dtype, int out_dtype,
                            unsigned *chunk_done, int *tiles_per_chunk, unsigned *slice_ready, unsigned timeout_ms, void *stream) {
  const void *w1[1] = {W};
  return run_chunks_gated(make_rs(X_slices, ldx, w1, ldw, S, m_slice, n, k, Y_chunks, ldy, in_dtype, out_dtype), chunk_done, tiles_per_chunk,
                          slice_ready, timeout_ms, stream, "ms_gemm_rs_gated");
}

MS_API int ms_time_os(const void *const *A_slices, const void *const *B_slices, int S, int m, int n, int k_slice,
                      int lda, int ldb, void *C, int ldc, int in_dtype, int out_dtype, void *stream,
                      int warmup, int reps, float *ms_out) {
  void *c1[1] = {C};
  return timed(make_os(A_slices, B_slices, S, m, n, k_slice, lda, ldb, c1, ldc, in_dtype, out_dtype), stream, warmup, reps, ms_out);
}

MS_API int ms_time_os_ws(const void *const *A_slices, const void *const *B_slices, int S, int m, int n, int k_slice,
                         int lda, int ldb, void *C, int ldc, int in_dtype, int out_dtype,
                         void *workspace, size_t workspace_bytes, void *stream, int warmup, int reps, float *ms_out) {
  void *c1[1] = {C};
  Problem p = make_os(A_slices, B_slices, S, m, n, k_slice, lda, ldb, c1, ldc, in_dtype, out_dtype);
  p.ws = workspace; p.ws_bytes = workspace ? workspace_bytes : 0;
  return timed(p, stream, warmup, reps, ms_out);
}

MS_API int ms_time_ls_ex(const void *A, int lda, const void *const *W_slices, int ldw, int S, int m, int n_slice, int k,
                         void *const *Y_chunks, int ldy, int in_dtype, int out_dtype, void *stream,
                         int warmup, int reps, float *ms_out) {
  const void *a1[1] = {A};
  return timed(make_ls(a1, lda, W_slices, ldw, S, m, n_slice, k, Y_chunks, ldy, in_dtype, out_dtype), stream, warmup, reps, ms_out);
}

MS_API int ms_time_rs_ex(const void *const *X_slices, int ldx, const void *W, int ldw, int S, int m_slice, int n, int k,
                         void *const *Y_chunks, int ldy, int in_dtype, int out_dtype, void *stream,
                         int warmup, int reps, float *ms_out) {
  const void *w1[1] = {W};
  return timed(make_rs(X_slices, ldx, w1, ldw, S, m_slice, n, k, Y_chunks, ldy, in_dtype, out_dtype), stream, warmup, reps, ms_out);
}

MS_API int ms_time_ls(const void *A, int lda, const void *const *W_slices, int ldw, int S, int m, int n_slice, int k,
                      float *const *Y_chunks, int ldy, int in_dtype, void *stream, int warmup, int reps, float *ms_out) {
  return ms_time_ls_ex(A, lda, W_slices, ldw, S, m, n_slice, k, (void *const *)Y_chunks, ldy, in_dtype, MS_DTYPE_F32, stream, warmup, reps, ms_out);
}

MS_API int ms_time_rs(const void *const *X_slices, int ldx, const void *W, int ldw, int S, int m_slice, int n, int k,
                      float *const *Y_chunks, int ldy, int in_dtype, void *stream, int warmup, int reps, float *ms_out) {
  return ms_time_rs_ex(X_slices, ldx, W, ldw, S, m_slice, n, k, (void *const *)Y_chunks, ldy, in_dtype, MS_DTYPE_F32, stream, warmup, reps, ms_out);
}
