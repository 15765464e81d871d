// libmeshslice_hip.so — C ABI over the block-cyclic layout kernels (declarations: include/meshslice_hip.h).
#include <hip/hip_runtime.h>

#include <cstdint>

#include "ms_common.hip.inc"

#include "ms_layout.hip.inc"

namespace {

using msi::fail;

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int elem_bytes(int dtype) { return dtype == MS_DTYPE_BF16 ? 2 : dtype == MS_DTYPE_F32 ? 4 : 0; }

// Threads along the row: the smallest of 64 / 128 / 256 that covers it.
int pick_tx(int ucols) { return ucols <= 64 ? 64 : ucols <= 128 ? 128 : 256; }

// Distance between consecutive table entries if it is the same (and not zero) for all of them, else 0.
long long table_stride(const void *const *tab, int n) {
  if (n < 2) return 0;
  const long long d = (long long)(reinterpret_cast<intptr_t>(tab[1]) - reinterpret_cast<intptr_t>(tab[0]));
  for (int i = 2; i < n; i++)
    if ((long long)(reinterpret_cast<intptr_t>(tab[i]) - reinterpret_cast<intptr_t>(tab[i - 1])) != d) return 0;
  return d;
}

int grid_for(int rows, int ucols, int tx, dim3 *g, const char *fn) {
  const int rows_per_block = (256 / tx) * msk::LAYOUT_RT;
  const long long gy = ((long long)rows + rows_per_block - 1) / rows_per_block;
  if (gy > 65535) return fail(MS_ERR_UNSUPPORTED, "%s: %d rows exceed one launch", fn, rows);
  *g = dim3((unsigned)((ucols + tx - 1) / tx), (unsigned)gy, 1);
  return MS_OK;
}

template <int UB>
int launch_pack(int axis, int tx, dim3 g, hipStream_t st, const msk::PackArgs &a) {
#define MS_PACK(TX)                                                                                  \
  if (tx == TX) {                                                                                    \
    if (axis == 1) hipLaunchKernelGGL((msk::pack_cols_kernel<UB, TX>), g, dim3(256), 0, st, a);      \
    else hipLaunchKernelGGL((msk::pack_rows_kernel<UB, TX>), g, dim3(256), 0, st, a);                \
  }
  MS_PACK(64) MS_PACK(128) MS_PACK(256)
#undef MS_PACK
  MS_HIP(hipGetLastError());
  return MS_OK;
}

template <typename TIN, typename TOUT, int VEC>
int launch_unpack(int axis, int tx, dim3 g, hipStream_t st, const msk::UnpackArgs &a) {
#define MS_UNPACK(TX)                                                                                          \
  if (tx == TX) {                                                                                              \
    if (axis == 1) hipLaunchKernelGGL((msk::unpack_cols_kernel<TIN, TOUT, VEC, TX>), g, dim3(256), 0, st, a);  \
    else hipLaunchKernelGGL((msk::unpack_rows_kernel<TIN, TOUT, VEC, TX>), g, dim3(256), 0, st, a);            \
  }
  MS_UNPACK(64) MS_UNPACK(128) MS_UNPACK(256)
#undef MS_UNPACK
  MS_HIP(hipGetLastError());
  return MS_OK;
}

template <int VEC>
int launch_unpack_typed(int in_dtype, int out_dtype, int axis, int tx, dim3 g, hipStream_t st, const msk::UnpackArgs &a) {
  typedef unsigned short bf16_bits;
  if (in_dtype == MS_DTYPE_F32)
    return out_dtype == MS_DTYPE_F32 ? launch_unpack<float, float, VEC>(axis, tx, g, st, a) : launch_unpack<float, bf16_bits, VEC>(axis, tx, g, st, a);
  return out_dtype == MS_DTYPE_F32 ? launch_unpack<bf16_bits, float, VEC>(axis, tx, g, st, a) : launch_unpack<bf16_bits, bf16_bits, VEC>(axis, tx, g, st, a);
}

}  // namespace

MS_API int ms_pack_slices(const void *src, int ld_src, int rows, int cols, int axis, int S, int B,
                          void *const *dst_slices, int ld_dst, int dtype, void *stream) {
  const char *fn = "ms_pack_slices";
  const int es = elem_bytes(dtype);
  if (!es) return fail(MS_ERR_UNSUPPORTED, "%s: unknown dtype %d", fn, dtype);
  if (axis != 0 && axis != 1) return fail(MS_ERR_ARG, "%s: axis must be 0 (rows) or 1 (columns), got %d", fn, axis);
  if (S < 1 || S > MS_MAX_SLICES) return fail(MS_ERR_ARG, "%s: S = %d outside [1, %d]", fn, S, MS_MAX_SLICES);
  if (B < 1 || rows <= 0 || cols <= 0) return fail(MS_ERR_ARG, "%s: non-positive extent (rows=%d cols=%d B=%d)", fn, rows, cols, B);
  if (!src || !dst_slices) return fail(MS_ERR_ARG, "%s: null pointer", fn);
  const int sliced = axis == 1 ? cols : rows;
  if (sliced % ((long long)S * B)) return fail(MS_ERR_ARG, "%s: sliced extent %d is not a multiple of S*B = %d*%d", fn, sliced, S, B);
  const int dcols = axis == 1 ? cols / S : cols;
  if (ld_src < cols || ld_dst < dcols) return fail(MS_ERR_ARG, "%s: leading dimension smaller than the row length", fn);
  bool wide = aligned16(src) && ((long long)cols * es) % 16 == 0 && ((long long)ld_src * es) % 16 == 0 && ((long long)ld_dst * es) % 16 == 0 &&
              (axis == 0 || (B * es) % 16 == 0);
  for (int s = 0; s < S; s++) {
    if (!dst_slices[s]) return fail(MS_ERR_ARG, "%s: slice pointer %d is null", fn, s);
    if (reinterpret_cast<uintptr_t>(dst_slices[s]) % es) return fail(MS_ERR_ARG, "%s: slice pointer %d is not aligned to the element size", fn, s);
    wide = wide && aligned16(dst_slices[s]);
  }
  if (reinterpret_cast<uintptr_t>(src) % es) return fail(MS_ERR_ARG, "%s: source pointer is not aligned to the element size", fn);
  const int ub = wide ? 16 : es;
  msk::PackArgs a;
  a.src = src;
  for (int s = 0; s < S; s++) a.dst[s] = dst_slices[s];
  a.rows = rows;
  a.ucols = (int)((long long)cols * es / ub);
  a.ld_src = (int)((long long)ld_src * es / ub);
  a.ld_dst = (int)((long long)ld_dst * es / ub);
  a.S = S;
  a.G = axis == 1 ? B * es / ub : B;
  a.tab_stride = table_stride(dst_slices, S);
  const int tx = pick_tx(a.ucols);
  dim3 g;
  if (int rc = grid_for(rows, a.ucols, tx, &g, fn)) return rc;
  hipStream_t st = (hipStream_t)stream;
  return ub == 16 ? launch_pack<16>(axis, tx, g, st, a) : ub == 4 ? launch_pack<4>(axis, tx, g, st, a) : launch_pack<2>(axis, tx, g, st, a);
}

MS_API int ms_unpack_chunks(const void *const *chunks, int P, int S, int ld_chunk, int row_off, int col_off,
                            int rows, int cols, int axis, int B, void *out, int ld_out,
                            int in_dtype, int out_dtype, void *stream) {
  const char *fn = "ms_unpack_chunks";
  const int esi = elem_bytes(in_dtype), eso = elem_bytes(out_dtype);
  if (!esi || !eso) return fail(MS_ERR_UNSUPPORTED, "%s: unknown dtype (%d, %d)", fn, in_dtype, out_dtype);
  if (axis != 0 && axis != 1) return fail(MS_ERR_ARG, "%s: axis must be 0 (rows) or 1 (columns), got %d", fn, axis);
  if (S < 1 || P < 1 || (long long)P * S > msk::LAYOUT_MAX_PTRS) return fail(MS_ERR_ARG, "%s: P*S = %d*%d outside [1, %d]", fn, P, S, msk::LAYOUT_MAX_PTRS);
  if (B < 1 || rows <= 0 || cols <= 0) return fail(MS_ERR_ARG, "%s: non-positive extent (rows=%d cols=%d B=%d)", fn, rows, cols, B);
  if (row_off < 0 || col_off < 0) return fail(MS_ERR_ARG, "%s: negative window offset", fn);
  if (!chunks || !out) return fail(MS_ERR_ARG, "%s: null pointer", fn);
  const int sliced = axis == 1 ? cols : rows;
  if (sliced % ((long long)S * B)) return fail(MS_ERR_ARG, "%s: interleaved extent %d is not a multiple of S*B = %d*%d", fn, sliced, S, B);
  const int wcols = axis == 1 ? cols / S : cols;  // columns of the window kept from each chunk
  if ((long long)col_off + wcols > ld_chunk || ld_out < cols) return fail(MS_ERR_ARG, "%s: leading dimension smaller than the row length", fn);
  bool wide = aligned16(out) && cols % 8 == 0 && col_off % 8 == 0 && ld_chunk % 8 == 0 && ld_out % 8 == 0 && (axis == 0 || B % 8 == 0);
  if (reinterpret_cast<uintptr_t>(out) % eso) return fail(MS_ERR_ARG, "%s: output pointer is not aligned to the element size", fn);
  msk::UnpackArgs a;
  for (int i = 0; i < P * S; i++) {
    if (!chunks[i]) return fail(MS_ERR_ARG, "%s: chunk pointer %d is null", fn, i);
    if (reinterpret_cast<uintptr_t>(chunks[i]) % esi) return fail(MS_ERR_ARG, "%s: chunk pointer %d is not aligned to the element size", fn, i);
    wide = wide && aligned16(chunks[i]);
    a.src[i] = chunks[i];
  }
  a.dst = out;
  a.rows = rows;
  // eight elements per thread, or the four of one 16-byte unit when fp32 chunks of one peer are only moved
  const bool move_f32 = wide && P == 1 && in_dtype == MS_DTYPE_F32 && out_dtype == MS_DTYPE_F32;
  const int vec = !wide ? 1 : move_f32 ? 4 : 8;
  a.ucols = cols / vec;
  a.ld_src = ld_chunk;
  a.ld_dst = ld_out;
  a.row_off = row_off;
  a.col_off = col_off;
  a.P = P;
  a.S = S;
  a.B = B;
  a.tab_stride = table_stride(chunks, P * S);
  const int tx = pick_tx(a.ucols);
  dim3 g;
  if (int rc = grid_for(rows, a.ucols, tx, &g, fn)) return rc;
  hipStream_t st = (hipStream_t)stream;
  if (move_f32) return launch_unpack<float, float, 4>(axis, tx, g, st, a);
  return wide ? launch_unpack_typed<8>(in_dtype, out_dtype, axis, tx, g, st, a) : launch_unpack_typed<1>(in_dtype, out_dtype, axis, tx, g, st, a);
}
