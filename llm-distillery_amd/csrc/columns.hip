// Column gather / expansion between a full-width row and its compacted form (a fixed subset of the columns,
// ascending): what lets the fused marginal + reverse-KL kernel serve a student vocabulary far wider than the
// marginal it can hold, when the teacher -> student map only ever reaches a fraction of the student ids.
// Both are plain moves of raw 2- or 4-byte elements; every output chunk is written once, by a 16-byte store.
#include "distill_common.hpp"
#include "distill_hip.h"

namespace dl {

// dst[r, c] = src[r, cols[c]]; cols[c] < 0 (padding behind the subset): -inf.  One thread per 16-byte chunk of dst.
template <int EB>
__global__ __launch_bounds__(256) void gather_columns_kernel(const char* __restrict__ src, int64_t src_stride, int64_t n_rows,
                                                             const int32_t* __restrict__ cols, int64_t n_chunks,
                                                             char* __restrict__ dst, int64_t dst_stride, unsigned fill) {
  constexpr int N = 16 / EB;
  const int64_t r = blockIdx.y;
  const int64_t ch = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (ch >= n_chunks) return;
  const char* srow = src + r * src_stride * EB;
  int id[N];
  const int4 a = *reinterpret_cast<const int4*>(cols + ch * N);
  id[0] = a.x; id[1] = a.y; id[2] = a.z; id[3] = a.w;
  if constexpr (N == 8) {
    const int4 b = *reinterpret_cast<const int4*>(cols + ch * N + 4);
    id[4] = b.x; id[5] = b.y; id[6] = b.z; id[7] = b.w;
  }
  u32x4 v;
  if constexpr (EB == 4) {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = id[e] >= 0 ? reinterpret_cast<const unsigned*>(srow)[id[e]] : fill;
  } else {
    unsigned short h[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = id[e] >= 0 ? reinterpret_cast<const unsigned short*>(srow)[id[e]] : (unsigned short)fill;
#pragma unroll
    for (int d = 0; d < 4; ++d) v[d] = (unsigned)h[2 * d] | ((unsigned)h[2 * d + 1] << 16);
  }
  store16_stream(dst + (r * dst_stride * EB) + ch * 16, v);
}

// dst[r, j] = src[r, col_src[j]], or 0 where col_src[j] < 0 (a column outside the subset).  One thread per 16-byte chunk of dst.
template <int EB>
__global__ __launch_bounds__(256) void expand_columns_kernel(const char* __restrict__ src, int64_t src_stride, int64_t n_rows,
                                                             const int32_t* __restrict__ col_src, int64_t n_chunks,
                                                             char* __restrict__ dst, int64_t dst_stride) {
  constexpr int N = 16 / EB;
  const int64_t r = blockIdx.y;
  const int64_t ch = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (ch >= n_chunks) return;
  const char* srow = src + r * src_stride * EB;
  int id[N];
  const int4 a = *reinterpret_cast<const int4*>(col_src + ch * N);
  id[0] = a.x; id[1] = a.y; id[2] = a.z; id[3] = a.w;
  if constexpr (N == 8) {
    const int4 b = *reinterpret_cast<const int4*>(col_src + ch * N + 4);
    id[4] = b.x; id[5] = b.y; id[6] = b.z; id[7] = b.w;
  }
  u32x4 v;
  if constexpr (EB == 4) {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = id[e] >= 0 ? reinterpret_cast<const unsigned*>(srow)[id[e]] : 0u;
  } else {
    unsigned short h[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = id[e] >= 0 ? reinterpret_cast<const unsigned short*>(srow)[id[e]] : (unsigned short)0;
#pragma unroll
    for (int d = 0; d < 4; ++d) v[d] = (unsigned)h[2 * d] | ((unsigned)h[2 * d + 1] << 16);
  }
  store16_stream(dst + (r * dst_stride * EB) + ch * 16, v);
}

static bool on_grid16(const void* ptr, int64_t stride, int eb) {
  return reinterpret_cast<uintptr_t>(ptr) % 16 == 0 && (stride * eb) % 16 == 0;
}

}  // namespace dl

extern "C" int dl_gather_columns(const void* src, int dtype, int64_t src_stride, int64_t n_rows, int64_t V, const int32_t* cols,
                                 int64_t n_cols, void* dst, int64_t dst_stride, void* stream) {
  using namespace dl;
  if (!src || !cols || !dst) return DL_ERR_NULL;
  if (dtype < DL_F32 || dtype > DL_F16) return DL_ERR_DTYPE;
  if (n_rows < 0 || V <= 0 || n_cols <= 0 || src_stride < V || dst_stride < n_cols) return DL_ERR_SHAPE;
  if (n_rows > 65535) return DL_ERR_LIMIT;
  const int eb = dtype == DL_F32 ? 4 : 2;
  if (n_cols % (16 / eb) != 0 || !on_grid16(dst, dst_stride, eb) || reinterpret_cast<uintptr_t>(cols) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(src) % eb != 0)
    return DL_ERR_ALIGN;
  if (n_rows == 0) return DL_OK;
  const int64_t n_chunks = n_cols / (16 / eb);
  const dim3 grid((unsigned)((n_chunks + 255) / 256), (unsigned)n_rows);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const unsigned neg_inf = dtype == DL_F32 ? 0xff800000u : dtype == DL_BF16 ? 0xff80u : 0xfc00u;
  if (eb == 4) {
    hipLaunchKernelGGL((gather_columns_kernel<4>), grid, dim3(256), 0, st, reinterpret_cast<const char*>(src), src_stride, n_rows,
                       cols, n_chunks, reinterpret_cast<char*>(dst), dst_stride, neg_inf);
  } else {
    hipLaunchKernelGGL((gather_columns_kernel<2>), grid, dim3(256), 0, st, reinterpret_cast<const char*>(src), src_stride, n_rows,
                       cols, n_chunks, reinterpret_cast<char*>(dst), dst_stride, neg_inf);
  }
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

extern "C" int dl_expand_columns(const void* src, int dtype, int64_t src_stride, int64_t n_rows, int64_t n_cols,
                                 const int32_t* col_src, int64_t V, void* dst, int64_t dst_stride, void* stream) {
  using namespace dl;
  if (!src || !col_src || !dst) return DL_ERR_NULL;
  if (dtype < DL_F32 || dtype > DL_F16) return DL_ERR_DTYPE;
  if (n_rows < 0 || V <= 0 || n_cols <= 0 || src_stride < n_cols || dst_stride < V) return DL_ERR_SHAPE;
  if (n_rows > 65535) return DL_ERR_LIMIT;
  const int eb = dtype == DL_F32 ? 4 : 2;
  if (V % (16 / eb) != 0 || !on_grid16(dst, dst_stride, eb) || reinterpret_cast<uintptr_t>(col_src) % 16 != 0 ||
      reinterpret_cast<uintptr_t>(src) % eb != 0)
    return DL_ERR_ALIGN;
  if (n_rows == 0) return DL_OK;
  const int64_t n_chunks = V / (16 / eb);
  const dim3 grid((unsigned)((n_chunks + 255) / 256), (unsigned)n_rows);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (eb == 4) {
    hipLaunchKernelGGL((expand_columns_kernel<4>), grid, dim3(256), 0, st, reinterpret_cast<const char*>(src), src_stride, n_rows,
                       col_src, n_chunks, reinterpret_cast<char*>(dst), dst_stride);
  } else {
    hipLaunchKernelGGL((expand_columns_kernel<2>), grid, dim3(256), 0, st, reinterpret_cast<const char*>(src), src_stride, n_rows,
                       col_src, n_chunks, reinterpret_cast<char*>(dst), dst_stride);
  }
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}
