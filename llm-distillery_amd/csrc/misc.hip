// ABI revision, status strings and the deterministic scalar reduction.
#include "distill_common.hpp"
#include "distill_hip.h"

namespace dl {

// One workgroup, fixed association order: thread t adds values t, t+NT, ... in double (eight loads
// in flight at a time), then the lanes of a wave fold by shuffles and thread 0 adds the waves' sums
// in order.  Same input => same bits.
template <int NT>
__global__ __launch_bounds__(NT) void reduce_sum_kernel(const float* v, int64_t n, float scale, float* out) {
  __shared__ double sh[NT / WAVE];
  double acc = 0.0;
  int64_t i = threadIdx.x;
  for (; i + 7 * NT < n; i += 8 * NT) {
    float x[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) x[k] = v[i + k * NT];
#pragma unroll
    for (int k = 0; k < 8; ++k) acc += (double)x[k];
  }
  for (; i < n; i += NT) acc += (double)v[i];
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) acc += __shfl_down(acc, o, WAVE);
  if ((threadIdx.x & (WAVE - 1)) == 0) sh[threadIdx.x / WAVE] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    double total = 0.0;
#pragma unroll
    for (int w = 0; w < NT / WAVE; ++w) total += sh[w];
    out[0] = (float)(total * (double)scale);
  }
}


// Plain streaming copy, 16 bytes per thread per step.  It is the yardstick for the HBM
// counters: its traffic is known exactly (n16*16 bytes read, n16*16 bytes written).
__global__ __launch_bounds__(256) void copy16_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
    __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// Copy of [n_rows, row_chunks] 16-byte chunks in the access shape of the row kernels: a row is cut into
// column parts of NT x NCH chunks, one workgroup per part; every thread issues all its loads, then
// all its stores.  ONE_XCD: the parts of a row sit 8 workgroup ids apart (ids are dealt round-robin to
// the 8 XCDs, so they run on one XCD back to back), as in the split loss kernels; else row-major.
// WAVE_MAJOR: ChunkMap<NT, NCH> (every wave owns NCH KiB in one piece) instead of the striped
// ChunkMap<NT, 0>.  Dynamic LDS is only asked for to bound the workgroups a CU holds.
template <int NT, int NCH, bool ONE_XCD, bool WAVE_MAJOR>
__global__ __launch_bounds__(NT) void copy_rows_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                       int64_t row_chunks, int64_t n_rows, int P) {
  using M = ChunkMap<NT, WAVE_MAJOR ? NCH : 0>;
  int64_t r;
  int h;
  if (ONE_XCD) {
    const unsigned grp = blockIdx.x / (8u * P), t = blockIdx.x % (8u * P);
    r = (int64_t)grp * 8 + (t & 7u);
    h = (int)(t >> 3);
  } else {
    r = blockIdx.x / P;
    h = (int)(blockIdx.x % P);
  }
  if (r >= n_rows) return;
  const int64_t c0 = (int64_t)h * NT * NCH;
  const int64_t nch = min((int64_t)NT * NCH, row_chunks - c0);
  const u32x4* s = src + r * row_chunks + c0;
  u32x4* d = dst + r * row_chunks + c0;
  u32x4 v[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int64_t c = M::chunk(i, threadIdx.x);
    if (c < nch) v[i] = __builtin_nontemporal_load(s + c);
  }
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int64_t c = M::chunk(i, threadIdx.x);
    if (c < nch) __builtin_nontemporal_store(v[i], d + c);
  }
}

template <int NT, int NCH>
static int launch_copy_rows(const void* src, void* dst, int64_t row_chunks, int64_t n_rows, int flags, hipStream_t st) {
  const int P = (int)((row_chunks + NT * NCH - 1) / (NT * NCH));
  const bool one_xcd = flags & DL_COPY_PARTS_ON_ONE_XCD, wave_major = flags & DL_COPY_WAVE_MAJOR;
  const size_t lds = (size_t)((flags >> DL_COPY_LDS_KB_SHIFT) & 0xff) * 1024;
  if (lds > 64 * 1024) return DL_ERR_LIMIT;
  const dim3 grid((unsigned)(one_xcd ? (n_rows + 7) / 8 * 8 * P : n_rows * P));
  const u32x4* s = reinterpret_cast<const u32x4*>(src);
  u32x4* d = reinterpret_cast<u32x4*>(dst);
#define DL_COPY_LAUNCH(X, W) hipLaunchKernelGGL((copy_rows_kernel<NT, NCH, X, W>), grid, dim3(NT), lds, st, s, d, row_chunks, n_rows, P)
  if (one_xcd && wave_major) DL_COPY_LAUNCH(true, true);
  else if (one_xcd) DL_COPY_LAUNCH(true, false);
  else if (wave_major) DL_COPY_LAUNCH(false, true);
  else DL_COPY_LAUNCH(false, false);
#undef DL_COPY_LAUNCH
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

}  // namespace dl

extern "C" int dl_abi_version(void) { return 2; }

extern "C" const char* dl_status_string(int status) {
  switch (status) {
    case DL_OK: return "ok";
    case DL_ERR_NULL: return "a required pointer is NULL";
    case DL_ERR_DTYPE: return "unknown dtype, index type or divergence kind";
    case DL_ERR_SHAPE: return "negative or inconsistent sizes";
    case DL_ERR_LIMIT: return "a size exceeds what the kernels support";
    case DL_ERR_LAUNCH: return "the HIP runtime refused the launch";
    case DL_ERR_ALIGN: return "a pointer or stride breaks an alignment rule";
    case DL_ERR_WORKSPACE: return "a required workspace is too small";
    case DL_ERR_SCRATCH: return "the problem needs more scratch than the static device array holds (use dl_div_topk with a workspace)";
    default: return "unknown status";
  }
}

extern "C" int dl_reduce_sum(const float* values, int64_t n, float scale, float* out, void* stream) {
  if (!out || (n > 0 && !values)) return DL_ERR_NULL;
  if (n < 0) return DL_ERR_SHAPE;
  hipLaunchKernelGGL((dl::reduce_sum_kernel<1024>), dim3(1), dim3(1024), 0,
                     reinterpret_cast<hipStream_t>(stream), values, n, scale, out);
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

extern "C" int dl_copy16(const void* src, void* dst, int64_t n_bytes, void* stream) {
  if (!src || !dst) return DL_ERR_NULL;
  if (n_bytes < 0 || n_bytes % 16) return DL_ERR_SHAPE;
  if (reinterpret_cast<uintptr_t>(src) % 16 || reinterpret_cast<uintptr_t>(dst) % 16) return DL_ERR_ALIGN;
  if (n_bytes == 0) return DL_OK;
  const int64_t n16 = n_bytes / 16;
  const int64_t want = (n16 + 255) / 256;
  const unsigned grid = (unsigned)(want < 256 * 64 ? want : 256 * 64);
  hipLaunchKernelGGL(dl::copy16_kernel, dim3(grid), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     reinterpret_cast<const dl::u32x4*>(src), reinterpret_cast<dl::u32x4*>(dst), n16);
  return hipGetLastError() == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

extern "C" int dl_copy_rows(const void* src, void* dst, int64_t n_rows, int64_t row_bytes, int threads, int chunks,
                            int flags, void* stream) {
  using namespace dl;
  if (!src || !dst) return DL_ERR_NULL;
  if (n_rows < 0 || row_bytes <= 0 || row_bytes % 16 != 0) return DL_ERR_SHAPE;
  if (reinterpret_cast<uintptr_t>(src) % 16 != 0 || reinterpret_cast<uintptr_t>(dst) % 16 != 0) return DL_ERR_ALIGN;
  const int64_t rc = row_bytes / 16;
  if (threads <= 0 || chunks <= 0 || n_rows > 0x7fffffffLL ||
      (rc + (int64_t)threads * chunks - 1) / ((int64_t)threads * chunks) * (n_rows + 8) > 0x7fffffffLL)
    return DL_ERR_LIMIT;
  if (n_rows == 0) return DL_OK;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
#define DL_COPY_SHAPE(NT, NCH) \
  if (threads == NT && chunks == NCH) return launch_copy_rows<NT, NCH>(src, dst, rc, n_rows, flags, st);
  DL_COPY_SHAPE(256, 2) DL_COPY_SHAPE(256, 4) DL_COPY_SHAPE(256, 8) DL_COPY_SHAPE(256, 12) DL_COPY_SHAPE(256, 16)
  DL_COPY_SHAPE(512, 4) DL_COPY_SHAPE(512, 8) DL_COPY_SHAPE(512, 16) DL_COPY_SHAPE(1024, 4) DL_COPY_SHAPE(1024, 16)
#undef DL_COPY_SHAPE
  return DL_ERR_LIMIT;
}
