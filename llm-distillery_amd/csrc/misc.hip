// ABI revision, status strings and the deterministic scalar reduction.
#include "distill_common.hpp"
#include "distill_hip.h"

namespace dl {

// One workgroup, fixed association order: thread t adds values t, t+NT, ... in double,
// then a fixed LDS tree.  Same input => same bits.
template <int NT>
__global__ __launch_bounds__(NT) void reduce_sum_kernel(const float* v, int64_t n, float scale, float* out) {
  __shared__ double sh[NT];
  double acc = 0.0;
  for (int64_t i = threadIdx.x; i < n; i += NT) acc += (double)v[i];
  sh[threadIdx.x] = acc;
  __syncthreads();
  for (int o = NT / 2; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) sh[threadIdx.x] += sh[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) out[0] = (float)(sh[0] * (double)scale);
}


// Plain streaming copy, 16 bytes per thread per step.  It is the yardstick for the HBM
// counters: its traffic is known exactly (n16*16 bytes read, n16*16 bytes written).
__global__ __launch_bounds__(256) void copy16_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ dst, int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
    __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
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
