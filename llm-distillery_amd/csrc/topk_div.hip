// dl_div_topk, dl_div_topk_static: forward / reverse KL against one sparse (top-K) teacher.
// The kernels live in topk_div.hpp.
#include "topk_div.hpp"
#include <mutex>

extern "C" int64_t dl_div_topk_workspace_bytes(int kind, int logits_dtype, int64_t n_rows, int64_t V) {
  if (kind != DL_FKL || n_rows <= 0 || V <= 0) return 0;
  const int epc = logits_dtype == DL_F32 ? 4 : 8;
  const int64_t nch = (V + epc - 1) / epc;      // a row that ends inside a chunk holds that chunk too
  if (nch <= 256 * 16 || nch > (int64_t)dl::MAX_COARSE_PARTS * 256 * 16) return 0;
  // up to 512 x 16 chunks only rows that cannot lie on the 16-byte grid are cut (in two)
  if (nch <= 512 * 16) return V % epc != 0 ? dl::RetryList::bytes(n_rows, 2) : 0;
  return dl::RetryList::bytes(n_rows, nch <= 1024 * 16 ? 4 : dl::MAX_COARSE_PARTS);
}

// Argument checks and dispatch shared by dl_div_topk and dl_div_topk_static.
static int div_topk_checked(int kind, const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows,
                            int64_t V, const int32_t* row_map, const void* t_val, int t_val_dtype,
                            const void* t_idx, int t_idx_itype, int K, int64_t n_teacher_rows,
                            const int32_t* t_cnt, float inv_T_student, float inv_T_teacher, float grad_scale, float* row_loss,
                            void* grad, int64_t grad_stride, void* workspace, int64_t workspace_bytes, int flags,
                            void* stream, bool launch) {
  using namespace dl;
  if (!logits || ((!t_val || !t_idx) && n_teacher_rows > 0)) return DL_ERR_NULL;      // no teacher rows: every row is masked
  if (kind != DL_FKL && kind != DL_RKL) return DL_ERR_DTYPE;
  if (logits_dtype < DL_F32 || logits_dtype > DL_F16 || t_val_dtype < DL_F32 || t_val_dtype > DL_F16 ||
      (t_idx_itype != DL_I32 && t_idx_itype != DL_I64))
    return DL_ERR_DTYPE;
  if (n_rows < 0 || V <= 0 || K <= 0 || n_teacher_rows < 0 || row_stride < V || (grad && grad_stride < V)) return DL_ERR_SHAPE;
  if (K > DL_MAX_TOPK || n_rows > 0x7fffffffLL || V > 0x7fffffffLL) return DL_ERR_LIMIT;
  if (n_rows == 0 || !launch) return DL_OK;
  const int eb = logits_dtype == DL_F32 ? 4 : 2;
  const int epc = 16 / eb;
  if (reinterpret_cast<uintptr_t>(logits) % eb != 0 || (grad && reinterpret_cast<uintptr_t>(grad) % eb != 0)) return DL_ERR_ALIGN;
  const bool on_grid = (reinterpret_cast<uintptr_t>(logits) % 16 == 0) && ((row_stride * eb) % 16 == 0) &&
                       (!grad || (reinterpret_cast<uintptr_t>(grad) % 16 == 0 && (grad_stride * eb) % 16 == 0));
  const bool aligned = on_grid && V % epc == 0;
  TopkParams p{logits, row_stride, n_rows, V, row_map, t_val, t_val_dtype, t_idx, t_idx_itype, K, n_teacher_rows,
               t_cnt, inv_T_student, inv_T_teacher, grad_scale, row_loss, grad, grad_stride,
               (reinterpret_cast<uintptr_t>(workspace) % 16 == 0) ? workspace : nullptr, 1,
               (flags & DL_TOPK_NO_WAIT) ? 0 : SPIN_LIMIT, flags};
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (kind == DL_FKL && on_grid && !aligned) return launch_fkl_tail(logits_dtype, p, workspace_bytes, st);
  if (kind == DL_FKL)
    return logits_dtype == DL_F32 ? launch_fkl<TagF32, false>(p, aligned, workspace_bytes, st)
           : logits_dtype == DL_BF16 ? launch_fkl<TagBF16, false>(p, aligned, workspace_bytes, st)
                                     : launch_fkl<TagF16, false>(p, aligned, workspace_bytes, st);
  const hipError_t e = logits_dtype == DL_F32 ? launch_rkl<TagF32>(p, aligned, st)
                       : logits_dtype == DL_BF16 ? launch_rkl<TagBF16>(p, aligned, st)
                                                 : launch_rkl<TagF16>(p, aligned, st);
  return e == hipSuccess ? DL_OK : DL_ERR_LAUNCH;
}

extern "C" int dl_div_topk(int kind, const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows,
                           int64_t V, const int32_t* row_map, const void* t_val, int t_val_dtype,
                           const void* t_idx, int t_idx_itype, int K, int64_t n_teacher_rows,
                           const int32_t* t_cnt, float inv_T_student, float inv_T_teacher, float grad_scale, float* row_loss,
                           void* grad, int64_t grad_stride, void* workspace, int64_t workspace_bytes, int flags,
                           void* stream) {
  return div_topk_checked(kind, logits, logits_dtype, row_stride, n_rows, V, row_map, t_val, t_val_dtype, t_idx,
                          t_idx_itype, K, n_teacher_rows, t_cnt, inv_T_student, inv_T_teacher, grad_scale, row_loss,
                          grad, grad_stride, workspace, workspace_bytes, flags, stream, true);
}

// ---------------------------------------------------------------------------------------
// dl_div_topk_static: the same launches with the split-row workspace in a static device array
// instead of caller memory, for callers that cannot allocate.
// ---------------------------------------------------------------------------------------
// Every GPU the library runs on holds its own copy of this array until the process ends.  In host
// code the name is only a handle: the array's device address comes from hipGetSymbolAddress, once
// per device, and that pointer is what the kernels receive.
static __device__ __align__(256) unsigned char scratch[DL_STATIC_SCRATCH_BYTES];

namespace dl {
constexpr int MAX_DEVICES = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[MAX_DEVICES];      // per device, filled on the first call with that device current

// Device address of `scratch` on the current device; no allocation, one symbol lookup per device.
static int static_scratch(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return DL_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return DL_ERR_LAUNCH;
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return DL_OK;
}
}  // namespace dl

extern "C" int dl_div_topk_static(int kind, const void* logits, int logits_dtype, int64_t row_stride, int64_t n_rows,
                                  int64_t V, const int32_t* row_map, const void* t_val, int t_val_dtype,
                                  const void* t_idx, int t_idx_itype, int K, int64_t n_teacher_rows,
                                  const int32_t* t_cnt, float inv_T_student, float inv_T_teacher, float grad_scale,
                                  float* row_loss, void* grad, int64_t grad_stride, int flags, void* stream) {
  // argument checks first, then the size against the array: both before anything touches the GPU
  const int st = div_topk_checked(kind, logits, logits_dtype, row_stride, n_rows, V, row_map, t_val, t_val_dtype, t_idx,
                                  t_idx_itype, K, n_teacher_rows, t_cnt, inv_T_student, inv_T_teacher, grad_scale,
                                  row_loss, grad, grad_stride, nullptr, 0, flags, stream, false);
  if (st != DL_OK || n_rows == 0) return st;
  const int64_t need = dl_div_topk_workspace_bytes(kind, logits_dtype, n_rows, V);
  if (need > (int64_t)DL_STATIC_SCRATCH_BYTES) return DL_ERR_SCRATCH;
  void* ws = nullptr;
  if (need > 0) {
    const int got = dl::static_scratch(&ws);
    if (got != DL_OK) return got;
  }
  // launch_split clears the records and the retry counter it is about to use with a fill kernel of
  // its own (no memset node), so what the previous call left in the array does not matter.
  return div_topk_checked(kind, logits, logits_dtype, row_stride, n_rows, V, row_map, t_val, t_val_dtype, t_idx,
                          t_idx_itype, K, n_teacher_rows, t_cnt, inv_T_student, inv_T_teacher, grad_scale, row_loss,
                          grad, grad_stride, ws, ws ? (int64_t)DL_STATIC_SCRATCH_BYTES : 0, flags, stream, true);
}
