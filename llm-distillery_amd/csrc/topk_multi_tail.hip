// Forward KL against several prepared teachers on rows that lie on the 16-byte grid but end inside a chunk:
// the ROWS_TAIL instantiations of the kernels in topk_div.hpp (see topk_multi.hip for the entry point).
#include "topk_div.hpp"

namespace dl {
int launch_fkl_tail_multi(int logits_dtype, const TopkParams& p, int64_t ws_bytes, hipStream_t st, bool ws_cleared) {
  return logits_dtype == DL_F32 ? launch_fkl<TagF32, true, ROWS_TAIL>(p, true, ws_bytes, st, ws_cleared)
         : logits_dtype == DL_BF16 ? launch_fkl<TagBF16, true, ROWS_TAIL>(p, true, ws_bytes, st, ws_cleared)
                                   : launch_fkl<TagF16, true, ROWS_TAIL>(p, true, ws_bytes, st, ws_cleared);
}
}  // namespace dl
