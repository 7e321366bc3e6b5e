// Forward KL against one sparse teacher on rows that lie on the 16-byte grid but end inside a chunk
// (logits[:, :, :crop] of a padded vocabulary): the ROWS_TAIL instantiations of the kernels in topk_div.hpp.
#include "topk_div.hpp"

namespace dl {
int launch_fkl_tail(int logits_dtype, const TopkParams& p, int64_t ws_bytes, hipStream_t st) {
  return logits_dtype == DL_F32 ? launch_fkl<TagF32, false, ROWS_TAIL>(p, true, ws_bytes, st)
         : logits_dtype == DL_BF16 ? launch_fkl<TagBF16, false, ROWS_TAIL>(p, true, ws_bytes, st)
                                   : launch_fkl<TagF16, false, ROWS_TAIL>(p, true, ws_bytes, st);
}
}  // namespace dl
