// Matrix-core kernel of gated sliding-window attention for bf16 prompt portions (see mixers_attn.hip for the mechanism).
#include "mixers_common.h"

namespace gbxm {

int launch_window_tiles(const gbxm_window_attn_args& a, hipStream_t s) {
  (void)a; (void)s;
  return GBXM_ERR_UNSUPPORTED;
}

}  // namespace gbxm
