// Grouped matrix-core products of routed experts for bf16 prompt portions (see mixers_moe.hip).
#include "mixers_common.h"

namespace gbxm {

size_t expert_grouped_workspace(int64_t T, int K, int F, int E, int top) {
  (void)T; (void)K; (void)F; (void)E; (void)top;
  return 0;
}

int launch_expert_grouped(const void* h, const void* gate_up, const void* down, const int32_t* idx, void* y, int64_t T, int K, int F, int E, int top,
                          void* ws, size_t ws_bytes, hipStream_t s) {
  (void)h; (void)gate_up; (void)down; (void)idx; (void)y; (void)T; (void)K; (void)F; (void)E; (void)top; (void)ws; (void)ws_bytes; (void)s;
  return GBXM_ERR_UNSUPPORTED;
}

}  // namespace gbxm
