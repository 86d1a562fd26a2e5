#include "bcattn_common.h"
namespace bcattn {
int launch_fwd_f32(const FwdArgs &, int, hipStream_t) { return BCATTN_ERR_UNSUPPORTED; }
int launch_bwd_bf16(const BwdArgs &, int, hipStream_t) { return BCATTN_ERR_UNSUPPORTED; }
int launch_bwd_f32(const BwdArgs &, int, hipStream_t) { return BCATTN_ERR_UNSUPPORTED; }
int launch_fwd_kvcache_bf16(const FwdArgs &, const SplitArgs &, int, hipStream_t) { return BCATTN_ERR_UNSUPPORTED; }
size_t kvcache_workspace_bytes(int, int, int, int, int, int, int *ns) { *ns = 1; return 0; }
}
