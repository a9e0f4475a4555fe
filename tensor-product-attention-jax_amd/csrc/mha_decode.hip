// Dense multi-head attention for few query tokens over a long dense K/V cache (placeholder
// until the split-key kernel lands: reports "not supported" so mha_fwd uses the other kernels).
#include "tpa_common.h"

int mha_decode_supported(const MhaFwdArgs*) { return 0; }
int mha_decode_launch(const MhaFwdArgs*, hipStream_t) { return TPA_ERR_UNSUPPORTED; }
extern "C" size_t mha_fwd_workspace_bytes(int32_t, int32_t, int32_t, int32_t, int32_t, int32_t) { return 0; }
