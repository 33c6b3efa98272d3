// placeholder until the MFMA backward lands
#include "common.h"
namespace mi355 {
bool bwd_mfma_supported(const mi355_sdpa_bwd_params&, const char** why) { *why = "not built"; return false; }
size_t bwd_mfma_workspace(const mi355_sdpa_bwd_params&) { return 0; }
int launch_bwd_mfma(const mi355_sdpa_bwd_params&, hipStream_t) { set_error("SDPA: MFMA backward not built"); return MI355_SDPA_ERR_UNSUPPORTED; }
}
