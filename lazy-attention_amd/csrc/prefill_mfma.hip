#include "common.hpp"
namespace lazyattn {
bool mfma_supports(const lazyattn_prefill_params &) { return false; }
size_t mfma_workspace_bytes(const lazyattn_prefill_params &) { return 0; }
int launch_prefill_mfma(const lazyattn_prefill_params &, hipStream_t) { return LAZYATTN_E_UNSUPPORTED; }
}
