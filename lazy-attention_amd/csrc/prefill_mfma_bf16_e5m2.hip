// Matrix-core prefill kernels for bf16 operands and fp8 e5m2 cache pages.
#include "prefill_mfma_kernel.hpp"

namespace lazyattn {
template int launch_mfma_family<bf16_t, 2>(const lazyattn_prefill_params &, int, int, int, const BatchShape &, hipStream_t);
}  // namespace lazyattn
