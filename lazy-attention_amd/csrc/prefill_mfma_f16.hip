// Matrix-core prefill kernels for float16 operands and cache pages of the same type.
#include "prefill_mfma_kernel.hpp"

namespace lazyattn {
template int launch_mfma_family<f16_t, 0>(const lazyattn_prefill_params &, int, int, int, const BatchShape &, hipStream_t);
}  // namespace lazyattn
