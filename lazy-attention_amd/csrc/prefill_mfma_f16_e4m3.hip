// Matrix-core prefill kernels for float16 operands and fp8 e4m3 cache pages.
#include "prefill_mfma_kernel.hpp"

namespace lazyattn {
template int launch_mfma_family<f16_t, 1>(const lazyattn_prefill_params &, int, int, int, const BatchShape &, hipStream_t);
}  // namespace lazyattn
