// MFMA tile GEMM for prefill-sized linears (M > 16).  Filled in by mfma_gemm(); until a shape is
// supported the caller falls back to the LDS-tiled FMA kernel in kernels_linear.hip.
#include "kernels.hpp"
#include "device_utils.hpp"

namespace gptrs {
namespace k {

bool mfma_gemm_supported(int, int64_t, int64_t, int64_t) { return false; }
void mfma_gemm(hipStream_t, int, const void*, const void*, const void*, const void*, void*, int64_t, int64_t, int64_t, int) {}

}  // namespace k
}  // namespace gptrs
