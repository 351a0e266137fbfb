// Skinny-M (decode-shaped) MXFP6 GEMM -- placeholder translation unit until the streaming kernel lands.
#include "common.hpp"
#include "kernels.hpp"
namespace mxfp6 {
bool gemm_skinny_supports(const GemmArgs&) { return false; }
hipError_t launch_gemm_skinny(const GemmArgs&, hipStream_t) { return hipErrorNotSupported; }
}  // namespace mxfp6
