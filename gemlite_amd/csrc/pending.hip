// Kernel families that are not built yet report "not eligible"; the generic path runs instead.
#include "common.hpp"
#include "dispatch.hpp"
namespace gla {
bool gemv_kmajor_eligible(const gla_matmul_args&) { return false; }
int launch_gemv_kmajor(const gla_matmul_args&, hipStream_t) { return GLA_ERR_UNSUPPORTED_MODE; }
}
