// Instantiates the matrix-product kernel for one MFMA flavour (see gemm_kernel.hpp).
#include "gemm_kernel.hpp"

namespace hg {
namespace gemm {
void launch_f64(const GemmParams& p, const LaunchArgs& a) { launch<MfmaF64>(p, a); }
}  // namespace gemm
}  // namespace hg
