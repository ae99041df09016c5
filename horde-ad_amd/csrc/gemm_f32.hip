// Instantiates the matrix-product kernel for one MFMA flavour (see gemm_kernel.hpp).
#include "gemm_kernel.hpp"

namespace hg {
namespace gemm {
void launch_f32(const GemmParams& p, const LaunchArgs& a) { launch<MfmaF32>(p, a); }
}  // namespace gemm
}  // namespace hg
