// Kernel instantiations for double storage (fp64 arithmetic).
#include "scan_launch.hpp"

namespace scanscam {
SCANSCAM_DEFINE_LAUNCH(double)
SCANSCAM_DEFINE_CL_LAUNCH(double)
SCANSCAM_DEFINE_FLAT_LAUNCH(double)
}  // namespace scanscam
