// Kernel instantiations for float storage (fp32 arithmetic).
#include "scan_launch.hpp"

namespace scanscam {
SCANSCAM_DEFINE_LAUNCH(float)
SCANSCAM_DEFINE_CL_LAUNCH(float)
SCANSCAM_DEFINE_FLAT_LAUNCH(float)
}  // namespace scanscam
