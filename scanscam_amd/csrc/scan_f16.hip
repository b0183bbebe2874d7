// Kernel instantiations for _Float16 storage (fp32 arithmetic).
#include "scan_launch.hpp"

namespace scanscam {
SCANSCAM_DEFINE_LAUNCH(_Float16)
SCANSCAM_DEFINE_CL_LAUNCH(_Float16)
SCANSCAM_DEFINE_FLAT_LAUNCH(_Float16)
}  // namespace scanscam
