// Kernel instantiations for __bf16 storage (fp32 arithmetic).
#include "scan_launch.hpp"

namespace scanscam {
SCANSCAM_DEFINE_LAUNCH(__bf16)
SCANSCAM_DEFINE_CL_LAUNCH(__bf16)
SCANSCAM_DEFINE_FLAT_LAUNCH(__bf16)
}  // namespace scanscam
