// The one-launch forward kernel (forward_single.hpp) for one row length: compiled once per
// -DPM_FS_NMMA=1 .. 16 (rows of 256 PM_FS_NMMA bf16 values), see forward_single_launch.hpp.
#include "forward_shared.hpp"
#include "forward_single_launch.hpp"

#ifndef PM_FS_NMMA
#error "compile with -DPM_FS_NMMA=1 .. 16"
#endif

namespace pm {
#define PM_FS_DEFINE_(n) PM_FS_DEFINE(n)
PM_FS_DEFINE_(PM_FS_NMMA)
} // namespace pm
