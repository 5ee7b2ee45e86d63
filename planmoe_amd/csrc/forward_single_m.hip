// The one-launch forward kernel (forward_single.hpp) for one row length: compiled once per
// -DPM_FS_NMMA=4|8|12|16 (rows of 1024, 2048, 3072, 4096 bf16 values), see forward_single_launch.hpp.
#include "forward_shared.hpp"
#include "forward_single_launch.hpp"

#ifndef PM_FS_NMMA
#error "compile with -DPM_FS_NMMA=4, 8, 12 or 16"
#endif

namespace pm {
#define PM_FS_DEFINE_(n) PM_FS_DEFINE(n)
PM_FS_DEFINE_(PM_FS_NMMA)
} // namespace pm
