// fp32 kernels in which workgroups walk long rows on their own or as one team per row (stream, team).
#include <hip/hip_runtime.h>

#include "stream_kernel.hpp"
#include "team_kernel.hpp"
#include "kernel_table.hpp"

LINREC_KERNEL_GROUP(kernels_f32_walk,
    // one workgroup walks a whole row
    STREAM_(F32, 4, 4, 4), STREAM_(F32, 8, 2, 4), STREAM_(F32, 8, 4, 4), STREAM_(F32, 16, 2, 4), STREAM_(F32, 8, 8, 4),
    // several workgroups walk one row side by side
    TEAM_(F32, 4, 2, 4), TEAM_(F32, 4, 4, 4), TEAM_(F32, 8, 2, 4), TEAM_(F32, 8, 4, 4)
)
