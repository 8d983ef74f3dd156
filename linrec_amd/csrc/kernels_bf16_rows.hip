// bf16 storage (fp32 arithmetic): kernels for rows on the unit-stride axis.
#include <hip/hip_runtime.h>

#include "tile_kernel.hpp"
#include "stream_kernel.hpp"
#include "team_kernel.hpp"
#include "sweep_kernel.hpp"
#include "drift_kernel.hpp"
#include "kernel_table.hpp"

LINREC_KERNEL_GROUP(kernels_bf16_rows,
    HALF_ROW_KERNELS(BF16)
)
