// f16 storage (fp32 arithmetic): kernels for short rows and for a strided scan axis.
#include <hip/hip_runtime.h>

#include "group_kernel.hpp"
#include "flat_kernel.hpp"
#include "column_kernel.hpp"
#include "colblock_kernel.hpp"
#include "coldrift_kernel.hpp"
#include "kernel_table.hpp"

LINREC_KERNEL_GROUP(kernels_f16_cols,
    HALF_COLUMN_KERNELS(F16)
)
