// fp32 kernels of one tile per workgroup (rows that fit a tile, and rows chained by look-back).
#include <hip/hip_runtime.h>

#include "tile_kernel.hpp"
#include "chain_kernel.hpp"
#include "kernel_table.hpp"

LINREC_KERNEL_GROUP(kernels_f32_rows,

    // one wave per row, rows up to 2048 elements
    TILE_(F32, 1, 1, 4, 0), TILE_(F32, 1, 2, 4, 0), TILE_(F32, 1, 4, 4, 0), TILE_(F32, 1, 8, 4, 0),
    // one workgroup per row
    TILE_(F32, 2, 1, 4, 0), TILE_(F32, 2, 2, 4, 0), TILE_(F32, 2, 4, 4, 0), TILE_(F32, 4, 1, 4, 0),
    TILE_(F32, 4, 2, 4, 0), TILE_(F32, 16, 2, 4, 0), TILE_(F32, 4, 4, 4, 0), TILE_(F32, 4, 8, 4, 0),
    TILE_(F32, 8, 2, 4, 0), TILE_(F32, 8, 4, 4, 0), TILE_(F32, 16, 4, 4, 0),
    // rows chained over several workgroups by look-back
    TILE_(F32, 1, 4, 4, 1), TILE_(F32, 4, 2, 4, 1), TILE_(F32, 4, 4, 4, 1), TILE_(F32, 4, 8, 4, 1),
    TILE_(F32, 8, 4, 4, 1), TILE_(F32, 8, 8, 4, 1), TILE_(F32, 16, 4, 4, 1),
    // tensors whose base addresses disagree modulo 16 bytes: element-sized accesses
    TILE_(F32, 4, 4, 1, 0), TILE_(F32, 4, 4, 1, 1),
    // look-back with several tiles (of different rows) per workgroup, next tile prefetched
    CHAIN_(F32, 4, 2, 4), CHAIN_(F32, 4, 4, 4), CHAIN_(F32, 8, 2, 4), CHAIN_(F32, 8, 4, 4)
)
