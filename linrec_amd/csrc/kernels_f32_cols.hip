// fp32 kernels for short rows (group, flat) and for a strided scan axis (column, segment, column block, column drift).
#include <hip/hip_runtime.h>

#include "group_kernel.hpp"
#include "flat_kernel.hpp"
#include "column_kernel.hpp"
#include "colblock_kernel.hpp"
#include "coldrift_kernel.hpp"
#include "kernel_table.hpp"

LINREC_KERNEL_GROUP(kernels_f32_cols,
    // short rows: several rows per wave
    GROUP_(F32, 4),
    // short rows that are not whole slots, dense: the tensor as one flat array
    FLAT_(F32, 4, 4), FLAT_(F32, 4, 2),
    // strided scan axis
    COLUMN_(F32, 4, 4), COLUMN_(F32, 4, 8),
    COLUMN_(F32, 2, 8), COLUMN_(F32, 2, 16), COLUMN_(F32, 1, 4), COLUMN_(F32, 1, 8), COLUMN_(F32, 1, 16),
    // strided scan axis, few rows: the scan axis cut into segments (reduce, carry, apply)
    SEGMENT_(F32, 4, 8), SEGMENT_(F32, 2, 8), SEGMENT_(F32, 1, 8), SEGMENT_(F32, 1, 16),
    // strided scan axis, a few thousand to a few ten thousand rows: the waves of a workgroup share rows
    // (two rows per lane: the backward holds three tensors, so it takes runs of 4 positions to stay in registers)
    COLBLOCK_FWD_(F32, 1, 8, 1), COLBLOCK_BWD_(F32, 1, 8, 1), COLBLOCK_FWD_(F32, 2, 8, 1), COLBLOCK_BWD_(F32, 2, 4, 1),
    // fewer rows: waves split into 2 groups of lanes that share rows (128-byte accesses; 4 groups of 16
    // floats run at half the rate: 4096 x 8192 151.8 / 270.7 us against 101.1 / 168.7 us)
    COLBLOCK_FWD_(F32, 1, 8, 2), COLBLOCK_BWD_(F32, 1, 8, 2), COLBLOCK_FWD_(F32, 2, 8, 2), COLBLOCK_BWD_(F32, 2, 4, 2),
    // strided scan axis, a few hundred to a few thousand rows: column blocks in teams along the scan axis
    // (the backward holds three tensors of four steps: runs of 4 positions)
    // (two rows per lane and runs of 8 positions in 8 waves were compiled and lost: 4096 x 16384 189 / 276 us)
    // (nor two rows per lane with runs of 4 positions in 16 waves, whose 512-byte accesses a memory-only kernel
    // likes better by 14 %: twice the team and half the positions per step make four times the exchange,
    // 4096 x 16384 forward 187 against 157 us, 2048 x 16384 124 against 85.3 us, 8192 x 4096 89.6 against 82.7 us)
    COLDRIFT_FWD_(F32, 16, 1, 8), COLDRIFT_BWD_(F32, 16, 1, 4), COLDRIFT_FWD_(F32, 8, 1, 16), COLDRIFT_BWD_(F32, 8, 1, 16)
)
