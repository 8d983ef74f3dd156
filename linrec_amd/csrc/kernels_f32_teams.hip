// fp32 kernels whose teams of workgroups go on from row to row (sweep, drift).
#include <hip/hip_runtime.h>

#include "sweep_kernel.hpp"
#include "drift_kernel.hpp"
#include "kernel_table.hpp"

LINREC_KERNEL_GROUP(kernels_f32_teams,
    // teams that go on from row to row so that the launch reads the tensors front to back
    SWEEP_(F32, 8, 4, 4), SWEEP_(F32, 8, 2, 4), SWEEP_(F32, 4, 4, 4), SWEEP_(F32, 8, 8, 4),
    // the same launch shape with a tile stored two steps late, so that nobody waits for the exchange
    DRIFT_FWD_(F32, 8, 4, 4), DRIFT_FWD_(F32, 8, 2, 4), DRIFT_BWD_(F32, 8, 2, 4), DRIFT_FWD_(F32, 4, 4, 4),
    // (16 waves of two slots forward: the 128 registers to be had suffice for teams of at most 64)
    DRIFT_BWD_(F32, 16, 1, 4), DRIFT_FWD_(F32, 16, 1, 4), DRIFT_FWD_(F32, 16, 2, 4),
    // rows of whole slots whose last tile is a partial one
    DRIFT_RAGGED_FWD_(F32, 16, 2, 4), DRIFT_RAGGED_BWD_(F32, 16, 1, 4), DRIFT_RAGGED_FWD_(F32, 8, 4, 4)
)
