// Placeholder for the matrix-core evaluation of plain L2 Similarity (SIMNETS_ALGO_MFMA).
#include <hip/hip_runtime.h>

#include "internal.h"

namespace simnets {

size_t sim_mfma_workspace_bytes(const SimPlan &) { return 0; }

int sim_mfma_launch(const SimPlan &, const float *, const float *, const float *, float *, void *, size_t, hipStream_t)
{
    return SIMNETS_ERR_ALGO;
}

}  // namespace simnets
