// The Similarity combine of one patch element (include/utils/similarity_utils.hpp:23-66 in the reference) on packed
// parameters, and the packing itself; shared by the Similarity kernels and the kernel that evaluates a Similarity
// layer inside the MEX staging.
#pragma once

#include <hip/hip_runtime.h>

#include "internal.h"
#include "valu_tile.h"

namespace simnets {

// Packed parameters of element (m, k): a0 = template (sqrt-weight form: sqrt(w) t), a1 = the negative weight,
// halved for the normalized modes (sqrt-weight form: -sqrt(w)); c = the logarithm term of the normalized modes.
__device__ __forceinline__ void sim_pack_element(int mode, bool valid, float t, float w, float fudge, float &a0,
                                                 float &a1, float &c)
{
    c = 0.0f;
    if (valid) {
        if (mode == SIM_MODE_L2_NORM)
            c = 0.5f * logf(w + fudge);
        else if (mode == SIM_MODE_L2_NORM_IGNORE_NAN)
            c = (float)(0.5 * ((double)logf(w + fudge) - 1.8378770664093453 /* log(2 pi) */));
    }
    if (mode == SIM_MODE_L2_SQRTW) {
        const float sq = sqrtf(w);
        a0 = sq * t;
        a1 = -sq;
    } else {
        const float scale = (mode == SIM_MODE_L2_NORM || mode == SIM_MODE_L2_NORM_IGNORE_NAN) ? -0.5f : -1.0f;
        a0 = t;
        a1 = scale * w;
    }
}

// One k step for all MT templates and PT pixels of a lane.  VP: the parameters are already in VGPRs
// (fetched with vector loads); otherwise they are wave-uniform SGPR values and are moved once.
template <int MODE, int PT, int MT, bool VP = false>
__device__ __forceinline__ void sim_step(float (&acc)[MT][PT], const float (&x)[PT], const float (&pa)[2 * MT],
                                         const float (&pc)[MT])
{
    auto vg = [](float v) { return VP ? v : to_vgpr(v); };
    if (MODE == SIM_MODE_L2_NORM_IGNORE_NAN) {
        float keep[PT], xz[PT];
#pragma unroll
        for (int p = 0; p < PT; ++p) {
            const bool ok = x[p] == x[p];
            keep[p] = ok ? 1.0f : 0.0f;
            xz[p] = ok ? x[p] : 0.0f;
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const float t = vg(pa[2 * m]), nwh = vg(pa[2 * m + 1]), c = vg(pc[m]);
#pragma unroll
            for (int p = 0; p < PT; ++p) {
                const float d = t - xz[p];
                const float term = __builtin_fmaf(nwh * d, d, c);
                acc[m][p] = __builtin_fmaf(keep[p], term, acc[m][p]);
            }
        }
    } else {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const float t = vg(pa[2 * m]), nw = vg(pa[2 * m + 1]);
            float c = 0.0f;
            if (MODE == SIM_MODE_L2_NORM)
                c = vg(pc[m]);
            // The combine is a chain of dependent instructions per pixel; a dependent VALU instruction
            // issued right behind its producer stalls, so the chain is laid out stage by stage across
            // the PT pixels (PT independent instructions between producer and consumer).
            float d[PT], q[PT];
#pragma unroll
            for (int p = 0; p < PT; ++p)
                d[p] = (MODE == SIM_MODE_L2_SQRTW) ? __builtin_fmaf(nw, x[p], t) : t - x[p];
            __builtin_amdgcn_sched_barrier(0);
            if (MODE == SIM_MODE_L2 || MODE == SIM_MODE_L2_NORM) {
#pragma unroll
                for (int p = 0; p < PT; ++p)
                    q[p] = nw * d[p];
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int p = 0; p < PT; ++p) {
                if (MODE == SIM_MODE_L2_SQRTW)
                    acc[m][p] = __builtin_fmaf(-d[p], d[p], acc[m][p]);  // (sqrt(w)*t, -sqrt(w)) in pa
                else if (MODE == SIM_MODE_L1)
                    acc[m][p] = __builtin_fmaf(nw, __builtin_fabsf(d[p]), acc[m][p]);
                else if (MODE == SIM_MODE_L2)
                    acc[m][p] = __builtin_fmaf(q[p], d[p], acc[m][p]);
                else
                    q[p] = __builtin_fmaf(q[p], d[p], c);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (MODE == SIM_MODE_L2_NORM) {
#pragma unroll
                for (int p = 0; p < PT; ++p)
                    acc[m][p] += q[p];
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
}

}  // namespace simnets
