// Staging of input rows into LDS, shared by the Similarity kernels.
#pragma once

#include <hip/hip_runtime.h>

namespace simnets {

// Copies `nchan` channels x TR rows x TC columns of one image into LDS with a workgroup of
// NTHREADS threads.  LDS element (cc, r, c) = input[ch0 + cc][row0 + r][c - pad_w], or `oob`
// where that lies outside the image (the im2col_3d padding rule, src/utils/im2col.cpp:262-273),
// minus shift[ch0 + cc] when `shift` is given.  Channels cc >= nvalid are zero filled.
// The element loop is flattened and unrolled so that U global loads per thread are in flight
// before the first LDS store: the copy is latency bound, not bandwidth bound.
template <int NTHREADS, int U>
__device__ __forceinline__ void stage_input_tile(float *lds, const float *img, int H, int W, int ch0, int nchan,
                                                 int nvalid, int TR, int TC, int chan_pitch, int row0, int pad_w,
                                                 float oob, const float *shift)
{
    const int per_chan = TR * TC;
    const int total = nchan * per_chan;
    for (int base = threadIdx.x; base < total; base += NTHREADS * U) {
        float v[U];
        int dst[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int idx = base + u * NTHREADS;
            const bool in_range = idx < total;
            const int cc = idx / per_chan;
            const int rem = idx - cc * per_chan;
            const int r = rem / TC;
            const int c = rem - r * TC;
            const int ih = row0 + r, iw = c - pad_w;
            dst[u] = in_range ? cc * chan_pitch + r * TC + c : -1;
            float val = oob;
            const bool chan_ok = cc < nvalid;
            if (in_range && chan_ok && ih >= 0 && ih < H && iw >= 0 && iw < W)
                val = img[((size_t)(ch0 + cc) * H + ih) * W + iw];
            if (shift != nullptr && in_range && chan_ok)
                val -= shift[ch0 + cc];
            v[u] = chan_ok ? val : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (dst[u] >= 0)
                lds[dst[u]] = v[u];
    }
}

}  // namespace simnets
