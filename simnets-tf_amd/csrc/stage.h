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

// Division-free variant for tiles of at most NPOS * NTHREADS elements per channel.  Every channel of a
// tile has the same (row, column) geometry, so each thread resolves its NPOS positions once per
// kernel (TilePositions::init) and a chunk is staged with all its loads in flight before the first
// LDS store: one memory latency per chunk.
template <int NPOS>
struct TilePositions {
    int gofs[NPOS];  // offset inside a channel plane, -1: outside the image, -2: not a tile element
    int lofs[NPOS];  // offset inside an LDS channel slot

    template <int NTHREADS>
    __device__ __forceinline__ void init(int H, int W, int TR, int TC, int row0, int pad_w)
    {
        const int per_chan = TR * TC;
#pragma unroll
        for (int j = 0; j < NPOS; ++j) {
            const int pos = threadIdx.x + j * NTHREADS;
            const int r = pos / TC;
            const int c = pos - r * TC;
            const int ih = row0 + r, iw = c - pad_w;
            lofs[j] = pos;  // == r * TC + c
            if (pos >= per_chan)
                gofs[j] = -2;
            else if (ih >= 0 && ih < H && iw >= 0 && iw < W)
                gofs[j] = ih * W + iw;
            else
                gofs[j] = -1;
        }
    }
};

// CCMAX bounds the channels of one chunk (registers: NPOS * CCMAX values in flight).
template <int NPOS, int CCMAX>
__device__ __forceinline__ void stage_input_tile_fast(float *lds, const float *img, int H, int W, int ch0, int nchan,
                                                      int nvalid, int chan_pitch, float oob, const float *shift,
                                                      const TilePositions<NPOS> &tp)
{
    const size_t plane = (size_t)H * W;
    for (int cc0 = 0; cc0 < nchan; cc0 += CCMAX) {
        float v[CCMAX][NPOS];
#pragma unroll
        for (int i = 0; i < CCMAX; ++i) {
            const int cc = cc0 + i;
            const bool chan_ok = cc < nvalid;
            const float *chan = img + (size_t)(ch0 + (chan_ok ? cc : 0)) * plane;
            const float sh = (shift != nullptr && chan_ok) ? shift[ch0 + cc] : 0.0f;
#pragma unroll
            for (int j = 0; j < NPOS; ++j) {
                float val = oob;
                if (chan_ok && cc < nchan && tp.gofs[j] >= 0)
                    val = chan[tp.gofs[j]];
                v[i][j] = chan_ok ? val - sh : 0.0f;
            }
        }
#pragma unroll
        for (int i = 0; i < CCMAX; ++i) {
            const int cc = cc0 + i;
#pragma unroll
            for (int j = 0; j < NPOS; ++j)
                if (cc < nchan && tp.gofs[j] != -2)
                    lds[cc * chan_pitch + tp.lofs[j]] = v[i][j];
        }
    }
}

}  // namespace simnets
