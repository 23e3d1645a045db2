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

// Variant for small tiles: a thread's NPOS elements span a group of G channels (and, with several images per
// workgroup, the images' tiles side by side inside a channel slot), so that every thread has NPOS loads in flight
// however small the tile of one channel is.  LDS element (cc, image il, r, c) sits at cc * chan_pitch +
// il * TR * TC + r * TC + c and holds input[b0 + il][ch0 + cc][row0 + r][c - pad_w].
// Preconditions, which the host checks with grouped_tile_fits() where it picks this staging (a violation would drop
// tile elements or mix the two fields of `lofs` without any visible error):
//   * one channel slot has at most NPOS * NTHREADS elements (per_chan = nslots * TR * TC): with more, G = 1 would
//     cover only the first NPOS * NTHREADS of them;
//   * the LDS offsets of a group, (G - 1) * chan_pitch + per_chan, stay below 65536 (16 bits of `lofs`), and the
//     channel inside the group (< G <= max_group) fits the 15 bits above them.
__host__ __device__ inline bool grouped_tile_fits(long long elems_per_round, long long per_chan, long long chan_pitch,
                                                  long long max_group)
{
    if (per_chan < 1 || per_chan > elems_per_round)
        return false;
    long long G = elems_per_round / per_chan;
    if (G > max_group)
        G = max_group;
    if (G < 1)
        G = 1;
    return (G - 1) * chan_pitch + per_chan <= 65536 && G < 32768;
}

template <int NPOS>
struct GroupedTile {
    int gofs[NPOS];  // offset from (image b0, first channel of the group); -1: pad value; -2: not an element
    int lofs[NPOS];  // LDS offset from the group's first channel slot | channel inside the group << 16
    int G;           // channels per group

    // nslots images have a tile in a channel slot, the first nimg of them exist; image_stride = floats per image
    template <int NTHREADS>
    __device__ __forceinline__ void init(int H, int W, int TR, int TC, int row0, int pad_w, int nslots, int nimg,
                                         int image_stride, int chan_pitch, int max_group)
    {
        const int img_elems = TR * TC;
        const int per_chan = nslots * img_elems;
        G = max(1, min(NPOS * NTHREADS / per_chan, max_group));
#pragma unroll
        for (int j = 0; j < NPOS; ++j) {
            const int e = threadIdx.x + j * NTHREADS;
            const int cc = e / per_chan;
            const int rem = e - cc * per_chan;
            const int il = rem / img_elems;
            const int pos = rem - il * img_elems;
            const int r = pos / TC, c = pos - r * TC;
            const int ih = row0 + r, iw = c - pad_w;
            lofs[j] = (cc * chan_pitch + rem) | (cc << 16);
            if (cc >= G)
                gofs[j] = -2;
            else if (il < nimg && ih >= 0 && ih < H && iw >= 0 && iw < W)
                gofs[j] = il * image_stride + cc * H * W + ih * W + iw;
            else
                gofs[j] = -1;
        }
    }

    // src: channel ch0 of image b0; channels [0, nvalid) exist, [nvalid, nchan) are zero filled; shift: per-channel
    // value subtracted from the staged elements (indexed from channel ch0), or null.  R groups per round: R * NPOS
    // loads of a thread are in flight before its first LDS store.
    template <int R>
    __device__ __forceinline__ void stage(float *lds, const float *src, int plane, int nchan, int nvalid,
                                          int chan_pitch, float oob, const float *shift) const
    {
        for (int c0 = 0; c0 < nchan; c0 += R * G) {
            float v[R][NPOS];
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float *from = src + (size_t)(c0 + r * G) * plane;
#pragma unroll
                for (int j = 0; j < NPOS; ++j) {
                    const int ch = c0 + r * G + (lofs[j] >> 16);
                    float val = 0.0f;
                    if (gofs[j] != -2 && ch < nvalid) {
                        val = gofs[j] >= 0 ? from[gofs[j]] : oob;
                        if (shift != nullptr)
                            val -= shift[ch];
                    }
                    v[r][j] = val;
                }
            }
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int j = 0; j < NPOS; ++j)
                    if (gofs[j] != -2 && c0 + r * G + (lofs[j] >> 16) < nchan)
                        lds[(c0 + r * G) * chan_pitch + (lofs[j] & 0xffff)] = v[r][j];
        }
    }
};

}  // namespace simnets
