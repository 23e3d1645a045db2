// Similarity backward on the vector ALU (gfx950): gradient w.r.t. the input, and w.r.t. the
// templates and weights.
//
// Replaces SimilarityInputGradKernelGPU / SimilarityParametersGradKernelGPU
// (src/kernels/similarity_grad_kernel_gpu.cu), i.e. per image im2col_3d_gpu + ggemm_readc_gpu with
// the functors of include/utils/similarity_utils.hpp:82-150 (+ col2im_3d_gpu for the input
// gradient, + deinterlace for the parameters), by one launch over the whole batch each.
//
// Input gradient
//   dX[b,c,y,x] = sum_o sum_{taps (i,j) whose window covers (y,x)} g[b,o,yo,xo] * B(t[o,c,i,j], w[o,c,i,j], X[b,c,y,x])
//   with yo = (y + ph - i)/sh.  Input pixels are split by phase (ry, rx) = ((y+ph) mod sh, (x+pw) mod sw):
//   all pixels of a phase see the same tap subset i = ry + sh*ii, j = rx + sw*jj, and in phase
//   coordinates a = (y+ph)/sh the sum is a stride-1 correlation of g with that tap subset.  Each
//   phase is one launch of the same register-tile scheme as the forward kernel with the roles
//   swapped: g rows are staged in LDS (out of range -> 0), a lane owns PT pixels x MT input
//   channels (accumulators AND the X values they belong to in VGPRs), the packed parameters of a
//   (o, tap) step arrive through vector loads with a lane-uniform address, one step ahead.
// Parameter gradients
//   dT[o,k], dW[o,k] = sum over all B*oh*ow output pixels of W(g[px,o], patch(px)[k], t[o,k], w[o,k]).
//   A lane owns 8 templates x 4 patch elements (its t values and the running sums in VGPRs), a wave
//   64 x 32, a workgroup 128 x 64 (or 64 x 128); pixels stream through LDS in chunks of 64, g as
//   [o/4][pixel][4] and the gathered patch elements as [k/4][pixel][4], so that every lane reads its
//   operands with three 16-byte LDS reads per pixel.  The pixel range is split over workgroups; the
//   partial sums are written out and added up in a fixed order by a second kernel, which also
//   applies the factors that do not depend on the pixel (2w, -1, 1/(w+fudge)).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <vector>
#include <cmath>

#include "internal.h"
#include "stage.h"
#include "valu_tile.h"

namespace simnets {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kWaves = 4;
constexpr int kThreads = 64 * kWaves;
constexpr int kLdsBudgetFloats = 16384;
constexpr int kStagePos = 6;
constexpr int kStageChan = 6;

enum GradMode { GX_L2 = 0, GX_L1 = 1 };

// ------------------------------------------------------------------------------------------------
// input gradient
// ------------------------------------------------------------------------------------------------
struct GradXArgs {
    const float *g;    // output gradient [B,O,oh,ow]
    const float *x;    // input [B,C,H,W]
    float *dx;         // [B,C,H,W]
    const float *pb;   // this phase's parameters [ctile][K + 1][MT][2], K = O*nI*nJ, taps flipped
    const int *koff;   // [K + 2] LDS offset of step k = (o, dh, dw): (o % CC) * TRmax*TC + dh*TC + dw
    int B, C, H, W, O, oh, ow;
    int nI, nJ;        // taps of this phase along h and w
    int padh, padw;    // padding of g in phase coordinates: phase row h reads g rows h - padh + dh
    int na, nb;        // extent of the phase grid
    int y0, x0;        // input pixel of phase position (h, v): (y0 + sh*h, x0 + sw*v)
    int sh, sw;
    int K;
    int G, gpi, tiles, nws, nws_log2, n_ctiles, TC, TRmax, CC;
    int ignore_nan;
    int fast_stage;    // the g tile of a channel has at most kStagePos * kThreads elements: division-free staging
    int row_limit, col_limit;  // phase rows h <= row_limit (columns v <= col_limit) are covered by a window
    int NI;            // small phase grids (MULTI variant): a wave covers NI images (lane -> image, pixel group); their
                       // g tiles sit side by side in a channel's LDS slot
    int grid_x, grid_y;  // workgroups of this phase (a launch covers several phases: blockIdx.z)
};

constexpr int kGxMaxPhases = 16;   // stride phases per launch
struct GradXPhases {
    GradXArgs p[kGxMaxPhases];
};

template <int MODE, int PT, int MT>
__device__ __forceinline__ void gx_step(float (&acc)[MT][PT], const float (&xv)[MT][PT], const float (&gv)[PT],
                                        const float (&pb)[2 * MT])
{
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const float p0 = pb[2 * m], p1 = pb[2 * m + 1];  // already in VGPRs (vector loads)
        float u[PT];
        if (MODE == GX_L2) {
            // (s*w*t, -s*w): u = s*w*(t - x)
#pragma unroll
            for (int p = 0; p < PT; ++p)
                u[p] = __builtin_fmaf(p1, xv[m][p], p0);
        } else {
            // (copysign(2^100, w) * t, w): d = +-2^100 * (t - x) is either 0 or far outside [-|w|, |w|], so its
            // median with -|w| and |w| is w * sign(t - x) (exactly 0 for t == x).  NaN inputs never get here:
            // the tile holds 0 in their place and their gradient is stored as 0, which is what sign(NaN) = 0
            // gives in the reference.
            const float nbig = -__builtin_copysignf(0x1p100f, p1);
            const float lim = __builtin_fabsf(p1);
            float d[PT];
#pragma unroll
            for (int p = 0; p < PT; ++p)
                d[p] = __builtin_fmaf(nbig, xv[m][p], p0);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int p = 0; p < PT; ++p)
                u[p] = __builtin_amdgcn_fmed3f(d[p], -lim, lim);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int p = 0; p < PT; ++p)
            acc[m][p] = __builtin_fmaf(gv[p], u[p], acc[m][p]);
        __builtin_amdgcn_sched_barrier(0);
    }
}

constexpr int gx_waves_per_simd(int pt, int mt) { return pt * mt <= 32 ? 3 : 2; }
constexpr int gx_lds_budget(int pt, int mt) { return pt * mt <= 32 ? kLdsBudgetFloats / 2 : kLdsBudgetFloats; }

// MULTI: small phase grids, a wave covers a.NI images.
template <int MODE, int PT, int MT, bool MULTI = false>
__global__ __launch_bounds__(kThreads, gx_waves_per_simd(PT, MT)) void sim_grad_input_kernel(const GradXPhases phases)
{
    const GradXArgs &a = phases.p[blockIdx.z];
    if ((int)blockIdx.x >= a.grid_x || (int)blockIdx.y >= a.grid_y)
        return;   // a phase with fewer workgroups than the largest of the launch
    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    constexpr bool multi = MULTI;
    const int b0 = multi ? blockIdx.x * a.NI : blockIdx.x / a.tiles;
    const int tile = multi ? 0 : blockIdx.x - b0 * a.tiles;
    // (MULTI: the four waves of a workgroup share one channel tile and split the steps of every chunk)
    const int ws = multi ? 0 : wave & (a.nws - 1);
    const int wm = multi ? 0 : wave >> a.nws_log2;
    const int nwm = multi ? 1 : kWaves >> a.nws_log2;
    const int ctile = blockIdx.y * nwm + wm;
    const bool wave_active = ctile < a.n_ctiles;

    const int g_first = tile * 64 * a.nws;
    const int g_last = min(g_first + 64 * a.nws, a.gpi) - 1;
    const int row_first = g_first / a.G;
    const int nrows = g_last / a.G - row_first + 1;
    const int TR = nrows - 1 + a.nI;
    const int in_row0 = row_first - a.padh;

    // this lane's pixel group: of image b0 (a tile of its groups), or - small grids - of image b0 + lane / gpi
    const int img_l = multi ? lane / a.gpi : 0;
    int grp = multi ? lane - img_l * a.gpi : g_first + ws * 64 + lane;
    const bool lane_valid = multi ? (img_l < a.NI && b0 + img_l < a.B) : grp <= g_last;
    grp = min(grp, g_last);
    const int b = lane_valid ? b0 + img_l : b0;
    const int h = grp / a.G;
    const int gw = grp - h * a.G;
    const int lds_base = (lane_valid ? img_l : 0) * (TR * a.TC) + (h - row_first) * a.TC + gw * PT;
    const int v0 = gw * PT;

    // the X values of this lane's tile (NaN -> 0 when NaN inputs are ignored: their gradient is 0)
    // All of them are requested first, elements outside the tile on a clamped address: a load inside the condition
    // would be waited for before the next one is issued.  nan_at: bit m * PT + p = that element is a NaN whose
    // gradient is 0 (what the stores at the end need to know).
    float acc[MT][PT], xv[MT][PT];
    const size_t plane = (size_t)a.H * a.W;
    const float *xrow = a.x + (size_t)b * a.C * plane + (size_t)(a.y0 + a.sh * h) * a.W + a.x0;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int c = min(ctile * MT + m, a.C - 1);
#pragma unroll
        for (int p = 0; p < PT; ++p)
            xv[m][p] = xrow[(size_t)c * plane + (size_t)a.sw * max(min(v0 + p, a.nb - 1), 0)];
    }
    unsigned long long nan_at = 0;
    static_assert(MT * PT <= 64, "one bit per element of the lane tile");
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int c = ctile * MT + m;
#pragma unroll
        for (int p = 0; p < PT; ++p) {
            acc[m][p] = 0.0f;
            float val = (wave_active && lane_valid && c < a.C && v0 + p < a.nb) ? xv[m][p] : 0.0f;
            if ((a.ignore_nan || MODE == GX_L1) && !(val == val)) {
                val = 0.0f;
                nan_at |= 1ull << (m * PT + p);
            }
            xv[m][p] = val;
        }
    }

    // parameter stream: same address in every lane, fetched with vector loads so that the values arrive
    // in VGPRs (the zero is opaque to the compiler, which would otherwise turn them into scalar loads)
    unsigned zero_v;
    asm volatile("v_mov_b32 %0, 0" : "=v"(zero_v));
    const char *pb_base = reinterpret_cast<const char *>(a.pb + (size_t)(wave_active ? ctile : 0) * (a.K + 1) * MT * 2);
    unsigned pb_off = zero_v;  // byte offset of the NEXT step
    auto fetch_params = [&](float (&pbv)[2 * MT]) {
#pragma unroll
        for (int i = 0; i < 2 * MT / 4; ++i) {
            const float4 v = *reinterpret_cast<const float4 *>(pb_base + pb_off + 16 * i);
            pbv[4 * i] = v.x; pbv[4 * i + 1] = v.y; pbv[4 * i + 2] = v.z; pbv[4 * i + 3] = v.w;
        }
        pb_off += 2 * MT * sizeof(float);
    };
    const float *img = a.g + (size_t)b0 * a.O * a.oh * a.ow;
    const int chan_lds = (multi ? a.NI : 1) * a.TRmax * a.TC;
    float pb0[2 * MT], pb1[2 * MT];
    fetch_params(pb0);
    TilePositions<multi ? 1 : kStagePos> tp;
    GroupedTile<multi ? kStagePos : 1> gt;
    if constexpr (multi)
        gt.template init<kThreads>(a.oh, a.ow, TR, a.TC, in_row0, a.padw, a.NI, min(a.NI, a.B - b0), a.O * a.oh * a.ow,
                                   chan_lds, a.CC);
    else
        tp.template init<kThreads>(a.oh, a.ow, TR, a.TC, in_row0, a.padw);
    const int SIMNETS_CONST_AS *kt = (const int SIMNETS_CONST_AS *)(a.koff);

    for (int ch0 = 0; ch0 < a.O; ch0 += a.CC) {
        const int ccn = min(a.CC, a.O - ch0);
        __syncthreads();
        if constexpr (multi)
            gt.template stage<1>(lds, img + (size_t)ch0 * a.oh * a.ow, a.oh * a.ow, ccn, ccn, chan_lds, 0.0f, nullptr);
        else if (a.fast_stage)
            stage_input_tile_fast<kStagePos, kStageChan>(lds, img, a.oh, a.ow, ch0, ccn, ccn, chan_lds, 0.0f, nullptr, tp);
        else
            stage_input_tile<kThreads, 8>(lds, img, a.oh, a.ow, ch0, ccn, ccn, TR, a.TC, chan_lds, in_row0, a.padw, 0.0f,
                                          nullptr);
        __syncthreads();
        if (!wave_active)
            continue;
        // software pipeline over the (o, tap) steps of this chunk: the g values and the parameters of
        // the next step are requested before the arithmetic of the current one
        int nk = ccn * a.nI * a.nJ;
        if constexpr (multi) {
            // this wave's quarter of the chunk's templates
            const int taps = a.nI * a.nJ;
            const int cpw = (ccn + kWaves - 1) / kWaves;
            const int c_lo = min(wave * cpw, ccn), c_hi = min(c_lo + cpw, ccn);
            const int k_first = (ch0 + c_lo) * taps;
            nk = (c_hi - c_lo) * taps;
            kt = (const int SIMNETS_CONST_AS *)(a.koff) + k_first;
            pb_off = zero_v + (unsigned)k_first * (unsigned)(2 * MT * sizeof(float));
            fetch_params(pb0);
        }
        int off_next = kt[1];
        auto step = [&](const float (&gc)[PT], const float (&pbc)[2 * MT], float (&gnx)[PT], float (&pbnx)[2 * MT]) {
            __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): issued a whole step ago
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int p = 0; p < PT; ++p)
                gnx[p] = lds[lds_base + off_next + p];
            kt += 1;
            off_next = kt[1];
            fetch_params(pbnx);  // one step of slack exists behind each channel tile
            __builtin_amdgcn_sched_barrier(0);
            gx_step<MODE, PT, MT>(acc, xv, gc, pbc);
            __builtin_amdgcn_sched_barrier(0);
        };
        float g0[PT], g1[PT];
        {
            const int off0 = kt[0];
#pragma unroll
            for (int p = 0; p < PT; ++p)
                g0[p] = lds[lds_base + off0 + p];
        }
        int kk = 0;
        for (; kk + 2 <= nk; kk += 2) {
            step(g0, pb0, g1, pb1);
            step(g1, pb1, g0, pb0);
        }
        if (kk < nk) {
            step(g0, pb0, g1, pb1);
#pragma unroll
            for (int i = 0; i < 2 * MT; ++i)
                pb0[i] = pb1[i];
        }
    }

    if constexpr (multi) {
        // partial sums of waves 1..3 -> wave 0, in wave order; the tile's LDS is reused
        constexpr int kPart = MT * PT * 64;
        __syncthreads();
        if (wave > 0) {
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int p = 0; p < PT; ++p)
                    lds[(wave - 1) * kPart + (m * PT + p) * 64 + lane] = acc[m][p];
        }
        __syncthreads();
        if (wave > 0)
            return;
        for (int w = 1; w < kWaves; ++w)
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
                for (int p = 0; p < PT; ++p)
                    acc[m][p] += lds[(w - 1) * kPart + (m * PT + p) * 64 + lane];
    }
    if (!wave_active || !lane_valid)
        return;
    const bool row_covered = h <= a.row_limit;
    float *drow = a.dx + (size_t)b * a.C * plane + (size_t)(a.y0 + a.sh * h) * a.W + a.x0;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int c = ctile * MT + m;
        if (c >= a.C)
            break;
#pragma unroll
        for (int p = 0; p < PT; ++p) {
            if (v0 + p >= a.nb)
                continue;
            const size_t o = (size_t)c * plane + (size_t)a.sw * (v0 + p);
            float val = (row_covered && v0 + p <= a.col_limit) ? acc[m][p] : 0.0f;
            if ((nan_at >> (m * PT + p)) & 1)
                val = 0.0f;
            drow[o] = val;
        }
    }
}

// One input element per thread: the taps whose window covers the element outside, the templates inside (no
// divisions in the inner loop; the threads of a wave read neighbouring g values).  Used for geometries whose g
// rows do not fit the LDS budget and for inputs of one or two channels (the first layer of the reference's
// networks), where the channel lanes of the tiled kernel would idle and each stride phase costs two launches.
__global__ __launch_bounds__(256) void sim_grad_input_gather_kernel(const float *__restrict__ g,
                                                                    const float *__restrict__ x,
                                                                    const float *__restrict__ templates,
                                                                    const float *__restrict__ weights,
                                                                    float *__restrict__ dx, int B, int C, int H, int W,
                                                                    int O, int oh, int ow, int bh, int bw, int sh,
                                                                    int sw, int ph, int pw, int l1, float scale,
                                                                    int ignore_nan)
{
    const long long total = (long long)B * C * H * W;
    const size_t oplane = (size_t)oh * ow, tplane = (size_t)C * bh * bw;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long long)gridDim.x * blockDim.x) {
        const int xx = (int)(idx % W);
        long long r = idx / W;
        const int yy = (int)(r % H);
        r /= H;
        const int c = (int)(r % C);
        const int b = (int)(r / C);
        const float xin = x[idx];
        float acc = 0.0f;
        if (!(ignore_nan && !(xin == xin))) {
            for (int i = 0; i < bh; ++i) {
                const int ty = yy + ph - i;
                if (ty < 0 || ty % sh != 0 || ty / sh >= oh)
                    continue;
                for (int j = 0; j < bw; ++j) {
                    const int tx = xx + pw - j;
                    if (tx < 0 || tx % sw != 0 || tx / sw >= ow)
                        continue;
                    const float *gp = g + (size_t)b * O * oplane + (size_t)(ty / sh) * ow + tx / sw;
                    const size_t pi = ((size_t)c * bh + i) * bw + j;
                    for (int o = 0; o < O; ++o) {
                        const float gv = gp[(size_t)o * oplane];
                        const float t = templates[(size_t)o * tplane + pi], w = weights[(size_t)o * tplane + pi];
                        const float d = t - xin;
                        float u;
                        if (l1)
                            u = w * (float)((0.0f < d) - (d < 0.0f));
                        else
                            u = scale * w * d;
                        acc = __builtin_fmaf(gv, u, acc);
                    }
                }
            }
        }
        dx[idx] = acc;
    }
}

__global__ void fill_zero_kernel(float *__restrict__ p, long long n)
{
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
        p[i] = 0.0f;
}

// Packs the (template, weight) pairs of the stride phases (blockIdx.y) as [ctile][k = (o, dh, dw)][MT][2] with the
// taps flipped (dh = nI-1-ii, original tap i = ry + sh*ii) and the per-mode scaling folded in.
struct GxPackPhase {
    float *pb;
    int *koff;
    int ry, rx, nI, nJ, MT, n_ctiles, CC, chan_pitch, TC;
};
struct GxPackPhases {
    GxPackPhase p[kGxMaxPhases];
};

__global__ void sim_grad_input_pack_kernel(const float *__restrict__ templates, const float *__restrict__ weights,
                                           int O, int C, int bh, int bw, int sh, int sw, int l1, float scale,
                                           const GxPackPhases phases)
{
    const GxPackPhase &q = phases.p[blockIdx.y];
    const int ry = q.ry, rx = q.rx, nI = q.nI, nJ = q.nJ, MT = q.MT, n_ctiles = q.n_ctiles, CC = q.CC;
    const int chan_pitch = q.chan_pitch, TC = q.TC;
    float *__restrict__ pb = q.pb;
    int *__restrict__ koff = q.koff;
    const int K = O * nI * nJ;
    for (int k = blockIdx.x * blockDim.x + threadIdx.x; k < K + 2; k += gridDim.x * blockDim.x) {
        int off = 0;
        if (k < K) {
            const int dw = k % nJ, dh = (k / nJ) % nI, o = k / (nJ * nI);
            off = (o % CC) * chan_pitch + dh * TC + dw;
        }
        koff[k] = off;
    }
    const long long total = (long long)n_ctiles * (K + 1) * MT;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long long)gridDim.x * blockDim.x) {
        const int mi = (int)(idx % MT);
        const long long r = idx / MT;
        const int k = (int)(r % (K + 1));
        const int ctile = (int)(r / (K + 1));
        const int c = ctile * MT + mi;
        float p0 = 0.0f, p1 = 0.0f;
        if (k < K && c < C) {
            const int dw = k % nJ;
            const int dh = (k / nJ) % nI;
            const int o = k / (nJ * nI);
            const int i = ry + sh * (nI - 1 - dh), j = rx + sw * (nJ - 1 - dw);
            const size_t pi = (((size_t)o * C + c) * bh + i) * bw + j;
            const float t = templates[pi], w = weights[pi];
            if (l1) {
                p0 = copysignf(0x1p100f, w) * t;
                p1 = w;
            } else {
                p0 = scale * w * t;
                p1 = -(scale * w);
            }
        }
        pb[2 * idx] = p0;
        pb[2 * idx + 1] = p1;
    }
}

struct Phase {
    int ry, rx, nI, nJ, a0, b0, na, nb;
    bool empty() const { return nI <= 0 || nJ <= 0 || na <= 0 || nb <= 0; }
};

void phase_axis(int r, int block, int stride, int pad, int size, int *n_taps, int *first, int *count)
{
    *n_taps = r < block ? (block - r + stride - 1) / stride : 0;
    *first = pad > r ? (pad - r + stride - 1) / stride : 0;
    const int top = size - 1 + pad - r;  // largest y + pad - r
    *count = top >= 0 ? top / stride - *first + 1 : 0;
}

Phase make_phase(const SimPlan &p, int ry, int rx)
{
    Phase f;
    f.ry = ry; f.rx = rx;
    phase_axis(ry, p.bh, p.sh, p.ph, p.H, &f.nI, &f.a0, &f.na);
    phase_axis(rx, p.bw, p.sw, p.pw, p.W, &f.nJ, &f.b0, &f.nb);
    return f;
}

struct GxTiling {
    int PT, MT, nws, G, gpi, tiles, TC, TRmax, CC;
    int NI;   // images per wave (small phase grids), else 1
    bool ksplit;   // the variant for small grids: a wave covers NI >= 1 whole images, the four waves of a workgroup
                   // share a channel tile and split the templates
    bool lds_ok, fast_stage;
};

GxTiling gx_try(const SimPlan &p, const Phase &f, int PT, int nws, int MT = 8)
{
    GxTiling t;
    t.PT = PT; t.MT = MT; t.nws = nws;
    const int budget = gx_lds_budget(t.PT, t.MT);
    t.G = (f.nb + t.PT - 1) / t.PT;
    t.gpi = f.na * t.G;
    t.tiles = (t.gpi + 64 * nws - 1) / (64 * nws);
    t.TC = (t.G * t.PT - 1) + f.nJ;
    t.TC |= 1;
    const int max_rows = std::min(f.na, (64 * nws + t.G - 1) / t.G + 1);
    t.TRmax = max_rows - 1 + f.nI;
    // a phase grid of at most 32 pixel groups: a wave takes several images
    t.NI = 1;
    if (nws == 1 && t.tiles == 1 && 2 * t.gpi <= 64 && p.B >= 2) {
        int ni = std::min(64 / t.gpi, p.B);
        while (ni > 1 && (1LL * ni * t.TRmax * t.TC > kStagePos * kThreads || 1LL * ni * t.TRmax * t.TC > budget ||
                          1LL * ni * p.O * p.oh * p.ow >= (1LL << 31)))
            --ni;
        t.NI = ni;
    }
    // ... and so does a grid that would give the SIMDs at most one wave each (one image per wave then)
    const long long plain_waves = (long long)p.B * (((p.C + t.MT - 1) / t.MT + kWaves - 1) / kWaves) * kWaves;
    if (MT != 8)
        t.NI = 1;   // (the small-grid variant has the 4 x 8 lane tile)
    t.ksplit = MT != 8 ? false : t.NI > 1 || (nws == 1 && t.tiles == 1 && t.gpi <= 64 && plain_waves <= 1024 && p.O >= kWaves &&
                            1LL * t.TRmax * t.TC <= kStagePos * kThreads);
    const long long per_chan = 1LL * t.NI * t.TRmax * t.TC;
    t.lds_ok = per_chan <= budget;
    t.fast_stage = per_chan <= kStagePos * kThreads;
    t.CC = 1;
    if (t.NI > 1 && !grouped_tile_fits(kStagePos * kThreads, per_chan, per_chan, p.O)) {
        // (cannot happen while the loop above bounds NI * tile by kStagePos * kThreads; kept as the staging's own check)
        t.NI = 1;
        t.lds_ok = false;
    }
    if (t.lds_ok) {
        const int cc_max = (int)std::min<long long>(p.O, budget / per_chan);
        const int chunks = (p.O + cc_max - 1) / cc_max;
        t.CC = (p.O + chunks - 1) / chunks;
        // several images per wave: the four waves split a chunk's templates, a multiple of four keeps them even
        if (t.ksplit && t.CC > kWaves && t.CC % kWaves)
            t.CC = t.CC / kWaves * kWaves;
    }
    return t;
}

GxTiling gx_tiling(const SimPlan &p, const Phase &f)
{
    auto pick = [&](int PT) {
        const int n_ctiles = (p.C + 7) / 8;
        const int gpi = f.na * ((f.nb + PT - 1) / PT);
        int nws = 1;
        if (n_ctiles <= 2 && gpi >= 128)
            nws = 2;
        if (n_ctiles <= 1 && gpi >= 256)
            nws = 4;
        GxTiling t = gx_try(p, f, PT, nws);
        while (nws > 1 && !(t.lds_ok && t.fast_stage)) {   // fewer spatial waves: fewer g rows per workgroup
            nws >>= 1;
            t = gx_try(p, f, PT, nws);
        }
        return t;
    };
    // Three or four channels (an image): 8 pixels x 4 channels per lane, all pixel waves on the one channel tile
    if (p.C <= 4 && f.nb >= 16) {
        const int gpi = f.na * ((f.nb + 7) / 8);
        int nws = gpi >= 256 ? 4 : (gpi >= 128 ? 2 : 1);
        GxTiling t = gx_try(p, f, 8, nws, 4);
        while (nws > 1 && !(t.lds_ok && t.fast_stage)) {
            nws >>= 1;
            t = gx_try(p, f, 8, nws, 4);
        }
        if (t.lds_ok && !pick(4).ksplit)
            return t;
    }
    // 8 x 8 lane tile for wide phase grids with many channels, if the grid then still gives every SIMD two waves
    if (f.nb >= 32 && p.C >= 32) {
        const GxTiling big = pick(8);
        const int n_ctiles = (p.C + 7) / 8, nwm = kWaves / big.nws;
        const long long waves = (long long)p.B * big.tiles * ((n_ctiles + nwm - 1) / nwm) * kWaves;
        if (big.lds_ok && waves >= 1536)
            return big;
    }
    return pick(4);
}

size_t gx_phase_param_bytes(const SimPlan &p, const Phase &f)
{
    const size_t n_ctiles = (p.C + 7) / 8;
    return align_up(n_ctiles * ((size_t)p.O * f.nI * f.nJ + 1) * 8 * 2 * sizeof(float), 256);
}

size_t gx_phase_table_bytes(const SimPlan &p, const Phase &f)
{
    return align_up(((size_t)p.O * f.nI * f.nJ + 2) * sizeof(int), 256);
}

bool gx_all_phases_fit(const SimPlan &p)
{
    for (int ry = 0; ry < p.sh; ++ry)
        for (int rx = 0; rx < p.sw; ++rx) {
            const Phase f = make_phase(p, ry, rx);
            if (!f.empty() && !gx_tiling(p, f).lds_ok)
                return false;
        }
    return true;
}

// One launch for the phases that share a kernel variant (lane tile, small-grid form).
template <int MODE>
hipError_t gx_launch_phases(const GradXPhases &ph, int n, int PT, int MT, bool ksplit, hipStream_t s)
{
    unsigned gx = 1, gy = 1;
    size_t lds_floats = 0;
    for (int i = 0; i < n; ++i) {
        const GradXArgs &a = ph.p[i];
        gx = std::max(gx, (unsigned)a.grid_x);
        gy = std::max(gy, (unsigned)a.grid_y);
        size_t floats = (size_t)a.CC * std::max(a.NI, 1) * a.TRmax * a.TC;
        if (ksplit)  // the LDS also holds three waves' partial sums at the end
            floats = std::max<size_t>(floats, (size_t)(kWaves - 1) * 8 * 4 * 64);
        lds_floats = std::max(lds_floats, floats);
    }
    dim3 grid(gx, gy, (unsigned)n);
    const size_t lds_bytes = lds_floats * sizeof(float);
    if (ksplit)
        hipLaunchKernelGGL((sim_grad_input_kernel<MODE, 4, 8, true>), grid, dim3(kThreads), lds_bytes, s, ph);
    else if (MT == 4)
        hipLaunchKernelGGL((sim_grad_input_kernel<MODE, 8, 4>), grid, dim3(kThreads), lds_bytes, s, ph);
    else if (PT == 8)
        hipLaunchKernelGGL((sim_grad_input_kernel<MODE, 8, 8>), grid, dim3(kThreads), lds_bytes, s, ph);
    else
        hipLaunchKernelGGL((sim_grad_input_kernel<MODE, 4, 8>), grid, dim3(kThreads), lds_bytes, s, ph);
    return hipGetLastError();
}

}  // namespace

// the one-element-per-thread kernel: rows too long for the LDS tile, or one or two input channels
static bool gx_gather(const SimPlan &p) { return !gx_all_phases_fit(p) || p.C <= 2; }

size_t sim_grad_input_workspace_bytes(const SimPlan &p)
{
    if (sim_mfma_grad_input_supported(p))
        return sim_mfma_grad_input_workspace_bytes(p);
    if (gx_gather(p))
        return 0;
    size_t total = 0;
    for (int ry = 0; ry < p.sh; ++ry)
        for (int rx = 0; rx < p.sw; ++rx) {
            const Phase f = make_phase(p, ry, rx);
            if (!f.empty())
                total += gx_phase_param_bytes(p, f) + gx_phase_table_bytes(p, f);
        }
    return total;
}

int sim_grad_input(const SimPlan &p, const float *input, const float *templates, const float *weights,
                          const float *output_grad, float *input_grad, void *workspace, size_t workspace_bytes,
                          void *stream)
{
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const bool l1 = p.mode == SIM_MODE_L1;
    const bool norm = p.mode == SIM_MODE_L2_NORM || p.mode == SIM_MODE_L2_NORM_IGNORE_NAN;
    const float scale = norm ? 1.0f : 2.0f;  // the normalized functor halves the plain L2 one
    const int ignore_nan = p.mode == SIM_MODE_L2_NORM_IGNORE_NAN;
    const long long n_in = (long long)p.B * p.C * p.H * p.W;

    if (sim_mfma_grad_input_supported(p))
        return sim_mfma_grad_input_launch(p, input, templates, weights, output_grad, input_grad, workspace,
                                          workspace_bytes, stream);
    if (gx_gather(p)) {
        const int blocks = (int)std::min<long long>((n_in + 255) / 256, 1 << 20);
        hipLaunchKernelGGL(sim_grad_input_gather_kernel, dim3(blocks), dim3(256), 0, s, output_grad, input, templates,
                           weights, input_grad, p.B, p.C, p.H, p.W, p.O, p.oh, p.ow, p.bh, p.bw, p.sh, p.sw, p.ph,
                           p.pw, (int)l1, scale, ignore_nan);
        return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
    }
    if (workspace_bytes < sim_grad_input_workspace_bytes(p))
        return SIMNETS_ERR_WORKSPACE;

    // pixels of a phase without taps (stride larger than the block) are written by no launch
    if (p.sh > p.bh || p.sw > p.bw) {
        const int blocks = (int)std::min<long long>((n_in + 255) / 256, 65535);
        hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, s, input_grad, n_in);
        if (hipGetLastError() != hipSuccess)
            return SIMNETS_ERR_HIP;
    }

    // the phases' arguments, grouped by kernel variant (lane tile, small-grid form): one pack launch and one main
    // launch per group of at most kGxMaxPhases phases (ordinarily one group: the phase grids differ by a row or column)
    struct Job {
        GradXArgs a;
        GxPackPhase q;
        int PT, MT;
        bool ksplit;
    };
    std::vector<Job> jobs;
    char *ws = reinterpret_cast<char *>(workspace);
    for (int ry = 0; ry < p.sh; ++ry)
        for (int rx = 0; rx < p.sw; ++rx) {
            const Phase f = make_phase(p, ry, rx);
            if (f.empty())
                continue;
            const GxTiling t = gx_tiling(p, f);
            const int n_ctiles = (p.C + t.MT - 1) / t.MT;
            const int K = p.O * f.nI * f.nJ;
            float *pb = reinterpret_cast<float *>(ws);
            ws += gx_phase_param_bytes(p, f);
            int *koff = reinterpret_cast<int *>(ws);
            ws += gx_phase_table_bytes(p, f);

            Job j;
            j.PT = t.PT; j.MT = t.MT; j.ksplit = t.ksplit;
            j.q = {pb, koff, ry, rx, f.nI, f.nJ, t.MT, n_ctiles, t.CC, t.NI * t.TRmax * t.TC, t.TC};
            GradXArgs &a = j.a;
            a.g = output_grad; a.x = input; a.dx = input_grad; a.pb = pb; a.koff = koff;
            a.B = p.B; a.C = p.C; a.H = p.H; a.W = p.W; a.O = p.O; a.oh = p.oh; a.ow = p.ow;
            a.nI = f.nI; a.nJ = f.nJ;
            a.padh = f.nI - 1 - f.a0; a.padw = f.nJ - 1 - f.b0;
            a.na = f.na; a.nb = f.nb;
            a.y0 = p.sh * f.a0 + ry - p.ph; a.x0 = p.sw * f.b0 + rx - p.pw;
            a.sh = p.sh; a.sw = p.sw;
            a.K = K;
            a.G = t.G; a.gpi = t.gpi; a.tiles = t.tiles; a.nws = t.nws;
            a.nws_log2 = t.nws == 4 ? 2 : (t.nws == 2 ? 1 : 0);
            a.n_ctiles = n_ctiles; a.TC = t.TC; a.TRmax = t.TRmax; a.CC = t.CC;
            a.ignore_nan = ignore_nan;
            a.fast_stage = t.fast_stage;
            a.NI = t.NI;
            // phase row h (a = a0 + h) is covered by some window iff a - (nI-1) <= oh-1
            a.row_limit = p.oh - 1 + f.nI - 1 - f.a0;
            a.col_limit = p.ow - 1 + f.nJ - 1 - f.b0;
            const int nwm = kWaves / t.nws;
            a.grid_x = t.ksplit ? (p.B + t.NI - 1) / t.NI : p.B * t.tiles;
            a.grid_y = t.ksplit ? n_ctiles : (n_ctiles + nwm - 1) / nwm;
            jobs.push_back(j);
        }
    std::vector<bool> done(jobs.size(), false);
    for (size_t first = 0; first < jobs.size(); ++first) {
        if (done[first])
            continue;
        GradXPhases ph;
        GxPackPhases pk;
        int n = 0;
        long long pack_total = 0;
        for (size_t i = first; i < jobs.size() && n < kGxMaxPhases; ++i)
            if (!done[i] && jobs[i].PT == jobs[first].PT && jobs[i].MT == jobs[first].MT &&
                jobs[i].ksplit == jobs[first].ksplit) {
                ph.p[n] = jobs[i].a;
                pk.p[n] = jobs[i].q;
                pack_total = std::max(pack_total, (long long)jobs[i].q.n_ctiles * (jobs[i].a.K + 1) * jobs[i].q.MT);
                done[i] = true;
                ++n;
            }
        const int pack_blocks = (int)std::min<long long>((pack_total + 255) / 256, 4096);
        hipLaunchKernelGGL(sim_grad_input_pack_kernel, dim3(pack_blocks, n), dim3(256), 0, s, templates, weights, p.O, p.C,
                           p.bh, p.bw, p.sh, p.sw, (int)l1, scale, pk);
        if (hipGetLastError() != hipSuccess)
            return SIMNETS_ERR_HIP;
        const hipError_t e = l1 ? gx_launch_phases<GX_L1>(ph, n, jobs[first].PT, jobs[first].MT, jobs[first].ksplit, s)
                                : gx_launch_phases<GX_L2>(ph, n, jobs[first].PT, jobs[first].MT, jobs[first].ksplit, s);
        if (e != hipSuccess)
            return SIMNETS_ERR_HIP;
    }
    return SIMNETS_OK;
}

// ------------------------------------------------------------------------------------------------
// parameter gradients
// ------------------------------------------------------------------------------------------------
namespace {

constexpr int PC = 32;        // output pixels per LDS chunk (two chunk buffers: the next one is filled while this one is used)
constexpr int PCP = PC + 1;   // row pitch of the LDS tiles in float4 units: one more than a multiple of the bank
                              // period, so the 8 rows a wave reads at once (same pixel) fall into distinct banks
constexpr int LO = 8, LK = 4; // templates x patch elements per lane

struct GradPArgs {
    const float *g, *x, *templates;
    float *partial;    // [nacc][S][Opad][Kpad], then one [Opad][Kpad] slab of centres (moment form)
    int B, C, H, W, O, oh, ow, bh, bw, sh, sw, ph, pw, K;
    int Opad, Kpad;    // O, K rounded up to the workgroup tile
    int n_ktiles, n_tiles;
    long long npix;    // B*oh*ow
    int nchunks, cps;  // pixel chunks in total, and per split
    int S;
    float oob;
};

// MODE: SimMode of the forward op.  WO: waves along the templates (1 or 2).
// MOM (L2 modes): moment form.  With a centre c per (lane, patch element) - the mean of the lane's 8 templates -
// and xc = x - c, tc = t - c, the sums over the pixels are
//     sum g (x - t)   = S1 - tc G            S1 = sum g xc,  S2 = sum g xc^2,  G = sum g
//     sum g (x - t)^2 = S2 - 2 tc S1 + tc^2 G
// so a term costs two fused multiply-adds (xc and xc^2 are shared by the lane's 8 templates) instead of four
// instructions; the finish kernel combines the moments in double precision.  The centre keeps tc of the order
// of the spread of the templates, which bounds the cancellation: the error is eps sqrt(N) |g| (xc^2 + tc^2),
// the same order as that of the term-by-term sums unless every template and every patch sit in one point.
// MOM (L1): scaled-sign form.  With dB = 2^64 (x - t) (one fma against the pre-scaled template; exact scaling),
// sign(x - t) = med3(dB, -1, 1) and |x - t| = 2^-64 |dB|: four instructions per term (fma, med3, fma, fma against
// g and 2^-64 g) instead of seven with compares and selects, bit-identical to them unless 0 < |x - t| < 2^-64,
// |g| < 2^-62 or a value beyond 2^63.  A pixel chunk with a NaN input (found while staging, uniform for the
// workgroup) takes the compare-and-select arithmetic, which has the reference's NaN rules.
// MF (with MOM, L2 modes): the moments on the fp32 matrix cores.  S1 = g^T xc, S2 = g^T xc^2 (and, with ignore-NaN,
// G = g^T keep) are contractions over the pixels: a wave's 64 templates x 32 patch elements are two
// v_mfma_f32_32x32x2_f32 tiles per moment, templates = rows, patch elements = columns, two pixels per instruction;
// the operands come from the same LDS chunks (one ds_read_b32 each: lane = (row or column, pixel parity)).  The
// centre is then per (wave, patch element): the mean over the wave's 64 templates.
// ROW (with MF; output width a multiple of the chunk of 32 pixels, so a chunk is a piece of one output row): g and
// the patch elements are staged row by row - a thread loads four consecutive pixels of a template row (one 16-byte
// load) or of a patch-element row (bounds per element, constants per row) - into [row][pixel] LDS tiles of pitch
// 34, instead of element by element with the im2col arithmetic per element.
template <int MODE, int WO, bool MOM, bool MF = false, bool ROW = false>
__global__ __launch_bounds__(kThreads, 2) void sim_grad_params_kernel(const GradPArgs a)
{
    static_assert(!MF || (MOM && MODE != SIM_MODE_L1), "the matrix-core form computes the moments of the L2 modes");
    static_assert(!ROW || MF, "row staging feeds the matrix-core form");
    constexpr bool MOM2 = MOM && MODE != SIM_MODE_L1;   // moment form of the L2 modes
    constexpr bool SGN = MOM && MODE == SIM_MODE_L1;    // scaled-sign form of L1
    constexpr int WK = kWaves / WO;
    constexpr int OWG = WO * 64, KWG = WK * 32;
    constexpr bool NORM = MODE == SIM_MODE_L2_NORM || MODE == SIM_MODE_L2_NORM_IGNORE_NAN;
    constexpr bool IGN = MODE == SIM_MODE_L2_NORM_IGNORE_NAN;
    constexpr bool L1 = MODE == SIM_MODE_L1;
    constexpr int PR = 34;  // row pitch of the [row][pixel] tiles: rows r and r + 1 start two banks apart
    __shared__ __attribute__((aligned(16))) float gs[2][ROW ? OWG * PR : OWG / 4 * PCP * 4];
    __shared__ __attribute__((aligned(16))) float xs[2][ROW ? KWG * PR : KWG / 4 * PCP * 4];
    __shared__ int ktab[KWG * 2];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wo = wave % WO, wk = wave / WO;
    const int lo = lane & 7, lk = lane >> 3;
    // blockIdx.x -> (pixel split, tile): the tiles of one split get ids that agree mod 8, so they run on the
    // same XCD close in time and share the split's g and x chunks through that XCD's L2.  Fewer than 8 splits
    // (1, 2 or 4: many tiles, few pixels) spread over all 8 XCDs, 8 / S of them per split.
    int split, tile_id;
    if (a.S >= 8) {
        const int per_super = 8 * a.n_tiles;
        const int super = blockIdx.x / per_super;
        const int within = blockIdx.x - super * per_super;
        tile_id = within >> 3;
        split = super * 8 + (within & 7);
        if (split >= a.S)
            return;  // padding of the last group of 8 splits (uniform for the workgroup)
    } else {
        const int xcd = blockIdx.x & 7;
        split = xcd & (a.S - 1);
        tile_id = (blockIdx.x >> 3) * (8 / a.S) + xcd / a.S;
        if (tile_id >= a.n_tiles)
            return;
    }
    const int ktile = tile_id % a.n_ktiles, otile = tile_id / a.n_ktiles;
    const int o_wg = otile * OWG, k_wg = ktile * KWG;

    // patch element k -> offset inside an image and tap coordinates
    const int bhw = a.bh * a.bw;
    for (int kk = tid; kk < KWG; kk += kThreads) {
        const int k = k_wg + kk;
        const int c = k / bhw;
        const int rem = k - c * bhw;
        const int i = rem / a.bw, j = rem - i * a.bw;
        ktab[2 * kk] = k < a.K ? (c * a.H + i) * a.W + j : -1;
        ktab[2 * kk + 1] = (i << 16) | j;
    }

    // this lane's templates
    // templates of this lane: LDS rows lo and lo + 8 of its wave's 16 (4 templates each).  The 8 lanes that
    // are served together then read 8 consecutive rows, whose pitch of PCP float4 walks through all banks.
    auto lane_o = [&](int oo) { return o_wg + wo * 64 + (oo >> 2) * 32 + lo * 4 + (oo & 3); };
    const int k0 = k_wg + wk * 32 + lk * LK;
    float t[LO][LK], at[LO][LK], aw[LO][LK], an[NORM ? LO : 1][NORM ? LK : 1];
#pragma unroll
    for (int oo = 0; oo < LO; ++oo)
#pragma unroll
        for (int kk = 0; kk < LK; ++kk) {
            // (a clamped address rather than a load inside the condition: each of those would be waited for in turn)
            if constexpr (!MF)
                t[oo][kk] = a.templates[(size_t)min(lane_o(oo), a.O - 1) * a.K + min(k0 + kk, a.K - 1)];
        }
#pragma unroll
    for (int oo = 0; oo < LO; ++oo)
#pragma unroll
        for (int kk = 0; kk < LK; ++kk) {
            const bool ok = !MF && lane_o(oo) < a.O && k0 + kk < a.K;
            t[oo][kk] = ok ? t[oo][kk] : 0.0f;
            if constexpr (SGN)
                t[oo][kk] *= 0x1p64f;
            at[oo][kk] = 0.0f;
            aw[oo][kk] = 0.0f;
            if constexpr (NORM)
                an[oo][kk] = 0.0f;
        }
    // moment form: centre per patch element of this lane
    float ctr[LK] = {0.0f, 0.0f, 0.0f, 0.0f};
    // matrix-core form: this lane's column (patch element) and pixel parity, the centre of the column, accumulators
    const int mcol = lane & 31, mhalf = lane >> 5;
    const int mk = k_wg + wk * 32 + mcol;
    float mctr = 0.0f;
    floatx16 ms1[2], ms2[2], msn[2];
    if constexpr (MF) {
        float m = 0.0f;
        int nvalid = 0;
        for (int r = 0; r < 64; ++r) {
            const int o = o_wg + wo * 64 + r;
            if (o < a.O && mk < a.K) {
                m += a.templates[(size_t)o * a.K + mk];
                ++nvalid;
            }
        }
        m *= 1.0f / (float)max(nvalid, 1);
        mctr = __builtin_fabsf(m) < __builtin_inff() ? m : 0.0f;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                ms1[i][v] = 0.0f; ms2[i][v] = 0.0f; msn[i][v] = 0.0f;
            }
    }
    if constexpr (MOM2 && !MF) {
        int nvalid = 0;
#pragma unroll
        for (int oo = 0; oo < LO; ++oo)
            nvalid += lane_o(oo) < a.O ? 1 : 0;
        const float inv = 1.0f / (float)max(nvalid, 1);
#pragma unroll
        for (int kk = 0; kk < LK; ++kk) {
            float m = 0.0f;
#pragma unroll
            for (int oo = 0; oo < LO; ++oo)
                m += t[oo][kk];  // 0 for the templates past the last one
            m *= inv;
            ctr[kk] = __builtin_fabsf(m) < __builtin_inff() ? m : 0.0f;  // a NaN/inf template stays its own affair
        }
    }

    const int ohow = a.oh * a.ow;
    constexpr int NSG = kThreads / PC;        // staging groups: thread (sp, sg) handles pixel sp, every NSG-th row
    constexpr int GR = OWG / 4 / NSG, XR = KWG / 4 / NSG;
    const int sp = tid % PC, sg = tid / PC;
    const int g_row = (wo * 16 + lo) * PCP, x_row = (wk * 8 + lk) * PCP;

    // global -> registers: the g values and the patch elements (im2col_3d rule: outside the image -> oob) of
    // pixel sp of a chunk, four templates / four patch elements per float4
    auto load_chunk = [&](int chunk, float4 (&gv)[GR], float4 (&xv)[XR]) {
        const long long q = (long long)chunk * PC + sp;
        const bool qok = q < a.npix;
        const long long qq = qok ? q : 0;
        const int b = (int)(qq / ohow);
        const int pix = (int)(qq - (long long)b * ohow);
        const int yo = pix / a.ow, xo = pix - yo * a.ow;
        const float *gb = a.g + ((size_t)b * a.O) * ohow + pix;
#pragma unroll
        for (int r = 0; r < GR; ++r) {
            const int o = o_wg + (sg + NSG * r) * 4;
            float e[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                e[u] = (qok && o + u < a.O) ? gb[(size_t)(o + u) * ohow] : 0.0f;
            gv[r] = make_float4(e[0], e[1], e[2], e[3]);
        }
        const int iy0 = yo * a.sh - a.ph, ix0 = xo * a.sw - a.pw;
        const float *xb = a.x + (size_t)b * a.C * a.H * a.W + (ptrdiff_t)iy0 * a.W + ix0;
#pragma unroll
        for (int r = 0; r < XR; ++r) {
            const int kk = (sg + NSG * r) * 4;
            float e[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int kofs = ktab[2 * (kk + u)], ij = ktab[2 * (kk + u) + 1];
                const int iy = iy0 + (ij >> 16), ix = ix0 + (ij & 0xffff);
                float val = 0.0f;
                if (qok && kofs >= 0) {
                    val = a.oob;
                    if (iy >= 0 && iy < a.H && ix >= 0 && ix < a.W)
                        val = xb[kofs];
                }
                e[u] = val;
            }
            xv[r] = make_float4(e[0], e[1], e[2], e[3]);
        }
    };
    // registers -> LDS buffer `buf`: g as [o/4][pixel][4], patch elements as [k/4][pixel][4]
    // moment form without ignore-NaN: sum of g per template.  Every chunk passes through store_chunk once, so the
    // staging thread adds up what it stores (its pixel sp of every chunk); the 32 pixel slots are added at the end.
    float4 gacc[GR];
#pragma unroll
    for (int r = 0; r < GR; ++r)
        gacc[r] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    auto store_chunk = [&](int buf, const float4 (&gv)[GR], const float4 (&xv)[XR]) {
#pragma unroll
        for (int r = 0; r < GR; ++r) {
            reinterpret_cast<float4 *>(gs[buf])[(sg + NSG * r) * PCP + sp] = gv[r];
            if constexpr (MOM2 && !IGN) {
                gacc[r].x += gv[r].x; gacc[r].y += gv[r].y; gacc[r].z += gv[r].z; gacc[r].w += gv[r].w;
            }
        }
#pragma unroll
        for (int r = 0; r < XR; ++r)
            reinterpret_cast<float4 *>(xs[buf])[(sg + NSG * r) * PCP + sp] = xv[r];
    };

    const int chunk_begin = split * a.cps;
    const int chunk_end = min((split + 1) * a.cps, a.nchunks);
    // matrix-core form, one chunk: two pixels per step, rows = templates (g at ga, second tile a1_off further),
    // columns = patch elements (xc, xc^2, keep from xb); `ps` floats from pixel to pixel; the reads of the next step
    // are issued before this step's matrix instructions
    // a wave whose 64 templates or 32 patch elements all lie past the last one only takes part in the staging
    // (few templates or patch elements: the first layer of a network)
    const bool wave_has_work = o_wg + wo * 64 < a.O && k_wg + wk * 32 < a.K;
    auto mfma_steps = [&](const float *ga_, int a1_off, const float *xb_, int ps) {
        float a0 = ga_[0], a1 = ga_[a1_off], xv_ = xb_[0];
#pragma unroll 4
        for (int p = 0; p < PC; p += 2) {
            const int pn = p + 2 < PC ? p + 2 : p;
            const float na0 = ga_[pn * ps], na1 = ga_[a1_off + pn * ps], nx = xb_[pn * ps];
            const bool ok = !IGN || xv_ == xv_;
            const float xc = ok ? xv_ - mctr : 0.0f;
            const float x2 = xc * xc;
            ms1[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, xc, ms1[0], 0, 0, 0);
            ms1[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, xc, ms1[1], 0, 0, 0);
            ms2[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, x2, ms2[0], 0, 0, 0);
            ms2[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, x2, ms2[1], 0, 0, 0);
            if constexpr (IGN) {
                const float keep1 = ok ? 1.0f : 0.0f;
                msn[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, keep1, msn[0], 0, 0, 0);
                msn[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, keep1, msn[1], 0, 0, 0);
            }
            a0 = na0; a1 = na1; xv_ = nx;
        }
    };
    if constexpr (ROW) {
        constexpr int RG = OWG / 32, RX = KWG / 32;
        const int rrow = tid >> 3, jq = tid & 7;   // rows rrow + 32 r; pixels 4 jq .. 4 jq + 3 of the chunk
        int kch[RX], kdh[RX], kdw[RX];             // this thread's patch-element rows: channel (-1: past K), tap
#pragma unroll
        for (int r = 0; r < RX; ++r) {
            const int k = k_wg + rrow + 32 * r;
            const int c = k / bhw, rem = k - c * bhw;
            kch[r] = k < a.K ? c : -1;
            kdh[r] = rem / a.bw;
            kdw[r] = rem - kdh[r] * a.bw;
        }
        float4 rg[RG];
        float rx[RX][4], gsum[RG];
#pragma unroll
        for (int r = 0; r < RG; ++r)
            gsum[r] = 0.0f;
        auto row_load = [&](int chunk) {
            // the chunk's first pixel (uniform): image, output row, first output column
            const long long q0 = (long long)chunk * PC;
            const int b = (int)(q0 / ohow);
            const int pix0 = (int)(q0 - (long long)b * ohow);
            const int yo = pix0 / a.ow, xo0 = pix0 - yo * a.ow;
#pragma unroll
            for (int r = 0; r < RG; ++r) {
                const int o = o_wg + rrow + 32 * r;
                rg[r] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (o < a.O)
                    rg[r] = *reinterpret_cast<const float4 *>(a.g + ((size_t)b * a.O + o) * ohow + pix0 + 4 * jq);
            }
#pragma unroll
            for (int r = 0; r < RX; ++r) {
                const int iy = yo * a.sh - a.ph + kdh[r];
                const bool row_ok = kch[r] >= 0 && iy >= 0 && iy < a.H;
                const float fill = kch[r] >= 0 ? a.oob : 0.0f;
                const float *row = a.x + (((size_t)b * a.C + max(kch[r], 0)) * a.H + (row_ok ? iy : 0)) * a.W;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int ix = (xo0 + 4 * jq + e) * a.sw - a.pw + kdw[r];
                    rx[r][e] = fill;
                    if (row_ok && ix >= 0 && ix < a.W)
                        rx[r][e] = row[ix];
                }
            }
        };
        auto row_store = [&](int buf) {
#pragma unroll
            for (int r = 0; r < RG; ++r) {
                float2 *d = reinterpret_cast<float2 *>(gs[buf] + (rrow + 32 * r) * PR + 4 * jq);
                d[0] = make_float2(rg[r].x, rg[r].y);
                d[1] = make_float2(rg[r].z, rg[r].w);
                if constexpr (!IGN)
                    gsum[r] += (rg[r].x + rg[r].y) + (rg[r].z + rg[r].w);
            }
#pragma unroll
            for (int r = 0; r < RX; ++r) {
                float2 *d = reinterpret_cast<float2 *>(xs[buf] + (rrow + 32 * r) * PR + 4 * jq);
                d[0] = make_float2(rx[r][0], rx[r][1]);
                d[1] = make_float2(rx[r][2], rx[r][3]);
            }
        };
        if (chunk_begin < chunk_end) {
            row_load(chunk_begin);
            row_store(0);
        }
        __syncthreads();
        for (int chunk = chunk_begin; chunk < chunk_end; ++chunk) {
            const int buf = (chunk - chunk_begin) & 1;
            const bool more = chunk + 1 < chunk_end;
            if (more)
                row_load(chunk + 1);   // in flight while this chunk is used
            if (wave_has_work)
                mfma_steps(gs[buf] + (wo * 64 + mcol) * PR + mhalf, 32 * PR, xs[buf] + (wk * 32 + mcol) * PR + mhalf, 1);
            if (more)
                row_store(buf ^ 1);
            __syncthreads();  // the other buffer is complete; nobody reads this one any more
        }
        if constexpr (!IGN) {
            // sum of g per template: the 8 pixel groups of a row, in group order; the finish kernel reads
            // patch-element tile 0's copy
#pragma unroll
            for (int r = 0; r < RG; ++r)
                gs[0][(rrow + 32 * r) * PR + jq] = gsum[r];
            __syncthreads();
            if (tid < OWG) {
                float sum = 0.0f;
                for (int q = 0; q < 8; ++q)
                    sum += gs[0][tid * PR + q];
                a.partial[((size_t)2 * a.S + split) * (size_t)a.Opad * a.Kpad + (size_t)(o_wg + tid) * a.Kpad + k_wg] = sum;
            }
        }
    }
    float4 gv[GR], xv[XR];
    __syncthreads();  // ktab written
    auto has_nan = [](const float4 (&xv)[XR]) {
        bool any = false;
#pragma unroll
        for (int r = 0; r < XR; ++r)
            any |= xv[r].x != xv[r].x || xv[r].y != xv[r].y || xv[r].z != xv[r].z || xv[r].w != xv[r].w;
        return any;
    };
    bool nan_chunk = false;  // scaled-sign form: the chunk in use holds a NaN input (uniform for the workgroup)
    if (chunk_begin < chunk_end && !ROW) {
        load_chunk(chunk_begin, gv, xv);
        store_chunk(0, gv, xv);
        if constexpr (SGN)
            nan_chunk = has_nan(xv);
    }
    if constexpr (SGN)
        nan_chunk = __syncthreads_or(nan_chunk);
    else
        __syncthreads();
    for (int chunk = chunk_begin; chunk < chunk_end && !ROW; ++chunk) {
        const int buf = (chunk - chunk_begin) & 1;
        const bool more = chunk + 1 < chunk_end;
        if (more)
            load_chunk(chunk + 1, gv, xv);   // in flight while this chunk is used
        const float4 *g4 = reinterpret_cast<const float4 *>(gs[buf]) + g_row;
        const float4 *x4 = reinterpret_cast<const float4 *>(xs[buf]) + x_row;

        // scaled-sign form of a pixel (chunks without NaN inputs)
        auto compute_sgn = [&](const float4 &ga, const float4 &gb2, const float4 &xq) {
            const float gl[LO] = {ga.x, ga.y, ga.z, ga.w, gb2.x, gb2.y, gb2.z, gb2.w};
            const float xl[LK] = {xq.x, xq.y, xq.z, xq.w};
            float gsc[LO];
#pragma unroll
            for (int oo = 0; oo < LO; ++oo)
                gsc[oo] = gl[oo] * 0x1p-64f;
#pragma unroll
            for (int oo = 0; oo < LO; ++oo)
#pragma unroll
                for (int kk = 0; kk < LK; ++kk) {
                    const float db = __builtin_fmaf(xl[kk], 0x1p64f, -t[oo][kk]);
                    const float sg = __builtin_amdgcn_fmed3f(db, -1.0f, 1.0f);
                    at[oo][kk] = __builtin_fmaf(sg, gl[oo], at[oo][kk]);
                    aw[oo][kk] = __builtin_fmaf(gsc[oo], __builtin_fabsf(db), aw[oo][kk]);
                }
        };
        // scaled-sign form, chunk with a NaN input: the compare-and-select arithmetic below on the templates scaled
        // back.  The factor is opaque to the compiler (set per pixel) so that the 32 products are formed where they
        // are used and not kept in registers.
        auto compute = [&](const float4 &ga, const float4 &gb2, const float4 &xq) {
            const float gl[LO] = {ga.x, ga.y, ga.z, ga.w, gb2.x, gb2.y, gb2.z, gb2.w};
            float xl[LK] = {xq.x, xq.y, xq.z, xq.w};
            float keep[LK];
            float unscale = 1.0f;
            if constexpr (SGN)
                asm volatile("v_mov_b32 %0, 0x1f800000" : "=v"(unscale));  // 2^-64
            if constexpr (MOM2) {
                float xc[LK], x2[LK];
#pragma unroll
                for (int kk = 0; kk < LK; ++kk) {
                    const bool ok = !IGN || xl[kk] == xl[kk];
                    keep[kk] = ok ? 1.0f : 0.0f;
                    xc[kk] = ok ? xl[kk] - ctr[kk] : 0.0f;
                    x2[kk] = xc[kk] * xc[kk];
                }
#pragma unroll
                for (int oo = 0; oo < LO; ++oo)
#pragma unroll
                    for (int kk = 0; kk < LK; ++kk) {
                        at[oo][kk] = __builtin_fmaf(gl[oo], xc[kk], at[oo][kk]);
                        aw[oo][kk] = __builtin_fmaf(gl[oo], x2[kk], aw[oo][kk]);
                        if constexpr (IGN)
                            an[oo][kk] = __builtin_fmaf(gl[oo], keep[kk], an[oo][kk]);
                    }
                return;
            }
            if (IGN) {
#pragma unroll
                for (int kk = 0; kk < LK; ++kk) {
                    const bool ok = xl[kk] == xl[kk];
                    keep[kk] = ok ? 1.0f : 0.0f;
                    xl[kk] = ok ? xl[kk] : 0.0f;
                }
            }
#pragma unroll
            for (int oo = 0; oo < LO; ++oo) {
                float d[LK], e[LK], gg[LK];
#pragma unroll
                for (int kk = 0; kk < LK; ++kk) {
                    d[kk] = xl[kk] - (SGN ? t[oo][kk] * unscale : t[oo][kk]);
                    gg[kk] = IGN ? gl[oo] * keep[kk] : gl[oo];
                }
                if (L1) {
#pragma unroll
                    for (int kk = 0; kk < LK; ++kk) {
                        float sgn = d[kk] < 0.0f ? -gg[kk] : gg[kk];
                        sgn = __builtin_islessgreater(d[kk], 0.0f) ? sgn : 0.0f;
                        at[oo][kk] += sgn;
                        aw[oo][kk] = __builtin_fmaf(gg[kk], __builtin_fabsf(d[kk]), aw[oo][kk]);
                    }
                } else {
#pragma unroll
                    for (int kk = 0; kk < LK; ++kk)
                        e[kk] = gg[kk] * d[kk];
#pragma unroll
                    for (int kk = 0; kk < LK; ++kk) {
                        at[oo][kk] += e[kk];
                        aw[oo][kk] = __builtin_fmaf(e[kk], d[kk], aw[oo][kk]);
                        if constexpr (NORM)
                            an[oo][kk] += gg[kk];
                    }
                }
            }
        };
        // one pixel ahead: the three reads of pixel p+1 are issued before the arithmetic of pixel p
        auto pixels = [&](auto &&fn) {
            float4 ga = g4[0], gb2 = g4[8 * PCP], xq = x4[0];
            for (int p = 0; p < PC; p += 2) {
                const float4 ga1 = g4[p + 1], gb1 = g4[8 * PCP + p + 1], xq1 = x4[p + 1];
                fn(ga, gb2, xq);
                const int pn = p + 2 < PC ? p + 2 : p;
                ga = g4[pn]; gb2 = g4[8 * PCP + pn]; xq = x4[pn];
                fn(ga1, gb1, xq1);
            }
        };
        if constexpr (MF) {
            if (wave_has_work)
                mfma_steps(gs[buf] + ((size_t)(wo * 16 + (mcol >> 2)) * PCP + mhalf) * 4 + (mcol & 3), 8 * PCP * 4,
                           xs[buf] + ((size_t)(wk * 8 + (mcol >> 2)) * PCP + mhalf) * 4 + (mcol & 3), 4);
        } else if (SGN && !nan_chunk) {
            pixels(compute_sgn);
        } else if (SGN) {
            // rare: one pixel at a time, no read-ahead (keeps this loop out of the register budget of the other)
#pragma unroll 1
            for (int p = 0; p < PC; ++p)
                compute(g4[p], g4[8 * PCP + p], x4[p]);
        } else {
            pixels(compute);
        }
        if (more)
            store_chunk(buf ^ 1, gv, xv);
        // the other buffer is complete; nobody reads this one any more
        if constexpr (SGN)
            nan_chunk = __syncthreads_or(more && has_nan(xv));
        else
            __syncthreads();
    }

    // partial sums of this split
    const size_t slab = (size_t)a.Opad * a.Kpad;
    float *pt = a.partial + (size_t)split * slab;
    float *pw = a.partial + ((size_t)a.S + split) * slab;
    float *pn = a.partial + ((size_t)2 * a.S + split) * slab;
    if constexpr (MF) {
        // tile i, register v: template row 8 (v / 4) + 4 * parity + v % 4, column mcol
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int orow = o_wg + wo * 64 + i * 32 + 8 * (v / 4) + 4 * mhalf + (v % 4);
                if (orow >= a.O || mk >= a.K)
                    continue;  // nobody reads the padding of the tile
                const size_t o = (size_t)orow * a.Kpad + mk;
                pt[o] = ms1[i][v];
                pw[o] = ms2[i][v];
                if constexpr (IGN)
                    pn[o] = msn[i][v];
                if (split == 0)
                    a.partial[(size_t)3 * a.S * slab + o] = mctr;
            }
    }
#pragma unroll
    for (int oo = 0; oo < LO && !MF; ++oo) {
        const size_t o = (size_t)lane_o(oo) * a.Kpad + k0;
        *reinterpret_cast<float4 *>(pt + o) = make_float4(at[oo][0], at[oo][1], at[oo][2], at[oo][3]);
        *reinterpret_cast<float4 *>(pw + o) = make_float4(aw[oo][0], aw[oo][1], aw[oo][2], aw[oo][3]);
        if constexpr (IGN || (NORM && !MOM))
            *reinterpret_cast<float4 *>(pn + o) = make_float4(an[oo][0], an[oo][1], an[oo][2], an[oo][3]);
        if constexpr (MOM2) {
            if (split == 0)
                *reinterpret_cast<float4 *>(a.partial + (size_t)3 * a.S * slab + o) =
                    make_float4(ctr[0], ctr[1], ctr[2], ctr[3]);
        }
    }
    if constexpr (MOM2 && !IGN && !ROW) {
        // pixel slots -> one sum per template, in slot order; the finish kernel reads patch-element tile 0's copy
        // (the loop's last barrier has passed: nobody reads gs any more)
#pragma unroll
        for (int r = 0; r < GR; ++r)
            reinterpret_cast<float4 *>(gs[0])[(sg + NSG * r) * PCP + sp] = gacc[r];
        __syncthreads();
        if (tid < OWG) {
            const float *row = gs[0] + (size_t)(tid >> 2) * PCP * 4 + (tid & 3);
            float sum = 0.0f;
            for (int q = 0; q < PC; ++q)
                sum += row[q * 4];
            pn[(size_t)(o_wg + tid) * a.Kpad + k_wg] = sum;
        }
    }
}

// Few templates over short patches (K <= 9 and O <= 4 * (32 / K): the first layer of the reference's networks, 32
// templates over 2 x 2 patches of one channel), L2 modes, moment form.  The tiled kernel above would run its 64 x 128
// (template x patch element) tile on 32 x 4 of them.  Here lanes are output pixels: a wave keeps the moments S1, S2
// (and, with NaN inputs ignored, G) of its 32 / K templates x K patch elements in registers - at most 96 accumulators -
// over the 64-pixel groups of its workgroup's pixel range, gathers a pixel's K patch elements once (im2col rule) and
// reads its templates' output gradients along the pixels; at the end the lanes' sums are added by a butterfly (a
// fixed order: reproducible) and lane 0 writes the split's partial sums in the layout the finish kernel reads.
// a.cps: pixels per split here (a multiple of 64).
constexpr int kGpSmallGroups = 4;   // groups of 64 pixels whose loads are in flight together
template <int MODE, int K>
__global__ __launch_bounds__(256) void sim_grad_params_small_kernel(const GradPArgs a)
{
    constexpr bool IGN = MODE == SIM_MODE_L2_NORM_IGNORE_NAN;
    constexpr int TPW = 32 / K;   // templates per wave
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int split = blockIdx.x;
    const int o0 = wave * TPW;
    // centre of the moments: the mean of the wave's templates, per patch element (see sim_grad_params_kernel)
    float ctr[K];
    {
        const int n = max(0, min(TPW, a.O - o0));
#pragma unroll
        for (int k = 0; k < K; ++k) {
            // (all loads first, those past the last template on a clamped address: a load inside the condition would
            // be waited for before the next one is issued)
            float tv[TPW];
#pragma unroll
            for (int i = 0; i < TPW; ++i)
                tv[i] = a.templates[(size_t)min(o0 + i, a.O - 1) * K + k];
            float sum = 0.0f;
#pragma unroll
            for (int i = 0; i < TPW; ++i)
                sum += i < n ? tv[i] : 0.0f;
            ctr[k] = n > 0 ? sum / (float)n : 0.0f;
        }
    }
    // patch element k -> channel and tap
    int kc[K], kdh[K], kdw[K];
    {
        const int bhw = a.bh * a.bw;
#pragma unroll
        for (int k = 0; k < K; ++k) {
            kc[k] = k / bhw;
            const int rem = k - kc[k] * bhw;
            kdh[k] = rem / a.bw;
            kdw[k] = rem - kdh[k] * a.bw;
        }
    }
    float s1[TPW][K], s2[TPW][K], gk[TPW][IGN ? K : 1];
#pragma unroll
    for (int i = 0; i < TPW; ++i) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            s1[i][k] = 0.0f;
            s2[i][k] = 0.0f;
        }
#pragma unroll
        for (int k = 0; k < (IGN ? K : 1); ++k)
            gk[i][k] = 0.0f;
    }
    const int plane = a.oh * a.ow;
    // (pixel numbers fit 32 bits: checked by the host)
    const unsigned p_begin = (unsigned)split * (unsigned)a.cps, p_end = min((unsigned)a.npix, p_begin + (unsigned)a.cps);
    // groups of 64 pixels, kGpSmallGroups at a time: all their loads go out before the first value is used (a group
    // is a dozen loads and a hundred fused multiply-adds: one memory round trip per group would be the kernel's time)
    for (unsigned pg = p_begin; pg < p_end; pg += 64 * kGpSmallGroups) {
        float xv[kGpSmallGroups][K], gv[kGpSmallGroups][TPW];
        bool inside[kGpSmallGroups][K], valid[kGpSmallGroups];
#pragma unroll
        for (int u = 0; u < kGpSmallGroups; ++u) {
            const unsigned p = pg + 64 * u + lane;
            valid[u] = p < p_end;
            const unsigned pc = valid[u] ? p : p_begin;
            const int b = (int)(pc / (unsigned)plane), rem = (int)(pc - (unsigned)b * (unsigned)plane);
            const int y = (int)((unsigned)rem / (unsigned)a.ow), xw = rem - y * a.ow;
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const int hi = y * a.sh - a.ph + kdh[k], wi = xw * a.sw - a.pw + kdw[k];
                inside[u][k] = hi >= 0 && hi < a.H && wi >= 0 && wi < a.W;
                xv[u][k] = a.x[inside[u][k] ? (((size_t)b * a.C + kc[k]) * a.H + hi) * a.W + wi : 0];
            }
#pragma unroll
            for (int i = 0; i < TPW; ++i)
                gv[u][i] = a.g[((size_t)b * a.O + min(o0 + i, a.O - 1)) * plane + rem];
        }
#pragma unroll
        for (int u = 0; u < kGpSmallGroups; ++u) {
#pragma unroll
            for (int k = 0; k < K; ++k) {
                float x = inside[u][k] ? xv[u][k] : a.oob;
                float keep = 1.0f;
                if constexpr (IGN) {
                    keep = x == x ? 1.0f : 0.0f;
                    x = x == x ? x : 0.0f;
                }
                if (!valid[u]) {   // a lane past the range adds nothing (and no NaN of a pixel that is not its own)
                    x = ctr[k];
                    keep = 0.0f;
                }
                const float xc = x - ctr[k], xc2 = xc * xc;
#pragma unroll
                for (int i = 0; i < TPW; ++i) {
                    float g = valid[u] && o0 + i < a.O ? gv[u][i] : 0.0f;
                    if constexpr (IGN) {
                        g *= keep;
                        gk[i][k] += g;
                    }
                    s1[i][k] = __builtin_fmaf(g, xc, s1[i][k]);
                    s2[i][k] = __builtin_fmaf(g, xc2, s2[i][k]);
                }
            }
            if constexpr (!IGN) {
#pragma unroll
                for (int i = 0; i < TPW; ++i)
                    gk[i][0] += valid[u] && o0 + i < a.O ? gv[u][i] : 0.0f;
            }
        }
    }
    // Sums over the lanes, in a fixed order, through the data-parallel-primitive lane patterns (neighbour, pair,
    // half-row mirror, row mirror: every lane then holds its 16-lane row's sum) and four lane reads for the rows -
    // all accumulators stage by stage, so that the stages' latencies overlap -, then the split's partial sums.
    auto dpp = [](float v, auto ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), decltype(ctrl)::value,
                                                                      0xF, 0xF, false));
    };
    auto lane_of = [](float v, int l) {
        return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
    };
    using std::integral_constant;
    auto wave_sum = [&](auto &arr, auto nk) {
        constexpr int NK = decltype(nk)::value;
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int k = 0; k < NK; ++k) arr[i][k] += dpp(arr[i][k], integral_constant<int, 0xB1>{});
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int k = 0; k < NK; ++k) arr[i][k] += dpp(arr[i][k], integral_constant<int, 0x4E>{});
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int k = 0; k < NK; ++k) arr[i][k] += dpp(arr[i][k], integral_constant<int, 0x141>{});
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int k = 0; k < NK; ++k) arr[i][k] += dpp(arr[i][k], integral_constant<int, 0x140>{});
#pragma unroll
        for (int i = 0; i < TPW; ++i)
#pragma unroll
            for (int k = 0; k < NK; ++k)
                arr[i][k] = (lane_of(arr[i][k], 0) + lane_of(arr[i][k], 16)) + (lane_of(arr[i][k], 32) + lane_of(arr[i][k], 48));
    };
    wave_sum(s1, integral_constant<int, K>{});
    wave_sum(s2, integral_constant<int, K>{});
    wave_sum(gk, integral_constant<int, IGN ? K : 1>{});
    // every lane holds all sums now: lane j keeps pair j = (template j / K, element j % K) and the wave writes each
    // array with one store (the slabs are unpadded here: a.Kpad = K, so the wave's pairs are consecutive floats)
    const size_t slab = (size_t)a.Opad * a.Kpad;
    float *pt = a.partial + (size_t)split * slab;
    float *pw = a.partial + ((size_t)a.S + split) * slab;
    float *pn = a.partial + ((size_t)2 * a.S + split) * slab;
    float m1 = 0.0f, m2 = 0.0f, mg = 0.0f, mc = 0.0f;
#pragma unroll
    for (int i = 0; i < TPW; ++i)
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const bool me = lane == i * K + k;
            m1 = me ? s1[i][k] : m1;
            m2 = me ? s2[i][k] : m2;
            mg = me ? gk[i][IGN ? k : 0] : mg;
            mc = me ? ctr[k] : mc;
        }
    const int my_o = o0 + lane / K, my_k = lane % K;
    if (lane < TPW * K && my_o < a.O) {
        const size_t at = (size_t)my_o * a.Kpad + my_k;
        pt[at] = m1;
        pw[at] = m2;
        if (IGN || my_k == 0)
            pn[at] = mg;
        if (split == 0)
            a.partial[(size_t)3 * a.S * slab + at] = mc;
    }
}

// Adds the partial sums in a fixed order and applies the pixel-independent factors.  256 threads = E elements x
// 256 / E groups (E = 32, or 8 when there are few elements): group j adds the splits j, j + G, ..., the group sums
// are added in group order through LDS.
// moment != 0: the partial sums are the moments S1, S2, G of sim_grad_params_kernel<.., MOM = true>.
__global__ __launch_bounds__(256) void sim_grad_params_finish_kernel(
    const float *__restrict__ partial, const float *__restrict__ templates, const float *__restrict__ weights, int O,
    int K, int Opad, int Kpad, int S, int mode, int moment, float fudge, int E, float *__restrict__ dT,
    float *__restrict__ dW)
{
    __shared__ float sm[3][256];
    const long long total = (long long)O * K;
    const size_t slab = (size_t)Opad * Kpad;
    const bool norm = mode == SIM_MODE_L2_NORM || mode == SIM_MODE_L2_NORM_IGNORE_NAN;
    const bool ign = mode == SIM_MODE_L2_NORM_IGNORE_NAN;
    const int G = 256 / E;
    const int e = threadIdx.x % E, grp = threadIdx.x / E;
    const long long idx = (long long)blockIdx.x * E + e;
    const bool live = idx < total;
    const int k = live ? (int)(idx % K) : 0;
    const int o = live ? (int)(idx / K) : 0;
    const size_t src = (size_t)o * Kpad + k;
    // where the sum of g lives: per (o, k) with ignore-NaN, else once per template (see the kernel's epilogue)
    const size_t gsrc = moment && !ign ? (size_t)o * Kpad : src;
    float st = 0.0f, sw = 0.0f, sn = 0.0f;
    if (live) {
        // eight splits' loads in flight at a time (a load per addition would be waited for each in turn); the additions
        // keep their order, a split past the end adds 0
        const bool third = norm || moment;
        for (int s0 = grp; s0 < S; s0 += 8 * G) {
            float a[8], b[8], c[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int s = s0 + u * G;
                const int sc = s < S ? s : grp;
                a[u] = partial[(size_t)sc * slab + src];
                b[u] = partial[((size_t)S + sc) * slab + src];
                c[u] = third ? partial[((size_t)2 * S + sc) * slab + gsrc] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const bool in = s0 + u * G < S;
                st += in ? a[u] : 0.0f;
                sw += in ? b[u] : 0.0f;
                sn += in ? c[u] : 0.0f;
            }
        }
    }
    sm[0][threadIdx.x] = st; sm[1][threadIdx.x] = sw; sm[2][threadIdx.x] = sn;
    __syncthreads();
    if (grp != 0 || !live)
        return;
    st = sw = sn = 0.0f;
    for (int j = 0; j < G; ++j) {
        st += sm[0][j * E + e]; sw += sm[1][j * E + e]; sn += sm[2][j * E + e];
    }
    if (moment) {
        const double tc = (double)templates[idx] - (double)partial[(size_t)3 * S * slab + src];
        const double s1 = st, s2 = sw, g = sn;
        st = (float)(s1 - tc * g);
        // an infinite second moment (infinite inputs, overflow) is the answer as it stands; the correction would
        // turn it into inf - inf
        sw = __builtin_isfinite(s2) ? (float)(s2 + tc * (tc * g - 2.0 * s1)) : sw;
    }
    const float w = weights[idx];
    if (mode == SIM_MODE_L1) {
        dT[idx] = w * st;
        dW[idx] = -sw;
    } else if (!norm) {
        dT[idx] = 2.0f * w * st;
        dW[idx] = -sw;
    } else {
        dT[idx] = w * st;
        dW[idx] = 0.5f * (sn / (w + fudge) - sw);
    }
}

struct GpTiling {
    int WO, OWG, KWG, n_otiles, n_ktiles, Opad, Kpad, nchunks, cps, S, nacc;
    bool small;   // few templates over short patches: sim_grad_params_small_kernel (cps: pixels per split)
    bool fast;    // unless the caller asked for the term-by-term arithmetic (algo DIRECT): moment form (L2 modes),
                  // scaled-sign form (L1)
    bool moment;  // fast and an L2 mode
};

GpTiling gp_tiling(const SimPlan &p)
{
    GpTiling t;
    t.WO = p.O > 64 ? 2 : 1;
    t.OWG = t.WO * 64;
    t.KWG = (kWaves / t.WO) * 32;
    t.n_otiles = (p.O + t.OWG - 1) / t.OWG;
    t.n_ktiles = (p.K + t.KWG - 1) / t.KWG;
    t.Opad = t.n_otiles * t.OWG;
    t.Kpad = t.n_ktiles * t.KWG;
    const long long npix = (long long)p.B * p.oh * p.ow;
    t.nchunks = (int)((npix + PC - 1) / PC);
    const int tiles = t.n_otiles * t.n_ktiles;
    t.fast = !p.exact_terms;
    t.moment = t.fast && p.mode != SIM_MODE_L1;
    // workgroups per launch: two rounds of 2 per compute unit for the vector forms, more and shorter ones for the
    // matrix-core form (measured on 256x64x32x32, 128 templates 3x3: 0.85 / 0.86 / 0.80 / 0.83 ms for 512 / 1024 /
    // 1536 / 2048)
    int S = std::max(1, (t.moment ? 1536 : 1024) / tiles);
    S = std::min(S, std::max(1, t.nchunks));
    // every split costs a prologue, an epilogue and a slab of partial sums: at least 8 chunks (256 pixels) per
    // split as long as that still leaves two workgroups per compute unit
    // (fewer than 8 chunks in all: one split, decided above; with more than 512 tiles the right-hand side is 0)
    if (t.nchunks >= 8 && t.nchunks / 8 >= 512 / tiles)
        S = std::min(S, t.nchunks / 8);
    S = std::max(S, 1);
    t.cps = (t.nchunks + S - 1) / S;
    t.S = t.cps > 0 ? (t.nchunks + t.cps - 1) / t.cps : 1;
    if (t.S < 8) {
        // a power of two, so that 8 / S XCDs serve each split (a split past the last chunk adds zeros)
        const int want = t.S >= 6 ? 8 : (t.S >= 3 ? 4 : t.S);
        int s2 = 1;
        while (s2 < want && s2 * 2 <= std::max(t.nchunks, 1))
            s2 *= 2;
        t.S = s2;
        t.cps = (std::max(t.nchunks, 1) + s2 - 1) / s2;
    }
    t.nacc = (t.moment || p.mode == SIM_MODE_L2_NORM || p.mode == SIM_MODE_L2_NORM_IGNORE_NAN) ? 3 : 2;
    t.small = t.moment && p.K >= 1 && p.K <= 9 && p.O <= 4 * (32 / p.K) && npix < 0x7fffffffLL;
    if (t.small) {
        // unpadded slabs; about 256 pixels per workgroup (one round of four groups of 64 per wave), at most 1024
        // workgroups
        t.Opad = p.O;
        t.Kpad = p.K;
        const long long want = std::max<long long>(1, std::min<long long>(1024, npix / 256));
        long long per = (npix + want - 1) / want;
        per = std::max<long long>(64, (per + 63) / 64 * 64);
        t.cps = (int)std::min<long long>(per, 0x7fffffc0LL);
        t.S = (int)std::max<long long>(1, (npix + t.cps - 1) / t.cps);
    }
    return t;
}

// workgroups of a launch: splits in groups of 8 (one per XCD) times the tiles; below 8 splits, 8 XCD slots times the
// tiles each slot takes
long long gp_blocks(const GpTiling &t)
{
    const long long tiles = (long long)t.n_otiles * t.n_ktiles;
    if (t.S >= 8)
        return (long long)(t.S + 7) / 8 * 8 * tiles;
    const int per_split = 8 / t.S;
    return 8 * ((tiles + per_split - 1) / per_split);
}

template <int MODE>
hipError_t gp_launch(const GradPArgs &a, const GpTiling &t, hipStream_t s)
{
    constexpr bool L2M = MODE != SIM_MODE_L1;
    if constexpr (L2M) {
        if (t.small) {
            const dim3 sgrid((unsigned)t.S);
#define SIMNETS_GP_SMALL(KK)                                                                                  \
    case KK:                                                                                                   \
        hipLaunchKernelGGL((sim_grad_params_small_kernel<MODE, KK>), sgrid, dim3(256), 0, s, a);               \
        break;
            switch (a.K) {
                SIMNETS_GP_SMALL(1) SIMNETS_GP_SMALL(2) SIMNETS_GP_SMALL(3) SIMNETS_GP_SMALL(4) SIMNETS_GP_SMALL(5)
                SIMNETS_GP_SMALL(6) SIMNETS_GP_SMALL(7) SIMNETS_GP_SMALL(8) SIMNETS_GP_SMALL(9)
            default: return hipErrorInvalidValue;
            }
#undef SIMNETS_GP_SMALL
            return hipGetLastError();
        }
    }
    dim3 grid((unsigned)gp_blocks(t));
    if (t.fast && L2M && a.ow % PC == 0) {
        if (t.WO == 2)
            hipLaunchKernelGGL((sim_grad_params_kernel<MODE, 2, true, L2M, L2M>), grid, dim3(kThreads), 0, s, a);
        else
            hipLaunchKernelGGL((sim_grad_params_kernel<MODE, 1, true, L2M, L2M>), grid, dim3(kThreads), 0, s, a);
    } else if (t.fast && L2M) {
        if (t.WO == 2)
            hipLaunchKernelGGL((sim_grad_params_kernel<MODE, 2, true, L2M>), grid, dim3(kThreads), 0, s, a);
        else
            hipLaunchKernelGGL((sim_grad_params_kernel<MODE, 1, true, L2M>), grid, dim3(kThreads), 0, s, a);
    } else if (t.fast) {
        if (t.WO == 2)
            hipLaunchKernelGGL((sim_grad_params_kernel<MODE, 2, true>), grid, dim3(kThreads), 0, s, a);
        else
            hipLaunchKernelGGL((sim_grad_params_kernel<MODE, 1, true>), grid, dim3(kThreads), 0, s, a);
    } else if (t.WO == 2) {
        hipLaunchKernelGGL((sim_grad_params_kernel<MODE, 2, false>), grid, dim3(kThreads), 0, s, a);
    } else {
        hipLaunchKernelGGL((sim_grad_params_kernel<MODE, 1, false>), grid, dim3(kThreads), 0, s, a);
    }
    return hipGetLastError();
}

}  // namespace

size_t sim_grad_params_workspace_bytes(const SimPlan &p)
{
    const GpTiling t = gp_tiling(p);
    return align_up(((size_t)t.nacc * t.S + (t.moment ? 1 : 0)) * t.Opad * t.Kpad * sizeof(float), 256);
}

int sim_grad_params(const SimPlan &p, const float *input, const float *templates, const float *weights,
                    const float *output_grad, float *templates_grad, float *weights_grad, void *workspace,
                    size_t workspace_bytes, void *stream)
{
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (workspace_bytes < sim_grad_params_workspace_bytes(p))
        return SIMNETS_ERR_WORKSPACE;
    const GpTiling t = gp_tiling(p);
    if (p.bh > 0xffff || p.bw > 0xffff || (!t.small && gp_blocks(t) > 0x7fffffffLL))
        return SIMNETS_ERR_TOO_LARGE;
    GradPArgs a;
    a.g = output_grad; a.x = input; a.templates = templates;
    a.partial = reinterpret_cast<float *>(workspace);
    a.B = p.B; a.C = p.C; a.H = p.H; a.W = p.W; a.O = p.O; a.oh = p.oh; a.ow = p.ow;
    a.bh = p.bh; a.bw = p.bw; a.sh = p.sh; a.sw = p.sw; a.ph = p.ph; a.pw = p.pw; a.K = p.K;
    a.Opad = t.Opad; a.Kpad = t.Kpad; a.n_ktiles = t.n_ktiles; a.n_tiles = t.n_otiles * t.n_ktiles;
    a.npix = (long long)p.B * p.oh * p.ow;
    a.nchunks = t.nchunks; a.cps = t.cps; a.S = t.S;
    a.oob = p.oob;
    hipError_t e;
    switch (p.mode) {
    case SIM_MODE_L1: e = gp_launch<SIM_MODE_L1>(a, t, s); break;
    case SIM_MODE_L2: e = gp_launch<SIM_MODE_L2>(a, t, s); break;
    case SIM_MODE_L2_NORM: e = gp_launch<SIM_MODE_L2_NORM>(a, t, s); break;
    default: e = gp_launch<SIM_MODE_L2_NORM_IGNORE_NAN>(a, t, s); break;
    }
    if (e != hipSuccess)
        return SIMNETS_ERR_HIP;
    const long long total = (long long)p.O * p.K;
    if (total == 0)
        return SIMNETS_OK;
    const int E = total <= 4096 ? 8 : 32;  // few elements: more threads per element
    if ((total + E - 1) / E > 0x7fffffffLL)
        return SIMNETS_ERR_TOO_LARGE;
    const unsigned blocks = (unsigned)((total + E - 1) / E);
    hipLaunchKernelGGL(sim_grad_params_finish_kernel, dim3(blocks), dim3(256), 0, s, a.partial, templates, weights,
                       p.O, p.K, t.Opad, t.Kpad, t.S, p.mode, t.moment ? 1 : 0, p.fudge, E, templates_grad, weights_grad);
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

}  // namespace simnets
