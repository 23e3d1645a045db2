// Similarity on the fp32 matrix cores (gfx950 v_mfma_f32_32x32x2_f32): the plain L2 forward (opt-in) and the input
// gradient of the L2 modes (sim_mfma_kernel<GRAD = true>, sim_mfma_grad_strided_kernel; described at the kernels).
//
// The weighted squared distance is expanded into dense contractions over k:
//   out[b,m,p] = -sum_k w (t - x)^2
//              = sum_k (-w[m,k]) * x[p,k]^2  +  sum_k (2 w[m,k] t[m,k]) * x[p,k]  -  sum_k w[m,k] t[m,k]^2
// i.e. one GEMM with K' = 2K whose left operand is the packed parameter matrix [-w | 2wt] and whose
// right operand is the implicit im2col matrix [x^2 ; x], plus a per-template bias.  Same operator as
// the direct kernel (src/kernels/similarity_kernel_gpu.cu:24-133 + sim_l2_forward,
// include/utils/similarity_utils.hpp:23-36 in the reference) but a different rounding path: the three
// sums cancel where a patch is close to a template, and NaN / Inf inputs do not marginalise, so this
// path is opt-in (SIMNETS_ALGO_MFMA) and is checked against the direct path.
// To keep the cancellation benign, templates and input are shifted per input channel by the mean
// template value of that channel before squaring ((t - c) - (x - c) = t - x).
//
// Work split: a workgroup of 4 waves owns 256 consecutive output pixels of one image and up to 128
// templates; wave (wm, wp) owns 64 templates x 128 pixels = 2 x 4 MFMA tiles of 32x32 (128
// accumulator VGPRs).  Templates are the MFMA row index and pixels the column index, so each lane
// ends up with 16 values of ONE pixel column and stores run along w: coalesced.
//   * input rows are staged, a chunk of channels at a time, into LDS (out of image -> out_of_bounds_value,
//     shift applied); a lane reads the pixel operand with one ds_read_b32 per tile and k-pair and
//     squares it in the VALU, which is otherwise idle;
//   * maps of at most 128 output pixels: the 256 pixel columns of a workgroup are the pixels of several images,
//     whose tiles sit side by side in a channel's LDS slot;
//   * the two k of an MFMA k-pair are the same tap (dh, dw) of two adjacent channels, so the
//     per-lane LDS address is base + uniform offset;
//   * the parameter operand is read straight from a pre-packed global array in consumption order
//     (L1/L2 resident: every workgroup walks it in the same order), two steps ahead of its use.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <vector>

#include "internal.h"
#include "stage.h"

namespace simnets {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int RM = 2;           // 32-template tiles per wave
constexpr int RP = 4;           // 32-pixel tiles per wave
constexpr int WG_PIX = 2 * RP * 32;   // 256 pixels per workgroup (2 pixel waves)
constexpr int WG_TPL = 2 * RM * 32;   // 128 templates per workgroup (2 template waves)
constexpr int kLdsBudgetFloats = 12288;  // 48 KiB input tile per workgroup
constexpr int kStagePos = 8;             // tile elements per thread and channel (at most kStagePos * 256 floats)
constexpr int kStageGroups = 2;          // channel groups whose loads are in flight at once while staging

// Geometry of one launch grid: the forward op's, or one stride phase of the input gradient.
struct MfmaGeom {
    int ow, npix;            // output grid width and size
    int bh, bw, sh, sw, ph, pw;
    int tiles;               // workgroup pixel tiles per image
    int TC, chan_lds, CC;
    int NI;                  // images per workgroup (maps of at most half a pixel tile; then tiles == 1), else 1
    int oy0, ox0;            // input gradient: first input row / column of the phase
    long long pm_off;        // this grid's packed operands inside pm, floats
};

constexpr int kMaxPhases = 16;
constexpr int kMaxTaps = 64;    // window size limit of the kernel that interleaves the stride phases
constexpr int kPmAhead = 8;     // ... and the steps per block of parameter operands it requests ahead

struct MfmaArgs {
    const float *in;
    float *out;
    const float *pm;    // [step][type][half][Opad]
    const float *bias;  // [Opad]
    const float *ctr;   // [C] per-channel shift
    const float *x;     // input-gradient variant: the forward op's input (one value per output element)
    int x_channels;     // ... and its channel count (rows of the product that exist)
    int ignore_nan;     // ... NaN inputs get gradient 0
    // ... where pixel (r, c) of a phase's grid sits in the forward op's input plane: row oy0 + r * oys,
    // column ox0 + c * oxs of a plane x_w wide and x_plane large (the whole plane at stride 1)
    int oys, oxs, x_w, x_plane;
    int B, C, H, W, O, Opad;
    int grid_tiles;     // pixel tiles per image in blockIdx.x (the largest phase's count)
    float oob;
    // input gradient with few workgroups: blockIdx.z = phase * nsplit + split, split s takes the chunks
    // [s n / nsplit, (s + 1) n / nsplit) of the output gradient's channels and writes its partial result to
    // part + s * part_stride (same layout as out); a second kernel adds the parts in order
    int nsplit;
    float *part;
    long long part_stride;
    MfmaGeom g;         // the forward op's grid
};

// The stride phases of one input-gradient launch, one per blockIdx.z.
struct MfmaPhases {
    MfmaGeom g[kMaxPhases];
};

// GRAD: the same contraction machinery computes the input gradient of the L2 modes.  At stride 1, with
// P0 = s w (t - c), P1 = s w (s = 2, or 1 with the normalization term; c = the channel's centre),
//   dX[b,ch,y,x] = sum_{m,dh,dw} g[b,m,y+ph-dh,x+pw-dw] (P0 - (X - c) P1)[m,ch,dh,dw] = A - (X[b,ch,y,x] - c) B,
// two products over (m, dh, dw) whose right operand is the output gradient read like an input image padded by
// (bh-1-ph, bw-1-pw) with zeros, taps flipped (src/kernels/similarity_grad_kernel_cpu.cpp:148-270 computes the
// same sums term by term).  Here the "image" is g (its channels are the templates), the rows are input channels:
// row tile 0 of a wave accumulates A and row tile 1 accumulates B for the same 32 channels, so a lane ends up
// with both values of an element and combines them with X at the store.
// At stride (sh, sw) the input pixels fall into sh * sw phases, (ry, rx) = ((y + ph) mod sh, (x + pw) mod sw).
// Only the taps dh = ry + sh a, dw = rx + sw b reach a pixel of that phase, and with Y = (y + ph - ry) / sh the
// window rows they come from are Y - a: each phase is a stride-1 problem of the same kind over its own taps,
// on the grid of its pixels, and gets a grid of its own (blockIdx.z) that stores to (and reads X at) the phase's
// pixels.
template <bool GRAD>
__global__ __launch_bounds__(kThreads, 2) void sim_mfma_kernel(const MfmaArgs a, const MfmaPhases phases)
{
    const int split = GRAD ? blockIdx.z % a.nsplit : 0;
    const MfmaGeom &g = GRAD ? phases.g[blockIdx.z / a.nsplit] : a.g;
    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wp = wave >> 1;
    const int col = lane & 31, half = lane >> 5;

    // a workgroup covers a tile of one image's pixels, or all pixels of g.NI images (positions = image, pixel)
    const bool multi = g.NI > 1;
    const int b = multi ? blockIdx.x * g.NI : blockIdx.x / a.grid_tiles;
    const int tile = multi ? 0 : blockIdx.x - b * a.grid_tiles;
    if (tile >= g.tiles || b >= a.B)
        return;  // a phase with fewer workgroups than the largest one
    const int nimg = multi ? min(g.NI, a.B - b) : 1;
    const int p_first = tile * WG_PIX;
    const int p_last = multi ? nimg * g.npix - 1 : min(p_first + WG_PIX, g.npix) - 1;
    const int h_first = p_first / g.ow;
    const int nrows = (multi ? g.npix - 1 : p_last) / g.ow - h_first + 1;
    const int TR = (nrows - 1) * g.sh + g.bh;
    const int in_row0 = h_first * g.sh - g.ph;
    const int mbase = GRAD ? blockIdx.y * (WG_TPL / 2) + wm * 32 : blockIdx.y * WG_TPL + wm * (RM * 32);

    // per pixel tile: LDS address of this lane's pixel (k-pair half folded in)
    int xbase[RP], pix[RP], pimg[RP];   // pixel inside its image, image (-1: none)
#pragma unroll
    for (int j = 0; j < RP; ++j) {
        const int p = p_first + (wp * RP + j) * 32 + col;
        const int pc = min(p, p_last);
        const int il = multi ? pc / g.npix : 0;
        const int pr = pc - il * g.npix;
        pix[j] = pr;
        pimg[j] = p <= p_last ? b + il : -1;
        const int h = pr / g.ow, w = pr - h * g.ow;
        xbase[j] = il * (TR * g.TC) + (h - h_first) * g.sh * g.TC + w * g.sw + half * g.chan_lds;
    }

    floatx16 acc[RM][RP];
#pragma unroll
    for (int i = 0; i < RM; ++i) {
        floatx16 init;
#pragma unroll
        for (int v = 0; v < 16; ++v)
            init[v] = GRAD ? 0.0f : a.bias[mbase + i * 32 + 8 * (v / 4) + 4 * half + (v % 4)];
#pragma unroll
        for (int j = 0; j < RP; ++j)
            acc[i][j] = init;
    }

    // parameter operand: this lane's element within a [type][half][Opad] step record
    const int step_stride = 4 * a.Opad;
    const float *pm = a.pm + g.pm_off + half * a.Opad + mbase + col;
    if (GRAD && a.nsplit > 1) {
        const int nchunks = (a.C + g.CC - 1) / g.CC;
        pm += (size_t)(split * nchunks / a.nsplit) * (g.CC / 2) * g.bh * g.bw * step_stride;
    }
    const float *img = a.in + (size_t)b * a.C * a.H * a.W;

    float pw_cur[RM], pt_cur[RM], pw_nxt[RM], pt_nxt[RM], pw_nn[RM], pt_nn[RM];
    auto load_params = [&](const float *p, float (&w_)[RM], float (&t_)[RM]) {
#pragma unroll
        for (int i = 0; i < RM; ++i) {
            if (GRAD && i > 0)
                break;  // one row tile of parameters: type 0 feeds accumulator tile 0, type 1 tile 1
            w_[i] = p[i * 32];
            t_[i] = p[2 * a.Opad + i * 32];
        }
    };
    load_params(pm, pw_cur, pt_cur);
    load_params(pm + step_stride, pw_nxt, pt_nxt);
    pm += 2 * step_stride;

    GroupedTile<kStagePos> gt;
    gt.template init<kThreads>(a.H, a.W, TR, g.TC, in_row0, g.pw, g.NI, nimg, multi ? a.C * a.H * a.W : 0, g.chan_lds, g.CC);

    // this workgroup's chunks of the image channels (all of them unless the input gradient is split)
    int ch_first = 0, ch_end = a.C;
    if (GRAD && a.nsplit > 1) {
        const int nchunks = (a.C + g.CC - 1) / g.CC;
        ch_first = split * nchunks / a.nsplit * g.CC;
        ch_end = min(a.C, (split + 1) * nchunks / a.nsplit * g.CC);
    }
    for (int ch0 = ch_first; ch0 < ch_end; ch0 += g.CC) {
        const int ccn = min(g.CC, a.C - ch0);
        const int ccp = (ccn + 1) & ~1;
        __syncthreads();
        gt.template stage<kStageGroups>(lds, img + (size_t)ch0 * a.H * a.W, a.H * a.W, ccp, ccn, g.chan_lds, a.oob,
                                      GRAD ? nullptr : a.ctr + ch0);
        __syncthreads();

        // steps of this chunk in (channel pair, dh, dw) order; the pixel operand of step s+1 and the
        // parameter operand of step s+2 are requested before the MFMAs of step s are issued
        const int nsteps = (ccp / 2) * g.bh * g.bw;
        int dh = 0, dw = 0, row_off = 0, off = 0;
        float xn[RP];
#pragma unroll
        for (int j = 0; j < RP; ++j)
            xn[j] = lds[xbase[j]];
        // one step: the MFMAs on the operands in (w_use, t_use), the parameter loads of the step after next into
        // (w_load, t_load)
        auto do_step = [&](int st, const float (&w_use)[RM], const float (&t_use)[RM], float (&w_load)[RM],
                           float (&t_load)[RM]) {
            float x[RP], x2[RP];
#pragma unroll
            for (int j = 0; j < RP; ++j)
                x[j] = xn[j];
            int ndw = dw + 1, ndh = dh, nrow = row_off;
            if (ndw == g.bw) {
                ndw = 0;
                ++ndh;
                nrow += g.TC;
                if (ndh == g.bh) {
                    ndh = 0;
                    nrow += 2 * g.chan_lds - g.bh * g.TC;
                }
            }
            int noff = nrow + ndw;
            if (st + 1 == nsteps)
                noff = off;
#pragma unroll
            for (int j = 0; j < RP; ++j)
                xn[j] = lds[xbase[j] + noff];
            load_params(pm, w_load, t_load);
            pm += step_stride;
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (GRAD) {
#pragma unroll
                for (int j = 0; j < RP; ++j)
                    acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(w_use[0], x[j], acc[0][j], 0, 0, 0);
#pragma unroll
                for (int j = 0; j < RP; ++j)
                    acc[1][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(t_use[0], x[j], acc[1][j], 0, 0, 0);
            } else {
#pragma unroll
                for (int j = 0; j < RP; ++j)
                    x2[j] = x[j] * x[j];
#pragma unroll
                for (int i = 0; i < RM; ++i)
#pragma unroll
                    for (int j = 0; j < RP; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(w_use[i], x2[j], acc[i][j], 0, 0, 0);
#pragma unroll
                for (int i = 0; i < RM; ++i)
#pragma unroll
                    for (int j = 0; j < RP; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(t_use[i], x[j], acc[i][j], 0, 0, 0);
            }
            dw = ndw; dh = ndh; row_off = nrow; off = noff;
        };
        // Three steps per round, the three parameter sets taking turns as (in use, next, being loaded): a load
        // lands in the registers it is consumed from two steps later, and is waited for there.  (With one set
        // moved to the next after every step, each move waited for loads issued a single step earlier.)
        int st = 0;
        for (; st + 3 <= nsteps; st += 3) {
            do_step(st, pw_cur, pt_cur, pw_nn, pt_nn);
            do_step(st + 1, pw_nxt, pt_nxt, pw_cur, pt_cur);
            do_step(st + 2, pw_nn, pt_nn, pw_nxt, pt_nxt);
        }
        for (; st < nsteps; ++st) {
            do_step(st, pw_cur, pt_cur, pw_nn, pt_nn);
#pragma unroll
            for (int i = 0; i < RM; ++i) {
                if (GRAD && i > 0)
                    break;
                pw_cur[i] = pw_nxt[i]; pt_cur[i] = pt_nxt[i];
                pw_nxt[i] = pw_nn[i];  pt_nxt[i] = pt_nn[i];
            }
        }
    }

    const size_t plane = (size_t)g.npix;
    if constexpr (GRAD) {
        // ---- store: lane holds A (tile 0) and B (tile 1) of 16 channels of one pixel ----
        const size_t xplane = (size_t)a.x_plane;
        float *out = a.nsplit > 1 ? a.part + split * a.part_stride : a.out;
        // (per pixel the 16 input values and channel centres are loaded first, on clamped channel indices, then the
        // 16 gradients are formed and stored: with each load under its channel bound, in front of its store, a lane
        // waited for 64 memory round trips in turn)
#pragma unroll
        for (int j = 0; j < RP; ++j) {
            if (pimg[j] < 0)
                continue;
            float *ob = out + (size_t)pimg[j] * a.x_channels * xplane;
            const float *xb = a.x + (size_t)pimg[j] * a.x_channels * xplane;
            const int pr = pix[j] / g.ow, pc = pix[j] - pr * g.ow;
            const size_t at = (size_t)(g.oy0 + pr * a.oys) * a.x_w + (g.ox0 + pc * a.oxs);
            float xin[16], cen[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int ch = min(mbase + 8 * (v / 4) + 4 * half + (v % 4), a.x_channels - 1);
                xin[v] = xb[(size_t)ch * xplane + at];
                cen[v] = a.ctr[ch];
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int ch = mbase + 8 * (v / 4) + 4 * half + (v % 4);
                if (ch >= a.x_channels)
                    continue;
                float d = __builtin_fmaf(-(xin[v] - cen[v]), acc[1][j][v], acc[0][j][v]);
                if (a.ignore_nan && xin[v] != xin[v])
                    d = 0.0f;
                ob[(size_t)ch * xplane + at] = d;
            }
        }
        return;
    }
    // ---- store: lane holds, per tile, 16 templates of one pixel ----
#pragma unroll
    for (int j = 0; j < RP; ++j) {
        if (pimg[j] < 0)
            continue;
        float *ob = a.out + (size_t)pimg[j] * a.O * plane;
#pragma unroll
        for (int i = 0; i < RM; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = mbase + i * 32 + 8 * (v / 4) + 4 * half + (v % 4);
                if (m < a.O)
                    ob[(size_t)m * plane + pix[j]] = acc[i][j][v];
            }
    }
}

// Input gradient at strides whose phases number two or four (1x2, 2x1, 2x2), all phases in one workgroup.
// Input pixel (y, x) = (sh Yb + ry, sw Xb + rx): the residue (ry, rx) names the phase, (Yb, Xb) the position on a
// grid common to all phases.  Tap (i, j) reaches the pixels of one phase only, those with (ry + ph - i) divisible by
// sh, and comes from window row Yb + (ry + ph - i) / sh: a fixed offset from the position for every tap.  A wave's
// four pixel tiles are its 32 positions in each of four phases (two phases: 2 x 32 positions each), so one staged
// tile of the output gradient serves every phase, and a step - one tap of one template pair - feeds the pixel
// tiles of the tap's phase.  q.tap[t] = (phase << 24) | LDS offset of tap t relative to the position.
struct MfmaStrideArgs {
    int nXb, npos, tiles;   // position grid: width, size, workgroup tiles per image
    int T;                  // taps (bh * bw <= kMaxTaps)
    int TC, chan_lds, CC;
    int row_min, col_min;   // window row / column of tile element (0, 0), relative to the first position row / column 0
    int row_ext;            // tile rows = position rows - 1 + row_ext
    int tap[kMaxTaps];
};

template <int NPH>
__global__ __launch_bounds__(kThreads, 2) void sim_mfma_grad_strided_kernel(const MfmaArgs a, const MfmaStrideArgs q)
{
    constexpr int PB = RP / NPH;          // 32-position blocks per wave
    constexpr int WG_POS = 2 * PB * 32;   // positions per workgroup (2 pixel waves)
    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wp = wave >> 1;
    const int col = lane & 31, half = lane >> 5;

    const int b = blockIdx.x / q.tiles;
    const int tile = blockIdx.x - b * q.tiles;
    const int p_first = tile * WG_POS;
    const int p_last = min(p_first + WG_POS, q.npos) - 1;
    const int h_first = p_first / q.nXb;
    const int nrows = p_last / q.nXb - h_first + 1;
    const int TR = nrows - 1 + q.row_ext;
    const int mbase = blockIdx.y * (WG_TPL / 2) + wm * 32;

    int xbase[PB], pos_h[PB], pos_w[PB];
#pragma unroll
    for (int j = 0; j < PB; ++j) {
        const int p = p_first + (wp * PB + j) * 32 + col;
        const int pc = min(p, p_last);
        const int h = pc / q.nXb, w = pc - h * q.nXb;
        pos_h[j] = p <= p_last ? h : -1;
        pos_w[j] = w;
        xbase[j] = (h - h_first) * q.TC + w + half * q.chan_lds;
    }

    floatx16 acc[2][RP];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < RP; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v)
                acc[i][j][v] = 0.0f;

    // parameter operand: [step][type][half][Cpad] in the order of use (chunk, tap, template pair)
    const int step_stride = 4 * a.Opad;
    // this workgroup's chunks of the output gradient's channels (all of them unless the contraction is split)
    const int split = blockIdx.z;
    int ch_first = 0, ch_end = a.C;
    if (a.nsplit > 1) {
        const int nchunks = (a.C + q.CC - 1) / q.CC;
        ch_first = split * nchunks / a.nsplit * q.CC;
        ch_end = min(a.C, (split + 1) * nchunks / a.nsplit * q.CC);
    }
    const float *pm = a.pm + half * a.Opad + mbase + col + (size_t)(ch_first / 2) * q.T * step_stride;
    const float *img = a.in + (size_t)b * a.C * a.H * a.W;
    float pa[kPmAhead], pb[kPmAhead];
#pragma unroll
    for (int i = 0; i < kPmAhead; ++i) {
        pa[i] = pm[i * step_stride];
        pb[i] = pm[i * step_stride + 2 * a.Opad];
    }

    GroupedTile<kStagePos> gt;
    gt.template init<kThreads>(a.H, a.W, TR, q.TC, h_first + q.row_min, -q.col_min, 1, 1, 0, q.chan_lds, q.CC);

    for (int ch0 = ch_first; ch0 < ch_end; ch0 += q.CC) {
        const int ccn = min(q.CC, a.C - ch0);
        const int ccp = (ccn + 1) & ~1;
        __syncthreads();
        gt.template stage<kStageGroups>(lds, img + (size_t)ch0 * a.H * a.W, a.H * a.W, ccp, ccn, q.chan_lds, 0.0f, nullptr);
        __syncthreads();

        // taps outside, template pairs inside: the inner loop has one phase and walks the channel slots of the tile
        const int np = ccp / 2;
        int e_next = q.tap[0];
        float xn[PB];
#pragma unroll
        for (int j = 0; j < PB; ++j)
            xn[j] = lds[xbase[j] + (e_next & 0xffffff)];
        for (int t = 0; t < q.T; ++t) {
            const int e_cur = e_next;
            e_next = q.tap[t + 1 < q.T ? t + 1 : t];
            const int off = e_cur & 0xffffff, off_next = e_next & 0xffffff;
            const int phase = e_cur >> 24;
#pragma unroll
            for (int f = 0; f < NPH; ++f) {
                if (phase != f)
                    continue;
                int lo = off;
                // blocks of kPmAhead steps: the parameters of the next block (which may belong to the next tap or
                // chunk: the stream is continuous) are requested before the first step of this one
                for (int mp0 = 0; mp0 < np; mp0 += kPmAhead) {
                    const int n = min(kPmAhead, np - mp0);
                    const float *pmn = pm + n * step_stride;
                    float qa[kPmAhead], qb[kPmAhead];
#pragma unroll
                    for (int u = 0; u < kPmAhead; ++u) {
                        qa[u] = pmn[u * step_stride];
                        qb[u] = pmn[u * step_stride + 2 * a.Opad];
                    }
#pragma unroll
                    for (int u = 0; u < kPmAhead; ++u) {
                        if (u >= n)
                            break;
                        float x[PB];
#pragma unroll
                        for (int j = 0; j < PB; ++j)
                            x[j] = xn[j];
                        lo += 2 * q.chan_lds;
                        const int noff = mp0 + u + 1 < np ? lo : off_next;
#pragma unroll
                        for (int j = 0; j < PB; ++j)
                            xn[j] = lds[xbase[j] + noff];
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int j = 0; j < PB; ++j)
                            acc[0][f * PB + j] =
                                __builtin_amdgcn_mfma_f32_32x32x2f32(pa[u], x[j], acc[0][f * PB + j], 0, 0, 0);
#pragma unroll
                        for (int j = 0; j < PB; ++j)
                            acc[1][f * PB + j] =
                                __builtin_amdgcn_mfma_f32_32x32x2f32(pb[u], x[j], acc[1][f * PB + j], 0, 0, 0);
                    }
                    pm = pmn;
#pragma unroll
                    for (int u = 0; u < kPmAhead; ++u) {
                        pa[u] = qa[u];
                        pb[u] = qb[u];
                    }
                }
            }
        }
    }

    // ---- store: lane holds A (tile 0) and B (tile 1) of 16 channels of one pixel per phase ----
    const size_t xplane = (size_t)a.x_plane;
    const int x_h = a.x_plane / a.x_w;
    float *ob = (a.nsplit > 1 ? a.part + split * a.part_stride : a.out) + (size_t)b * a.x_channels * xplane;
    const float *xb = a.x + (size_t)b * a.x_channels * xplane;
#pragma unroll
    for (int f = 0; f < NPH; ++f) {
        const int ry = f / a.oxs, rx = f - ry * a.oxs;
#pragma unroll
        for (int j = 0; j < PB; ++j) {
            const int y = pos_h[j] * a.oys + ry, xx = pos_w[j] * a.oxs + rx;
            if (pos_h[j] < 0 || y >= x_h || xx >= a.x_w)
                continue;
            const size_t at = (size_t)y * a.x_w + xx;
            float xin[16], cen[16];   // loaded first, on clamped channel indices (see sim_mfma_kernel)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int ch = min(mbase + 8 * (v / 4) + 4 * half + (v % 4), a.x_channels - 1);
                xin[v] = xb[(size_t)ch * xplane + at];
                cen[v] = a.ctr[ch];
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int ch = mbase + 8 * (v / 4) + 4 * half + (v % 4);
                if (ch >= a.x_channels)
                    continue;
                float d = __builtin_fmaf(-(xin[v] - cen[v]), acc[1][f * PB + j][v], acc[0][f * PB + j][v]);
                if (a.ignore_nan && xin[v] != xin[v])
                    d = 0.0f;
                ob[(size_t)ch * xplane + at] = d;
            }
        }
    }
}

// ctr[c] = mean over (m, dh, dw) of templates[m, c, dh, dw]
__global__ __launch_bounds__(256) void mfma_center_kernel(const float *__restrict__ templates, int O, int C, int bhw,
                                                          float *__restrict__ ctr)
{
    __shared__ float red[256];
    const int c = blockIdx.x;
    float s = 0.0f;
    const int n = O * bhw;
    for (int i = threadIdx.x; i < n; i += 256) {
        const int m = i / bhw, r = i - m * bhw;
        s += templates[((size_t)m * C + c) * bhw + r];
    }
    red[threadIdx.x] = s;
    __syncthreads();
    for (int d = 128; d > 0; d >>= 1) {
        if ((int)threadIdx.x < d)
            red[threadIdx.x] += red[threadIdx.x + d];
        __syncthreads();
    }
    if (threadIdx.x == 0)
        ctr[c] = red[0] / (float)n;
}

// pm[step][type][half][Opad], step = ((cpair * bh) + dh) * bw + dw, channel = 2 * cpair + half
__global__ void mfma_pack_kernel(const float *__restrict__ templates, const float *__restrict__ weights,
                                 const float *__restrict__ ctr, int O, int Opad, int C, int bh, int bw,
                                 long long total, float *__restrict__ pm)
{
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long long)gridDim.x * blockDim.x) {
        const int m = (int)(i % Opad);
        long long r = i / Opad;
        const int half = (int)(r & 1); r >>= 1;
        const int type = (int)(r & 1); r >>= 1;
        const int dw = (int)(r % bw); r /= bw;
        const int dh = (int)(r % bh);
        const int cpair = (int)(r / bh);
        const int c = 2 * cpair + half;
        float v = 0.0f;
        if (m < O && c < C) {
            const size_t idx = (((size_t)m * C + c) * bh + dh) * bw + dw;
            const float w = weights[idx];
            const float t = templates[idx] - ctr[c];
            v = type == 0 ? -w : 2.0f * w * t;
        }
        pm[i] = v;
    }
}

// bias[m] = -sum_k w (t - ctr)^2
__global__ __launch_bounds__(256) void mfma_bias_kernel(const float *__restrict__ templates,
                                                        const float *__restrict__ weights,
                                                        const float *__restrict__ ctr, int O, int C, int bhw,
                                                        float *__restrict__ bias)
{
    __shared__ float red[256];
    const int m = blockIdx.x;
    float s = 0.0f;
    if (m < O) {
        const int K = C * bhw;
        for (int k = threadIdx.x; k < K; k += 256) {
            const float t = templates[(size_t)m * K + k] - ctr[k / bhw];
            s += weights[(size_t)m * K + k] * t * t;
        }
    }
    red[threadIdx.x] = s;
    __syncthreads();
    for (int d = 128; d > 0; d >>= 1) {
        if ((int)threadIdx.x < d)
            red[threadIdx.x] += red[threadIdx.x + d];
        __syncthreads();
    }
    if (threadIdx.x == 0)
        bias[m] = -red[0];
}

// Input-gradient variant: pm[step][type][half][Cpad], step = ((mpair * na) + dh) * nb + dw over the flipped taps
// of one stride phase (tap rows ry + sh a, a < na, columns rx + sw b, b < nb; all bh x bw taps at stride 1),
// template m = 2 * mpair + half, row = input channel: type 0 = s w (t - ctr), type 1 = s w.  blockIdx.y = phase.
struct MfmaGradPack {
    struct Phase {
        int ry, rx, na, nb;
        long long pm_off, total;
    } p[kMaxPhases];
    long long max_floats;
};

__global__ void mfma_grad_pack_kernel(const float *__restrict__ templates, const float *__restrict__ weights,
                                      const float *__restrict__ ctr, int O, int C, int Cpad, int bh, int bw, int sh,
                                      int sw, float scale, const MfmaGradPack pk, float *__restrict__ pm)
{
    const MfmaGradPack::Phase &q = pk.p[blockIdx.y];
    pm += q.pm_off;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < q.total;
         i += (long long)gridDim.x * blockDim.x) {
        const int c = (int)(i % Cpad);
        long long r = i / Cpad;
        const int half = (int)(r & 1); r >>= 1;
        const int type = (int)(r & 1); r >>= 1;
        const int dw = (int)(r % q.nb); r /= q.nb;
        const int dh = (int)(r % q.na);
        const int mpair = (int)(r / q.na);
        const int m = 2 * mpair + half;
        float v = 0.0f;
        if (m < O && c < C) {
            const size_t idx =
                (((size_t)m * C + c) * bh + (q.ry + sh * (q.na - 1 - dh))) * bw + (q.rx + sw * (q.nb - 1 - dw));
            const float w = scale * weights[idx];
            v = type == 0 ? w * (templates[idx] - ctr[c]) : w;
        }
        pm[i] = v;
    }
}

// Parameters of the kernel that interleaves the stride phases: pm[step][type][half][Cpad] with the steps in the
// kernel's order: chunks of CC templates, inside a chunk the taps (i * bw + j, unflipped: the tap table holds where
// each tap reads), inside a tap the chunk's template pairs.
__global__ void mfma_grad_strided_pack_kernel(const float *__restrict__ templates, const float *__restrict__ weights,
                                              const float *__restrict__ ctr, int O, int C, int Cpad, int T, int CC,
                                              float scale, long long total, float *__restrict__ pm)
{
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long long)gridDim.x * blockDim.x) {
        const int c = (int)(i % Cpad);
        long long r = i / Cpad;
        const int half = (int)(r & 1); r >>= 1;
        const int type = (int)(r & 1); r >>= 1;
        // step r: chunk k covers the pairs [k CC/2, min((k+1) CC/2, pairs)), T * (pairs in the chunk) steps
        const long long per_chunk = (long long)(CC / 2) * T;
        const int chunk = (int)(r / per_chunk);
        const int in_chunk = (int)(r - chunk * per_chunk);
        const int np = min(CC / 2, (O + 1) / 2 - chunk * (CC / 2));
        int m = O;
        int tap = 0;
        if (np > 0 && in_chunk < np * T) {
            tap = in_chunk / np;
            m = 2 * (chunk * (CC / 2) + in_chunk - tap * np) + half;
        }
        float v = 0.0f;
        if (m < O && c < C) {
            const size_t idx = ((size_t)m * C + c) * T + tap;
            const float w = scale * weights[idx];
            v = type == 0 ? w * (templates[idx] - ctr[c]) : w;
        }
        pm[i] = v;
    }
}

// out[i] = part[0][i] + part[1][i] + ... in that order (the partial input gradients of a split contraction)
__global__ __launch_bounds__(256) void mfma_sum_parts_kernel(const float *__restrict__ part, int nsplit, long long n,
                                                             float *__restrict__ out)
{
    for (long long i = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4; i < n;
         i += (long long)gridDim.x * blockDim.x * 4) {
        if (i + 4 <= n && (n & 3) == 0 && (reinterpret_cast<size_t>(out) & 15) == 0) {
            float4 acc = *reinterpret_cast<const float4 *>(part + i);
            for (int z = 1; z < nsplit; ++z) {
                const float4 v = *reinterpret_cast<const float4 *>(part + z * n + i);
                acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
            }
            *reinterpret_cast<float4 *>(out + i) = acc;
        } else {
            for (long long k = i; k < min(i + 4, n); ++k) {
                float acc = part[k];
                for (int z = 1; z < nsplit; ++z)
                    acc += part[z * n + k];
                out[k] = acc;
            }
        }
    }
}

struct MfmaTiling {
    int Opad, steps, TC, TRmax, chan_lds, CC;
    int NI;   // images per workgroup (small maps), else 1
    bool ok;
    size_t pm_floats;
};

MfmaTiling mfma_tiling(const SimPlan &p)
{
    MfmaTiling t;
    t.Opad = (p.O + WG_TPL - 1) / WG_TPL * WG_TPL;
    t.steps = (p.C + 1) / 2 * p.bh * p.bw;
    t.TC = (p.ow - 1) * p.sw + p.bw;
    const int max_rows = std::min(p.oh, (WG_PIX + p.ow - 1) / p.ow + 1);
    t.TRmax = (max_rows - 1) * p.sh + p.bh;
    // maps of at most half a pixel tile: a workgroup takes several images, their tiles side by side in a channel slot
    t.NI = 1;
    const int npix = p.oh * p.ow;
    if (2 * npix <= WG_PIX && p.B >= 2) {
        const long long img_elems = 1LL * ((p.oh - 1) * p.sh + p.bh) * t.TC;
        int ni = std::min(WG_PIX / npix, p.B);
        while (ni > 1 && (ni * img_elems > kStagePos * kThreads || 2 * (ni * img_elems + 64) > kLdsBudgetFloats))
            --ni;
        t.NI = ni;
    }
    const long long per_chan = t.NI > 1 ? t.NI * 1LL * ((p.oh - 1) * p.sh + p.bh) * t.TC : 1LL * t.TRmax * t.TC;
    // channel pitch = 32 mod 64 floats: the two k-pair halves of a wave land in disjoint LDS banks
    long long pitch = per_chan;
    pitch = (pitch + 31) / 64 * 64 + 32;
    if (pitch < per_chan)
        pitch += 64;
    t.ok = 2 * pitch <= kLdsBudgetFloats && per_chan <= kStagePos * kThreads &&
           grouped_tile_fits(kStagePos * kThreads, per_chan, pitch, (p.C + 1) & ~1);
    t.chan_lds = (int)pitch;
    int cc_max = t.ok ? (int)(kLdsBudgetFloats / pitch) & ~1 : 2;
    cc_max = std::min(cc_max, (p.C + 1) & ~1);
    const int chunks = (p.C + cc_max - 1) / cc_max;
    t.CC = ((p.C + chunks - 1) / chunks + 1) & ~1;
    // the staging addresses a group of channels (and the images of a tile) with 32-bit offsets
    const long long group = std::max<long long>(1, std::min<long long>(kStagePos * kThreads / std::max<long long>(per_chan, 1), t.CC));
    if ((group + 1) * p.H * p.W + (t.NI > 1 ? 1LL * t.NI * p.C * p.H * p.W : 0) >= (1LL << 31))
        t.ok = false;
    // two steps of slack: the parameter loads run two steps ahead
    t.pm_floats = (size_t)(t.steps + 2) * 4 * t.Opad;
    return t;
}

MfmaGeom mfma_geom(const SimPlan &p, const MfmaTiling &t)
{
    MfmaGeom g = {};
    g.ow = p.ow; g.npix = p.oh * p.ow;
    g.bh = p.bh; g.bw = p.bw; g.sh = p.sh; g.sw = p.sw; g.ph = p.ph; g.pw = p.pw;
    g.tiles = (g.npix + WG_PIX - 1) / WG_PIX;
    g.TC = t.TC; g.chan_lds = t.chan_lds; g.CC = t.CC; g.NI = t.NI;
    return g;
}

}  // namespace

size_t sim_mfma_workspace_bytes(const SimPlan &p)
{
    const MfmaTiling t = mfma_tiling(p);
    return align_up(t.pm_floats * sizeof(float), 256) + align_up((size_t)t.Opad * sizeof(float), 256) +
           align_up((size_t)p.C * sizeof(float), 256);
}

namespace {
struct MfmaLayout {
    float *pm, *bias, *ctr;
};
MfmaLayout mfma_layout(const MfmaTiling &t, void *workspace)
{
    char *ws = reinterpret_cast<char *>(workspace);
    MfmaLayout l;
    l.pm = reinterpret_cast<float *>(ws);
    l.bias = reinterpret_cast<float *>(ws + align_up(t.pm_floats * sizeof(float), 256));
    l.ctr = reinterpret_cast<float *>(ws + align_up(t.pm_floats * sizeof(float), 256) +
                                      align_up((size_t)t.Opad * sizeof(float), 256));
    return l;
}
}  // namespace

// Writes the parameter-only part of the workspace: channel centres, packed operands, per-template bias.
int sim_mfma_prepare(const SimPlan &p, const float *templates, const float *weights, void *workspace,
                     size_t workspace_bytes, hipStream_t s)
{
    const MfmaTiling t = mfma_tiling(p);
    if (!t.ok)
        return SIMNETS_ERR_ALGO;  // image rows too long for the LDS tile of this path
    if (workspace_bytes < sim_mfma_workspace_bytes(p))
        return SIMNETS_ERR_WORKSPACE;
    const MfmaLayout l = mfma_layout(t, workspace);
    const int bhw = p.bh * p.bw;
    hipLaunchKernelGGL(mfma_center_kernel, dim3(p.C), dim3(256), 0, s, templates, p.O, p.C, bhw, l.ctr);
    const long long total = (long long)t.pm_floats;
    hipLaunchKernelGGL(mfma_pack_kernel, dim3((unsigned)std::min<long long>((total + 255) / 256, 8192)), dim3(256), 0, s,
                       templates, weights, l.ctr, p.O, t.Opad, p.C, p.bh, p.bw, total, l.pm);
    hipLaunchKernelGGL(mfma_bias_kernel, dim3(t.Opad), dim3(256), 0, s, templates, weights, l.ctr, p.O, p.C, bhw, l.bias);
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

int sim_mfma_run(const SimPlan &p, const float *input, float *output, void *workspace, size_t workspace_bytes,
                 hipStream_t s)
{
    const MfmaTiling t = mfma_tiling(p);
    if (!t.ok)
        return SIMNETS_ERR_ALGO;
    if (workspace_bytes < sim_mfma_workspace_bytes(p))
        return SIMNETS_ERR_WORKSPACE;
    const MfmaLayout l = mfma_layout(t, workspace);
    MfmaArgs a = {};
    a.in = input; a.out = output; a.pm = l.pm; a.bias = l.bias; a.ctr = l.ctr;
    a.B = p.B; a.C = p.C; a.H = p.H; a.W = p.W; a.O = p.O; a.Opad = t.Opad;
    a.g = mfma_geom(p, t);
    a.grid_tiles = a.g.tiles;
    a.oob = p.oob;
    a.nsplit = 1;
    dim3 grid((unsigned)(t.NI > 1 ? (p.B + t.NI - 1) / t.NI : p.B * a.g.tiles), (unsigned)(t.Opad / WG_TPL));
    const size_t lds_bytes = (size_t)t.CC * t.chan_lds * sizeof(float);
    hipLaunchKernelGGL(sim_mfma_kernel<false>, grid, dim3(kThreads), lds_bytes, s, a, MfmaPhases{});
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

int sim_mfma_launch(const SimPlan &p, const float *input, const float *templates, const float *weights, float *output,
                    void *workspace, size_t workspace_bytes, hipStream_t s)
{
    const int rc = sim_mfma_prepare(p, templates, weights, workspace, workspace_bytes, s);
    return rc ? rc : sim_mfma_run(p, input, output, workspace, workspace_bytes, s);
}

namespace {

// The product the input gradient needs, in the forward kernel's terms: the output gradient is the image (its
// channels are the templates), the input grid is the output grid, padding (bh-1-ph, bw-1-pw), stride 1.
MfmaTiling mfma_grad_tiling(const SimPlan &q)
{
    MfmaTiling t = mfma_tiling(q);
    // a workgroup covers 64 rows (channels) here: 2 waves x one 32-row tile for each of the two products
    t.Opad = (q.O + WG_TPL / 2 - 1) / (WG_TPL / 2) * (WG_TPL / 2);
    t.pm_floats = (size_t)(t.steps + 2) * 4 * t.Opad;
    return t;
}

// One stride phase of the input gradient as a stride-1 forward problem: the output gradient is the image (its
// channels are the templates), the phase's pixels are the output grid, the phase's taps the window.
struct GradPhase {
    SimPlan q;
    int ry, rx, na, nb;   // tap rows ry + sh a (a < na), tap columns rx + sw b (b < nb)
    int oy0, ox0;         // first input row / column of the phase
    MfmaTiling t;
};

// Phases with pixels, in (ry, rx) order.  Returns false when a phase with pixels has no tap (stride larger than
// the window: its gradient is zero and this path leaves it to the caller's other kernel).
bool grad_phases(const SimPlan &p, std::vector<GradPhase> &out)
{
    out.clear();
    for (int ry = 0; ry < p.sh; ++ry)
        for (int rx = 0; rx < p.sw; ++rx) {
            GradPhase g;
            g.ry = ry; g.rx = rx;
            g.na = ry < p.bh ? (p.bh - ry + p.sh - 1) / p.sh : 0;
            g.nb = rx < p.bw ? (p.bw - rx + p.sw - 1) / p.sw : 0;
            // pixels y = sh Y + ry - ph in [0, H): Y from Y0 = ceil((ph - ry) / sh) (>= 0 as ry < sh)
            const int Y0 = p.ph > ry ? (p.ph - ry + p.sh - 1) / p.sh : 0;
            const int X0 = p.pw > rx ? (p.pw - rx + p.sw - 1) / p.sw : 0;
            g.oy0 = p.sh * Y0 + ry - p.ph;
            g.ox0 = p.sw * X0 + rx - p.pw;
            const int nY = g.oy0 < p.H ? (p.H - 1 - g.oy0) / p.sh + 1 : 0;
            const int nX = g.ox0 < p.W ? (p.W - 1 - g.ox0) / p.sw + 1 : 0;
            if (nY <= 0 || nX <= 0)
                continue;
            if (g.na == 0 || g.nb == 0)
                return false;
            SimPlan q = p;
            q.C = p.O; q.H = p.oh; q.W = p.ow;
            q.O = p.C; q.oh = nY; q.ow = nX;
            q.bh = g.na; q.bw = g.nb; q.sh = 1; q.sw = 1;
            // phase row r reads window rows Y0 + r - a = r - (na - 1 - Y0) + (na - 1 - a)
            q.ph = g.na - 1 - Y0; q.pw = g.nb - 1 - X0;
            q.K = p.O * g.na * g.nb;
            g.q = q;
            g.t = mfma_grad_tiling(q);
            out.push_back(g);
        }
    return true;
}

// Tiling of the kernel that interleaves the stride phases (two or four of them, windows of at most kMaxTaps taps).
struct StrideTiling {
    bool ok;
    int nph, Cpad;
    size_t pm_floats, lds_bytes;
    MfmaStrideArgs q;
};

// residue r of an input coordinate that tap i reaches, and the window coordinate it comes from relative to the
// position: input = stride * position + r, (r + pad - i) divisible by stride, window = position + (r + pad - i) / stride
void stride_tap(int i, int stride, int pad, int *r, int *d)
{
    *r = ((i - pad) % stride + stride) % stride;
    *d = (*r + pad - i) / stride;   // exact division; negative for taps beyond the padding
}

StrideTiling stride_tiling(const SimPlan &p)
{
    StrideTiling t = {};
    t.nph = p.sh * p.sw;
    const int T = p.bh * p.bw;
    if ((t.nph != 2 && t.nph != 4) || p.sh > p.bh || p.sw > p.bw || T > kMaxTaps)
        return t;
    const int PB = RP / t.nph, wg_pos = 2 * PB * 32;
    const int nYb = (p.H + p.sh - 1) / p.sh, nXb = (p.W + p.sw - 1) / p.sw;
    int rmin = 1 << 30, rmax = -(1 << 30), cmin = 1 << 30, cmax = -(1 << 30);
    for (int i = 0; i < p.bh; ++i) {
        int r, d;
        stride_tap(i, p.sh, p.ph, &r, &d);
        rmin = std::min(rmin, d); rmax = std::max(rmax, d);
    }
    for (int j = 0; j < p.bw; ++j) {
        int r, d;
        stride_tap(j, p.sw, p.pw, &r, &d);
        cmin = std::min(cmin, d); cmax = std::max(cmax, d);
    }
    MfmaStrideArgs &q = t.q;
    q.nXb = nXb; q.npos = nYb * nXb; q.tiles = (q.npos + wg_pos - 1) / wg_pos;
    q.T = T;
    q.row_min = rmin; q.col_min = cmin; q.row_ext = rmax - rmin + 1;
    q.TC = nXb - 1 + (cmax - cmin + 1);
    const int max_rows = std::min(nYb, (wg_pos + nXb - 1) / nXb + 1);
    const int TRmax = max_rows - 1 + q.row_ext;
    long long pitch = 1LL * TRmax * q.TC;
    pitch = (pitch + 31) / 64 * 64 + 32;
    if (pitch < 1LL * TRmax * q.TC)
        pitch += 64;
    if (2 * pitch > kLdsBudgetFloats || 1LL * TRmax * q.TC > kStagePos * kThreads ||
        !grouped_tile_fits(kStagePos * kThreads, 1LL * TRmax * q.TC, pitch, (p.O + 1) & ~1))
        return t;
    q.chan_lds = (int)pitch;
    int cc_max = (int)(kLdsBudgetFloats / pitch) & ~1;
    cc_max = std::min(cc_max, (p.O + 1) & ~1);
    const int chunks = (p.O + cc_max - 1) / cc_max;
    q.CC = ((p.O + chunks - 1) / chunks + 1) & ~1;
    // the staging addresses a group of channels with 32-bit offsets
    const long long group = std::max<long long>(1, std::min<long long>(kStagePos * kThreads / (1LL * TRmax * q.TC), q.CC));
    if ((group + 1) * p.oh * p.ow >= (1LL << 31))
        return t;
    for (int i = 0; i < p.bh; ++i)
        for (int j = 0; j < p.bw; ++j) {
            int ry, dy, rx, dx;
            stride_tap(i, p.sh, p.ph, &ry, &dy);
            stride_tap(j, p.sw, p.pw, &rx, &dx);
            q.tap[i * p.bw + j] = ((ry * p.sw + rx) << 24) | ((dy - rmin) * q.TC + (dx - cmin));
        }
    t.Cpad = (p.C + WG_TPL / 2 - 1) / (WG_TPL / 2) * (WG_TPL / 2);
    t.pm_floats = ((size_t)((p.O + 1) / 2) * T + kPmAhead) * 4 * t.Cpad;
    t.lds_bytes = (size_t)q.CC * q.chan_lds * sizeof(float);
    t.ok = true;
    return t;
}

// The same split for the kernel that interleaves the stride phases.
int stride_split(const SimPlan &p, const StrideTiling &st)
{
    const long long wgs = (long long)p.B * st.q.tiles * (st.Cpad / (WG_TPL / 2));
    const int nchunks = (p.O + st.q.CC - 1) / st.q.CC;
    if (wgs >= 256)
        return 1;
    return (int)std::max<long long>(1, std::min<long long>(std::min(nchunks, 16), (512 + wgs - 1) / wgs));
}

// Workgroups along blockIdx.x of one phase's grid.
unsigned grad_phase_blocks(const SimPlan &p, const GradPhase &g)
{
    const int tiles = (g.q.oh * g.q.ow + WG_PIX - 1) / WG_PIX;
    return (unsigned)(g.t.NI > 1 ? (p.B + g.t.NI - 1) / g.t.NI : p.B * tiles);
}

// Small problems give the chip too few workgroups: the channels of the output gradient (the contraction) are then
// split over up to 16 workgroups whose partial results a second kernel adds in order.
int grad_split(const SimPlan &p, const std::vector<GradPhase> &ph)
{
    if (ph.empty())
        return 1;
    long long wgs = 0;
    int min_chunks = 1 << 30;
    for (const GradPhase &g : ph) {
        wgs += (long long)grad_phase_blocks(p, g) * (g.t.Opad / (WG_TPL / 2));
        min_chunks = std::min(min_chunks, (g.q.C + g.t.CC - 1) / g.t.CC);
    }
    if (wgs >= 256)
        return 1;
    return (int)std::max<long long>(1, std::min<long long>(std::min(min_chunks, 16), (512 + wgs - 1) / wgs));
}

}  // namespace

bool sim_mfma_grad_input_supported(const SimPlan &p)
{
    if (p.mode == SIM_MODE_L1 || p.exact_terms || p.ph > p.bh - 1 || p.pw > p.bw - 1)
        return false;
    // 32 channels per row tile, two templates per step: smaller problems leave the tiles mostly empty
    if (p.C < 24 || p.O < 8 || p.B == 0)
        return false;
    if (stride_tiling(p).ok)
        return true;
    std::vector<GradPhase> ph;
    if (p.sh * p.sw > kMaxPhases || !grad_phases(p, ph) || ph.empty())
        return false;
    for (const GradPhase &g : ph)
        if (!g.t.ok)
            return false;
    return true;
}

size_t sim_mfma_grad_input_workspace_bytes(const SimPlan &p)
{
    const StrideTiling st = stride_tiling(p);
    if (st.ok) {
        const int nsplit = stride_split(p, st);
        return align_up((size_t)p.C * sizeof(float), 256) + align_up(st.pm_floats * sizeof(float), 256) +
               (nsplit > 1 ? align_up((size_t)nsplit * p.B * p.C * p.H * p.W * sizeof(float), 256) : 0);
    }
    std::vector<GradPhase> ph;
    grad_phases(p, ph);
    size_t bytes = align_up((size_t)p.C * sizeof(float), 256);
    for (const GradPhase &g : ph)
        bytes += align_up(g.t.pm_floats * sizeof(float), 256);
    const int nsplit = grad_split(p, ph);
    if (nsplit > 1)
        bytes += align_up((size_t)nsplit * p.B * p.C * p.H * p.W * sizeof(float), 256);
    return bytes;
}

int sim_mfma_grad_input_launch(const SimPlan &p, const float *input, const float *templates, const float *weights,
                               const float *output_grad, float *input_grad, void *workspace, size_t workspace_bytes,
                               void *stream)
{
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const StrideTiling st = stride_tiling(p);
    if (st.ok) {
        if (workspace_bytes < sim_mfma_grad_input_workspace_bytes(p))
            return SIMNETS_ERR_WORKSPACE;
        char *ws = reinterpret_cast<char *>(workspace);
        float *ctr = reinterpret_cast<float *>(ws);
        float *pm = reinterpret_cast<float *>(ws + align_up((size_t)p.C * sizeof(float), 256));
        const bool norm = p.mode == SIM_MODE_L2_NORM || p.mode == SIM_MODE_L2_NORM_IGNORE_NAN;
        hipLaunchKernelGGL(mfma_center_kernel, dim3(p.C), dim3(256), 0, s, templates, p.O, p.C, p.bh * p.bw, ctr);
        const long long total = (long long)st.pm_floats;
        hipLaunchKernelGGL(mfma_grad_strided_pack_kernel, dim3((unsigned)std::min<long long>((total + 255) / 256, 8192)),
                           dim3(256), 0, s, templates, weights, ctr, p.O, p.C, st.Cpad, st.q.T, st.q.CC,
                           norm ? 1.0f : 2.0f, total, pm);
        MfmaArgs a = {};
        a.in = output_grad; a.out = input_grad; a.pm = pm; a.ctr = ctr;
        a.x = input; a.x_channels = p.C; a.ignore_nan = p.mode == SIM_MODE_L2_NORM_IGNORE_NAN;
        a.oys = p.sh; a.oxs = p.sw; a.x_w = p.W; a.x_plane = p.H * p.W;
        a.B = p.B; a.C = p.O; a.H = p.oh; a.W = p.ow; a.O = p.C; a.Opad = st.Cpad;
        const long long n_in = (long long)p.B * p.C * p.H * p.W;
        a.nsplit = stride_split(p, st);
        a.part = reinterpret_cast<float *>(ws + align_up((size_t)p.C * sizeof(float), 256) +
                                           align_up(st.pm_floats * sizeof(float), 256));
        a.part_stride = n_in;
        dim3 grid((unsigned)(p.B * st.q.tiles), (unsigned)(st.Cpad / (WG_TPL / 2)), (unsigned)a.nsplit);
        if (st.nph == 4)
            hipLaunchKernelGGL(sim_mfma_grad_strided_kernel<4>, grid, dim3(kThreads), st.lds_bytes, s, a, st.q);
        else
            hipLaunchKernelGGL(sim_mfma_grad_strided_kernel<2>, grid, dim3(kThreads), st.lds_bytes, s, a, st.q);
        if (a.nsplit > 1)
            hipLaunchKernelGGL(mfma_sum_parts_kernel, dim3((unsigned)std::min<long long>((n_in + 1023) / 1024, 4096)),
                               dim3(256), 0, s, a.part, a.nsplit, n_in, input_grad);
        return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
    }
    std::vector<GradPhase> phases;
    if (!grad_phases(p, phases) || phases.empty())
        return SIMNETS_ERR_ALGO;
    for (const GradPhase &g : phases)
        if (!g.t.ok)
            return SIMNETS_ERR_ALGO;
    if (workspace_bytes < sim_mfma_grad_input_workspace_bytes(p))
        return SIMNETS_ERR_WORKSPACE;
    char *ws = reinterpret_cast<char *>(workspace);
    float *ctr = reinterpret_cast<float *>(ws);
    ws += align_up((size_t)p.C * sizeof(float), 256);
    const bool norm = p.mode == SIM_MODE_L2_NORM || p.mode == SIM_MODE_L2_NORM_IGNORE_NAN;
    hipLaunchKernelGGL(mfma_center_kernel, dim3(p.C), dim3(256), 0, s, templates, p.O, p.C, p.bh * p.bw, ctr);
    MfmaArgs a = {};
    MfmaPhases ph = {};
    MfmaGradPack pk = {};
    const int Cpad = phases[0].t.Opad;
    long long pm_off = 0;
    size_t lds_bytes = 0;
    unsigned blocks_x = 0;
    for (size_t i = 0; i < phases.size(); ++i) {
        const GradPhase &g = phases[i];
        ph.g[i] = mfma_geom(g.q, g.t);
        ph.g[i].oy0 = g.oy0; ph.g[i].ox0 = g.ox0;
        ph.g[i].pm_off = pm_off;
        pk.p[i] = {g.ry, g.rx, g.na, g.nb, pm_off, (long long)g.t.pm_floats};
        pm_off += (long long)(align_up(g.t.pm_floats * sizeof(float), 256) / sizeof(float));
        if (g.t.NI == 1)
            a.grid_tiles = std::max(a.grid_tiles, ph.g[i].tiles);
        blocks_x = std::max(blocks_x, grad_phase_blocks(p, g));
        lds_bytes = std::max(lds_bytes, (size_t)g.t.CC * g.t.chan_lds * sizeof(float));
        pk.max_floats = std::max(pk.max_floats, (long long)g.t.pm_floats);
    }
    a.grid_tiles = std::max(a.grid_tiles, 1);
    float *pm = reinterpret_cast<float *>(ws);
    hipLaunchKernelGGL(mfma_grad_pack_kernel,
                       dim3((unsigned)std::min<long long>((pk.max_floats + 255) / 256, 4096), (unsigned)phases.size()),
                       dim3(256), 0, s, templates, weights, ctr, p.O, p.C, Cpad, p.bh, p.bw, p.sh, p.sw,
                       norm ? 1.0f : 2.0f, pk, pm);
    const long long n_in = (long long)p.B * p.C * p.H * p.W;
    a.nsplit = grad_split(p, phases);
    a.part = reinterpret_cast<float *>(ws + (size_t)pm_off * sizeof(float));
    a.part_stride = n_in;
    a.in = output_grad; a.out = input_grad; a.pm = pm; a.bias = nullptr; a.ctr = ctr;
    a.x = input; a.x_channels = p.C; a.ignore_nan = p.mode == SIM_MODE_L2_NORM_IGNORE_NAN;
    a.oys = p.sh; a.oxs = p.sw; a.x_w = p.W; a.x_plane = p.H * p.W;
    a.B = p.B; a.C = p.O; a.H = p.oh; a.W = p.ow; a.O = p.C; a.Opad = Cpad;
    a.oob = 0.0f;
    dim3 grid(blocks_x, (unsigned)(Cpad / (WG_TPL / 2)), (unsigned)(phases.size() * a.nsplit));
    hipLaunchKernelGGL(sim_mfma_kernel<true>, grid, dim3(kThreads), lds_bytes, s, a, ph);
    if (a.nsplit > 1)
        hipLaunchKernelGGL(mfma_sum_parts_kernel, dim3((unsigned)std::min<long long>((n_in + 1023) / 1024, 4096)),
                           dim3(256), 0, s, a.part, a.nsplit, n_in, input_grad);
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

}  // namespace simnets
