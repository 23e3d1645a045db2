// Similarity forward, plain L2 only, on the fp32 matrix cores (gfx950 v_mfma_f32_32x32x2_f32).
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
//   * input rows are staged, a few channels at a time, into LDS (out of image -> out_of_bounds_value,
//     shift applied); a lane reads the pixel operand with one ds_read_b32 per tile and k-pair and
//     squares it in the VALU, which is otherwise idle;
//   * the two k of an MFMA k-pair are the same tap (dh, dw) of two adjacent channels, so the
//     per-lane LDS address is base + uniform offset;
//   * the parameter operand is read straight from a pre-packed global array in consumption order
//     (L1/L2 resident: every workgroup walks it in the same order), two steps ahead of its use.
#include <hip/hip_runtime.h>

#include <algorithm>

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
constexpr int kStageChan = 4;            // channels whose loads are in flight at once while staging

struct MfmaArgs {
    const float *in;
    float *out;
    const float *pm;    // [step][type][half][Opad]
    const float *bias;  // [Opad]
    const float *ctr;   // [C] per-channel shift
    const float *x;     // input-gradient variant: the forward op's input (one value per output element)
    int x_channels;     // ... and its channel count (rows of the product that exist)
    int ignore_nan;     // ... NaN inputs get gradient 0
    int B, C, H, W, O, Opad, oh, ow, npix;
    int bh, bw, sh, sw, ph, pw;
    int tiles;          // workgroup pixel tiles per image
    int TC, TRmax, chan_lds, CC;
    float oob;
};

// GRAD: the same contraction machinery computes the input gradient of the L2 modes at stride 1.  With
// P0 = s w (t - c), P1 = s w (s = 2, or 1 with the normalization term; c = the channel's centre),
//   dX[b,ch,y,x] = sum_{m,dh,dw} g[b,m,y+ph-dh,x+pw-dw] (P0 - (X - c) P1)[m,ch,dh,dw] = A - (X[b,ch,y,x] - c) B,
// two products over (m, dh, dw) whose right operand is the output gradient read like an input image padded by
// (bh-1-ph, bw-1-pw) with zeros, taps flipped (src/kernels/similarity_grad_kernel_cpu.cpp:148-270 computes the
// same sums term by term).  Here the "image" is g (its channels are the templates), the rows are input channels:
// row tile 0 of a wave accumulates A and row tile 1 accumulates B for the same 32 channels, so a lane ends up
// with both values of an element and combines them with X at the store.
template <bool GRAD>
__global__ __launch_bounds__(kThreads, 2) void sim_mfma_kernel(const MfmaArgs a)
{
    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wp = wave >> 1;
    const int col = lane & 31, half = lane >> 5;

    const int b = blockIdx.x / a.tiles;
    const int tile = blockIdx.x - b * a.tiles;
    const int p_first = tile * WG_PIX;
    const int p_last = min(p_first + WG_PIX, a.npix) - 1;
    const int h_first = p_first / a.ow;
    const int nrows = p_last / a.ow - h_first + 1;
    const int TR = (nrows - 1) * a.sh + a.bh;
    const int in_row0 = h_first * a.sh - a.ph;
    const int mbase = GRAD ? blockIdx.y * (WG_TPL / 2) + wm * 32 : blockIdx.y * WG_TPL + wm * (RM * 32);

    // per pixel tile: LDS address of this lane's pixel (k-pair half folded in)
    int xbase[RP], pix[RP];
#pragma unroll
    for (int j = 0; j < RP; ++j) {
        const int p = p_first + (wp * RP + j) * 32 + col;
        pix[j] = p;
        const int pc = min(p, p_last);
        const int h = pc / a.ow, w = pc - h * a.ow;
        xbase[j] = (h - h_first) * a.sh * a.TC + w * a.sw + half * a.chan_lds;
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
    const float *pm = a.pm + half * a.Opad + mbase + col;
    const float *img = a.in + (size_t)b * a.C * a.H * a.W;

    float pw_cur[RM], pt_cur[RM], pw_nxt[RM], pt_nxt[RM];
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

    TilePositions<kStagePos> tp;
    tp.template init<kThreads>(a.H, a.W, TR, a.TC, in_row0, a.pw);

    for (int ch0 = 0; ch0 < a.C; ch0 += a.CC) {
        const int ccn = min(a.CC, a.C - ch0);
        const int ccp = (ccn + 1) & ~1;
        __syncthreads();
        stage_input_tile_fast<kStagePos, kStageChan>(lds, img, a.H, a.W, ch0, ccp, ccn, a.chan_lds, a.oob,
                                                     GRAD ? nullptr : a.ctr, tp);
        __syncthreads();

        // steps of this chunk in (channel pair, dh, dw) order; the pixel operand of step s+1 and the
        // parameter operand of step s+2 are requested before the MFMAs of step s are issued
        const int nsteps = (ccp / 2) * a.bh * a.bw;
        int dh = 0, dw = 0, row_off = 0, off = 0;
        float xn[RP];
#pragma unroll
        for (int j = 0; j < RP; ++j)
            xn[j] = lds[xbase[j]];
        for (int st = 0; st < nsteps; ++st) {
            float x[RP], x2[RP];
#pragma unroll
            for (int j = 0; j < RP; ++j)
                x[j] = xn[j];
            int ndw = dw + 1, ndh = dh, nrow = row_off;
            if (ndw == a.bw) {
                ndw = 0;
                ++ndh;
                nrow += a.TC;
                if (ndh == a.bh) {
                    ndh = 0;
                    nrow += 2 * a.chan_lds - a.bh * a.TC;
                }
            }
            int noff = nrow + ndw;
            if (st + 1 == nsteps)
                noff = off;
#pragma unroll
            for (int j = 0; j < RP; ++j)
                xn[j] = lds[xbase[j] + noff];
            float pw_nn[RM], pt_nn[RM];
            load_params(pm, pw_nn, pt_nn);
            pm += step_stride;
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (GRAD) {
#pragma unroll
                for (int j = 0; j < RP; ++j)
                    acc[0][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(pw_cur[0], x[j], acc[0][j], 0, 0, 0);
#pragma unroll
                for (int j = 0; j < RP; ++j)
                    acc[1][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(pt_cur[0], x[j], acc[1][j], 0, 0, 0);
            } else {
#pragma unroll
                for (int j = 0; j < RP; ++j)
                    x2[j] = x[j] * x[j];
#pragma unroll
                for (int i = 0; i < RM; ++i)
#pragma unroll
                    for (int j = 0; j < RP; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(pw_cur[i], x2[j], acc[i][j], 0, 0, 0);
#pragma unroll
                for (int i = 0; i < RM; ++i)
#pragma unroll
                    for (int j = 0; j < RP; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(pt_cur[i], x[j], acc[i][j], 0, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < RM; ++i) {
                if (GRAD && i > 0)
                    break;
                pw_cur[i] = pw_nxt[i]; pt_cur[i] = pt_nxt[i];
                pw_nxt[i] = pw_nn[i];  pt_nxt[i] = pt_nn[i];
            }
            dw = ndw; dh = ndh; row_off = nrow; off = noff;
        }
    }

    const size_t plane = (size_t)a.npix;
    if constexpr (GRAD) {
        // ---- store: lane holds A (tile 0) and B (tile 1) of 16 channels of one pixel ----
        float *ob = a.out + (size_t)b * a.x_channels * plane;
        const float *xb = a.x + (size_t)b * a.x_channels * plane;
#pragma unroll
        for (int j = 0; j < RP; ++j) {
            if (pix[j] > p_last)
                continue;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int ch = mbase + 8 * (v / 4) + 4 * half + (v % 4);
                if (ch >= a.x_channels)
                    continue;
                const float xin = xb[(size_t)ch * plane + pix[j]];
                float d = __builtin_fmaf(-(xin - a.ctr[ch]), acc[1][j][v], acc[0][j][v]);
                if (a.ignore_nan && xin != xin)
                    d = 0.0f;
                ob[(size_t)ch * plane + pix[j]] = d;
            }
        }
        return;
    }
    // ---- store: lane holds, per tile, 16 templates of one pixel ----
    float *ob = a.out + (size_t)b * a.O * plane;
#pragma unroll
    for (int j = 0; j < RP; ++j) {
        if (pix[j] > p_last)
            continue;
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

// Input-gradient variant: pm[step][type][half][Cpad], step = ((mpair * bh) + dh) * bw + dw over the flipped taps,
// template m = 2 * mpair + half, row = input channel: type 0 = s w (t - ctr), type 1 = s w.
__global__ void mfma_grad_pack_kernel(const float *__restrict__ templates, const float *__restrict__ weights,
                                      const float *__restrict__ ctr, int O, int C, int Cpad, int bh, int bw,
                                      float scale, long long total, float *__restrict__ pm)
{
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long long)gridDim.x * blockDim.x) {
        const int c = (int)(i % Cpad);
        long long r = i / Cpad;
        const int half = (int)(r & 1); r >>= 1;
        const int type = (int)(r & 1); r >>= 1;
        const int dw = (int)(r % bw); r /= bw;
        const int dh = (int)(r % bh);
        const int mpair = (int)(r / bh);
        const int m = 2 * mpair + half;
        float v = 0.0f;
        if (m < O && c < C) {
            const size_t idx = (((size_t)m * C + c) * bh + (bh - 1 - dh)) * bw + (bw - 1 - dw);
            const float w = scale * weights[idx];
            v = type == 0 ? w * (templates[idx] - ctr[c]) : w;
        }
        pm[i] = v;
    }
}

struct MfmaTiling {
    int Opad, steps, TC, TRmax, chan_lds, CC;
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
    // channel pitch = 32 mod 64 floats: the two k-pair halves of a wave land in disjoint LDS banks
    long long pitch = 1LL * t.TRmax * t.TC;
    pitch = (pitch + 31) / 64 * 64 + 32;
    if (pitch < 1LL * t.TRmax * t.TC)
        pitch += 64;
    t.ok = 2 * pitch <= kLdsBudgetFloats && 1LL * t.TRmax * t.TC <= kStagePos * kThreads;
    t.chan_lds = (int)pitch;
    int cc_max = t.ok ? (int)(kLdsBudgetFloats / pitch) & ~1 : 2;
    cc_max = std::min(cc_max, (p.C + 1) & ~1);
    const int chunks = (p.C + cc_max - 1) / cc_max;
    t.CC = ((p.C + chunks - 1) / chunks + 1) & ~1;
    // two steps of slack: the parameter loads run two steps ahead
    t.pm_floats = (size_t)(t.steps + 2) * 4 * t.Opad;
    return t;
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
    MfmaArgs a;
    a.in = input; a.out = output; a.pm = l.pm; a.bias = l.bias; a.ctr = l.ctr;
    a.B = p.B; a.C = p.C; a.H = p.H; a.W = p.W; a.O = p.O; a.Opad = t.Opad;
    a.oh = p.oh; a.ow = p.ow; a.npix = p.oh * p.ow;
    a.bh = p.bh; a.bw = p.bw; a.sh = p.sh; a.sw = p.sw; a.ph = p.ph; a.pw = p.pw;
    a.tiles = (a.npix + WG_PIX - 1) / WG_PIX;
    a.TC = t.TC; a.TRmax = t.TRmax; a.chan_lds = t.chan_lds; a.CC = t.CC;
    a.oob = p.oob;
    dim3 grid((unsigned)(p.B * a.tiles), (unsigned)(t.Opad / WG_TPL));
    const size_t lds_bytes = (size_t)t.CC * t.chan_lds * sizeof(float);
    hipLaunchKernelGGL(sim_mfma_kernel<false>, grid, dim3(kThreads), lds_bytes, s, a);
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

SimPlan grad_as_forward(const SimPlan &p)
{
    SimPlan q = p;
    q.C = p.O; q.H = p.oh; q.W = p.ow;
    q.O = p.C; q.oh = p.H; q.ow = p.W;
    q.ph = p.bh - 1 - p.ph; q.pw = p.bw - 1 - p.pw;
    q.K = p.O * p.bh * p.bw;
    return q;
}

}  // namespace

bool sim_mfma_grad_input_supported(const SimPlan &p)
{
    if (p.mode == SIM_MODE_L1 || p.exact_terms || p.sh != 1 || p.sw != 1 || p.ph > p.bh - 1 || p.pw > p.bw - 1)
        return false;
    // 32 channels per row tile, two templates per step: smaller problems leave the tiles mostly empty
    if (p.C < 24 || p.O < 8 || p.B == 0)
        return false;
    return mfma_grad_tiling(grad_as_forward(p)).ok;
}

size_t sim_mfma_grad_input_workspace_bytes(const SimPlan &p)
{
    const MfmaTiling t = mfma_grad_tiling(grad_as_forward(p));
    return align_up(t.pm_floats * sizeof(float), 256) + align_up((size_t)p.C * sizeof(float), 256);
}

int sim_mfma_grad_input_launch(const SimPlan &p, const float *input, const float *templates, const float *weights,
                               const float *output_grad, float *input_grad, void *workspace, size_t workspace_bytes,
                               void *stream)
{
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const SimPlan q = grad_as_forward(p);
    const MfmaTiling t = mfma_grad_tiling(q);
    if (!t.ok)
        return SIMNETS_ERR_ALGO;
    if (workspace_bytes < sim_mfma_grad_input_workspace_bytes(p))
        return SIMNETS_ERR_WORKSPACE;
    char *ws = reinterpret_cast<char *>(workspace);
    float *pm = reinterpret_cast<float *>(ws);
    float *ctr = reinterpret_cast<float *>(ws + align_up(t.pm_floats * sizeof(float), 256));
    const bool norm = p.mode == SIM_MODE_L2_NORM || p.mode == SIM_MODE_L2_NORM_IGNORE_NAN;
    hipLaunchKernelGGL(mfma_center_kernel, dim3(p.C), dim3(256), 0, s, templates, p.O, p.C, p.bh * p.bw, ctr);
    const long long total = (long long)t.pm_floats;
    hipLaunchKernelGGL(mfma_grad_pack_kernel, dim3((unsigned)std::min<long long>((total + 255) / 256, 8192)), dim3(256),
                       0, s, templates, weights, ctr, p.O, p.C, t.Opad, p.bh, p.bw, norm ? 1.0f : 2.0f, total, pm);
    if (hipGetLastError() != hipSuccess)
        return SIMNETS_ERR_HIP;

    MfmaArgs a;
    a.in = output_grad; a.out = input_grad; a.pm = pm; a.bias = nullptr; a.ctr = ctr;
    a.x = input; a.x_channels = p.C; a.ignore_nan = p.mode == SIM_MODE_L2_NORM_IGNORE_NAN;
    a.B = q.B; a.C = q.C; a.H = q.H; a.W = q.W; a.O = q.O; a.Opad = t.Opad;
    a.oh = q.oh; a.ow = q.ow; a.npix = q.oh * q.ow;
    a.bh = q.bh; a.bw = q.bw; a.sh = 1; a.sw = 1; a.ph = q.ph; a.pw = q.pw;
    a.tiles = (a.npix + WG_PIX - 1) / WG_PIX;
    a.TC = t.TC; a.TRmax = t.TRmax; a.chan_lds = t.chan_lds; a.CC = t.CC;
    a.oob = 0.0f;
    dim3 grid((unsigned)(q.B * a.tiles), (unsigned)(t.Opad / (WG_TPL / 2)));
    const size_t lds_bytes = (size_t)t.CC * t.chan_lds * sizeof(float);
    hipLaunchKernelGGL(sim_mfma_kernel<true>, grid, dim3(kThreads), lds_bytes, s, a);
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

}  // namespace simnets
