// MEX backward (gfx950): gradients w.r.t. the input and w.r.t. the offsets.
//
// Replaces MEXGradInputKernelGPU / MEXGradOffsetsKernelGPU (src/kernels/mex_grad_kernel_gpu.cu), i.e.
// per image im2col_3d_gpu + split_patches + ggemm_readc_gpu with mex_backward_bottom_finite /
// _infinite (include/utils/mex_utils.hpp:31-46) + reverse split_patches + col2im_3d_gpu (input) or
// the accumulation over images (offsets), by one launch over the whole batch each.
//
// Both gradients are sums of the same term
//   e(px, m, k) = g[px,m] * exp(eps * (patch(px)[k] + off[r(px),m,k] - out[px,m]) + ey)        finite eps
//               = g[px,m] * (patch(px)[k] + off[r(px),m,k] == out[px,m])                        eps = +-inf
//   d patch(px)[k]  = sum_m e(px, m, k)          (then stored to the input element the patch element is; patches
//                                                 that overlap are added per element by mex_col2im_kernel)
//   d off[r, m, k]  = sum_{px in region r} e(px, m, k)
// Output pixels are enumerated region-major exactly like the forward kernel does, a lane owns
// pixel slots, so the offsets a wave needs are the same for all its lanes (scalar loads).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>

#include "internal.h"
#include "mex_common.h"
#include "valu_tile.h"

namespace simnets {

namespace {

struct MexGradArgs {
    MexKernelArgs k;       // geometry; k.in = input, k.out unused
    const float *off;      // [R][M][K] offsets as the forward op used them
    const float *out;      // forward output
    const float *g;        // output gradient
    int gpool;             // g is the gradient of the 2 x 2 sum-pooled output, [B][M][H/2][W/2]: the gradient of output
                           // pixel (h, w) is its window's, g[h / 2][w / 2]
    float *dx;             // input gradient
    float *partial;        // offsets gradient partial sums [chunk][R][M][K]
    int overlap;           // patches overlap: the per-patch gradients go to `col`, mex_col2im_kernel adds them up
    float *col;            // [B][Co*Ho*Wo][K] gradient of every patch element (overlapping patches only)
    int cpr;               // pixel chunks per region
    int msplit;            // input gradient: the instances are split over gridDim.z workgroups (1: no split) ...
    int mg_per_split;      // ... of this many packed groups (GM_TM instances) each, which write their partial
    float *dx_splits;      // gradients to [split][input] for mex_sum_splits_kernel
    // Factor buffers (finite epsilon, optional): the pixel factors W [R][slots_pad][Mp] and the patch exponentials
    // EX [R][slots_pad][Kp] of mex_grad_factors_kernel, which the matrix kernels then load instead of forming them
    // (again and again: once per tile of the other dimension).  nullptr: the kernels form them themselves.
    float *wbuf, *exbuf;
    int slots_pad, Mp, Kp;
    int pxl;               // pixel slots per lane (offsets gradient)
};

// Output gradient given as the gradient of the 2 x 2 sum-pooled output (ga.gpool; one output channel per instance,
// even height and width): plane size and the offset of output pixel `out_off`'s window.
__device__ __forceinline__ size_t pooled_g_plane(const MexGradArgs &ga, size_t plane)
{
    return ga.gpool ? plane >> 2 : plane;
}

__device__ __forceinline__ int pooled_g_offset(const MexGradArgs &ga, int out_off)
{
    if (!ga.gpool)
        return out_off;
    const int h = out_off / ga.k.Wo, w = out_off - h * ga.k.Wo;
    return (h >> 1) * (ga.k.Wo >> 1) + (w >> 1);
}

// patch element k of the pixel -> value (im2col_3d rule) and, if inside the image, its offset from the
// image start; -1 otherwise
__device__ __forceinline__ float patch_element(const MexKernelArgs &a, const PixelRef &px, int k, ptrdiff_t *img_off)
{
    const int bhw = a.bh * a.bw;
    const int dc = k / bhw;
    const int rem = k - dc * bhw;
    const int dh = rem / a.bw;
    const int dw = rem - dh * a.bw;
    const int ci = px.ci0 + dc, hi = px.hi0 + dh, wi = px.wi0 + dw;
    const bool ok = ci >= 0 && ci < a.C && hi >= 0 && hi < a.H && wi >= 0 && wi < a.W;
    const ptrdiff_t o = ((ptrdiff_t)ci * a.H + hi) * a.W + wi;
    *img_off = ok ? o : -1;
    // (the load on an address that is always valid, the choice afterwards: loads inside conditions are waited for one
    // by one)
    const float v = a.in[(size_t)px.b * a.C * a.H * a.W + (ok ? o : 0)];
    return ok ? v : a.oob;
}

__device__ __forceinline__ float mex_term(float x_plus_off, float out, float g, float c1, float c0, bool finite)
{
    if (finite)
        return g * __builtin_amdgcn_exp2f(__builtin_fmaf(x_plus_off - out, c1, c0));
    return x_plus_off == out ? g : 0.0f;
}

constexpr int GX_KT = 8;   // patch elements per lane (input gradient)

// One wave: the 64 pixel slots of (region r, chunk) x GX_KT patch elements from k0, term by term.
__device__ __forceinline__ void mex_grad_input_wave(const MexGradArgs &ga, int r, int chunk, int k0, int lane,
                                                    int m_begin, int m_end, float *dx)
{
    const MexKernelArgs &a = ga.k;
    const PixelRef px = locate(a, r, chunk * 64 + lane);
    const bool valid = px.out_off >= 0;

    float xk[GX_KT], acc[GX_KT];
    ptrdiff_t io[GX_KT];
#pragma unroll
    for (int j = 0; j < GX_KT; ++j) {
        acc[j] = 0.0f;
        io[j] = -1;
        xk[j] = 0.0f;
        if (k0 + j < a.K)
            xk[j] = patch_element(a, px, k0 + j, &io[j]);
    }
    const size_t plane = (size_t)a.Co * a.Ho * a.Wo;
    const size_t gplane = pooled_g_plane(ga, plane);
    const float *gp = ga.g + (size_t)px.b * a.M * gplane + (valid ? pooled_g_offset(ga, px.out_off) : 0);
    const float *op = ga.out + (size_t)px.b * a.M * plane + (valid ? px.out_off : 0);
    const float SIMNETS_CONST_AS *off = (const float SIMNETS_CONST_AS *)(ga.off) + (size_t)r * a.M * a.K + k0;
    const bool finite = a.finite_eps != 0;
    // four instances at a time: their gradient and output values requested together (the additions keep their order)
    for (int m4 = m_begin; m4 < m_end; m4 += 4) {
        float gv[4], ov[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int mc = min(m4 + u, m_end - 1);
            gv[u] = gp[(size_t)mc * gplane];
            ov[u] = op[(size_t)mc * plane];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int m = m4 + u;
            if (m < m_end) {
                const float g = valid ? gv[u] : 0.0f;
#pragma unroll
                for (int j = 0; j < GX_KT; ++j) {
                    const float of = (k0 + j < a.K) ? off[(size_t)m * a.K + j] : 0.0f;
                    acc[j] += mex_term(xk[j] + of, ov[u], g, a.c1, a.c0, finite);
                }
            }
        }
    }
    if (!valid)
        return;
    float *dimg = dx + (size_t)px.b * a.C * a.H * a.W;
    float *dcol = ga.col + ((size_t)px.b * plane + px.out_off) * a.K + k0;
#pragma unroll
    for (int j = 0; j < GX_KT; ++j) {
        if (io[j] < 0)
            continue;
        if (ga.overlap)
            dcol[j] = acc[j];
        else
            dimg[io[j]] = acc[j];
    }
}

// grid.x: (region, pixel chunk of 64 slots); grid.y: tile of 4*GX_KT patch elements (one GX_KT per wave)
__global__ __launch_bounds__(256) void mex_grad_input_kernel(const MexGradArgs ga)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = blockIdx.x / ga.cpr;
    const int chunk = blockIdx.x - r * ga.cpr;
    const int k0 = (blockIdx.y * 4 + wave) * GX_KT;
    if (k0 < ga.k.K)
        mex_grad_input_wave(ga, r, chunk, k0, lane, 0, ga.k.M, ga.dx);
}

// Finite epsilon, product form on the fp32 matrix cores.  In the scaled domain (xs = c1 x, os = c1 off, outs = c1 out,
// c1 = eps log2 e) a term is g 2^(xs_k + os_mk - outs_m + c0), and outs_m - c0 = log2 sum_k 2^(xs_k + os_mk) bounds every
// xs_k + os_mk from above.  With lo_m = min_k os_mk and a = min_m (outs_m - c0 - lo_m) >= every xs_k of the pixel:
//   term = 2^(xs_k - a) * 2^(os_mk - mo_m) * [ g_m 2^(a + mo_m - outs_m + c0) ],
// all three factors at most 2^(range of the instance's offsets), and for the terms that matter (near 1) at least
// 2^-range: d patch_k = 2^(xs_k - a) * sum_m W_m EO_mk is a GEMM over the instances (v_mfma_f32_16x16x4_f32 tiles:
// 16 patch elements x 16 pixels x 4 instances) of the pixel factors W (computed from g and out, which the kernel
// reads anyway: no pass over the patches is needed for the bound) with the packed offset exponentials EO of the
// forward pass.  Used when every instance of the region has an offsets range of at most kGradProductRange; otherwise the
// workgroup falls back to the term-by-term waves.
// grid.x: (region, pixel chunk of 64 slots); grid.y: tile of GM_KT patch elements (16 per wave)
constexpr int GM_TM = kGradPackTm;   // (32) instances per packed group = contraction chunk
// Widest offsets range (an exponent of two) the gradients' product form takes on the loose bound a (below).  Its factors
// 2^(xs - a), 2^(os - mo) and W then carry exponents of up to the range, each rounded once: an error of ulp(range) in an
// exponent is a relative error of about 4e-8 * range in the factor - two to four times the error of the reference's own
// fp32 arithmetic on the same data.  Measured against the fp64 oracle the gradients stay within the 1e-4 bar up to
// ranges of about 50 (at most 8e-5 at 48, 1.15e-4 at 64, 1.2e-4 at 77 on the tests' data; the reference's fp32 arithmetic:
// 1.5 ... 3e-5); the forward pass's 90 is a bound against overflow, not this one.  Beyond it the gathering kernels take
// a region term by term (about 12 times slower); the row-wise kernels switch to a tight bound (kGradRowsRange).
constexpr float kGradProductRange = 48.0f;
// Row-wise kernels: widest patch range of a pixel (exponents of two) for which a region with large offsets ranges
// keeps the product form on the pixel's own maximum as the bound (the factors' exponents stay within this range)
constexpr float kGradPixelRange = 64.0f;
// ... and the widest offsets range such a region may have.  With the tight bound the factors' errors follow the size of
// the offsets themselves, as the reference's own do, at 1.5 to 4 times its error; what an element of the gradient sees
// of it depends on how far its terms cancel: 4e-5 ... 7e-5 at 77 and 1.5e-4 at 88 on the tests' seeded layers, but
// 1.1e-4 at a range of 55 on another (a sum of 4.8 in absolute terms that cancels to 0.08; error 2e-6 of the terms).  The
// same limit as the gathering kernels' keeps such elements rare; beyond it a region goes term by term.
constexpr float kGradRowsRange = 48.0f;
constexpr float kLooseBoundRange = 24.0f;  // offsets ranges (exponents of two) up to which a few instances give the bound
constexpr int GM_KT = 64;
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Pixel factors and patch exponentials of the product form, once per pixel: for the 64 pixel slots of
// (region, chunk) the bound a, W_m = g_m 2^(a + mo_m - outs_m + c0) for every instance and 2^(xs_k - a) for every
// patch element, written as rows [slot][Mp] and [slot][Kp] (through LDS, so that the stores run along the rows);
// a workgroup forms one block of 32 instances or 32 patch elements (grid.y), each from the same bound.
// Regions with an offsets range beyond kGradProductRange are left alone: the matrix kernels fall back to the
// term-by-term waves there and never look at the buffers.
__global__ __launch_bounds__(256) void mex_grad_factors_kernel(const MexGradArgs ga)
{
    const MexKernelArgs &a = ga.k;
    __shared__ float tile[32 * 65];   // [instance or patch element][pixel], padded rows
    __shared__ float pmn[4 * 64];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = blockIdx.x / ga.cpr;
    const int chunk = blockIdx.x - r * ga.cpr;
    const int n_mg = a.n_mgroups;
    const float *omax_r = a.omax + (size_t)r * n_mg * GM_TM, *orng_r = a.orng + (size_t)r * n_mg * GM_TM;
    int wide = 0, big = 0;
    for (int m = tid; m < a.M; m += 256) {
        wide |= !(orng_r[m] <= kGradProductRange);
        big |= !(orng_r[m] <= kLooseBoundRange);
    }
    const int roomy = __syncthreads_or(big);
    if (__syncthreads_or(wide))
        return;
    const PixelRef px = locate(a, r, chunk * 64 + lane);
    const bool valid = px.out_off >= 0;
    const size_t plane = (size_t)a.Co * a.Ho * a.Wo, gplane = pooled_g_plane(ga, plane);
    const float *gp = ga.g + (size_t)px.b * a.M * gplane + (valid ? pooled_g_offset(ga, px.out_off) : 0);
    const float *op = ga.out + (size_t)px.b * a.M * plane + (valid ? px.out_off : 0);
    const int m_scan = roomy ? a.M : min(a.M, 4);   // see mex_grad_input_mfma_kernel
    float amin = INFINITY;
#pragma unroll 4
    for (int m = wave; m < m_scan; m += 4)   // (unrolled: four loads in flight instead of one)
        amin = fminf(amin, __builtin_fmaf(op[(size_t)m * plane], a.c1, -(a.c0 + (omax_r[m] - orng_r[m]))));
    pmn[wave * 64 + lane] = amin;
    __syncthreads();
    const float a_p = valid ? fminf(fminf(pmn[lane], pmn[64 + lane]), fminf(pmn[128 + lane], pmn[192 + lane])) : 0.0f;
    // (below, all loads of a block go out first, those past the last instance or patch element on a clamped
    // address: a load inside the condition would be waited for before the next one is issued)
    // rows of this chunk; thread (column c, pixels pr, pr + 8, ...) writes the tile out
    const size_t row0 = (size_t)r * ga.slots_pad + (size_t)chunk * 64;
    const int c = tid & 31, pr = tid >> 5;
    // grid.y: one block of 32 columns per workgroup - the instance groups first, then the patch-element blocks
    if ((int)blockIdx.y < n_mg) {
        const int mg = blockIdx.y;
        float ovv[GM_TM / 4], gvv[GM_TM / 4], omv[GM_TM / 4];
#pragma unroll
        for (int i = 0; i < GM_TM / 4; ++i) {
            const int mc = min(mg * GM_TM + wave + 4 * i, a.M - 1);
            ovv[i] = op[(size_t)mc * plane];
            gvv[i] = gp[(size_t)mc * gplane];
            omv[i] = omax_r[mc];
        }
#pragma unroll
        for (int i = 0; i < GM_TM / 4; ++i) {
            const int mm = wave + 4 * i, m = mg * GM_TM + mm;
            float w = 0.0f;
            if (valid && m < a.M) {
                const float e = __builtin_fmaf(-ovv[i], a.c1, a_p) + (omv[i] + a.c0);
                w = gvv[i] * __builtin_amdgcn_exp2f(e);
            }
            tile[mm * 65 + lane] = w;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 8; ++j)
            ga.wbuf[(row0 + pr + 8 * j) * ga.Mp + mg * GM_TM + c] = tile[c * 65 + pr + 8 * j];
    } else {
        const int kb = ((int)blockIdx.y - n_mg) * 32;
        int4 ke[8];  // wave-uniform: {offset inside an image, dc, dh, dw}
#pragma unroll
        for (int i = 0; i < 8; ++i)
            ke[i] = a.ktab[min(kb + wave + 4 * i, a.K - 1)];
        float xg[8];
        unsigned inside = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int ci = px.ci0 + ke[i].y, hi = px.hi0 + ke[i].z, wi = px.wi0 + ke[i].w;
            const bool ok = ci >= 0 && ci < a.C && hi >= 0 && hi < a.H && wi >= 0 && wi < a.W;
            inside |= ok ? 1u << i : 0u;
            const float *src = ok ? px.base + ke[i].x : a.in;
            xg[i] = *src;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int kk = wave + 4 * i, k = kb + kk;
            float e = 0.0f;
            if (valid && k < a.K) {
                const float x = (inside >> i) & 1u ? xg[i] : a.oob;
                e = __builtin_amdgcn_exp2f(__builtin_fmaf(x, a.c1, -a_p));
            }
            tile[kk * 65 + lane] = e;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 8; ++j)
            ga.exbuf[(row0 + pr + 8 * j) * ga.Kp + kb + c] = tile[c * 65 + pr + 8 * j];
    }
}

__global__ __launch_bounds__(256) void mex_grad_input_mfma_kernel(const MexGradArgs ga)
{
    const MexKernelArgs &a = ga.k;
    __shared__ float eo[GM_KT * (GM_TM + 1)];   // [k][instance], padded rows
    __shared__ float wt[GM_TM * 65];            // [instance][pixel], padded rows
    __shared__ float pmn[4 * 64], ap[64];
    __shared__ int pb[64], pc0[64], ph0[64], pw0[64];   // pixel table: image (-1: empty slot), patch origin
    __shared__ int pout[64];                            // ... and the pixel's offset within the image's output
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = blockIdx.x / ga.cpr;
    const int chunk = blockIdx.x - r * ga.cpr;
    const int k0 = blockIdx.y * GM_KT;
    const int n_mg = a.n_mgroups;
    // this workgroup's share of the instances (all of them unless the launch splits them over gridDim.z) and where
    // its gradients go
    const int mg_begin = blockIdx.z * ga.mg_per_split, mg_end = min(n_mg, mg_begin + ga.mg_per_split);
    float *dxo = ga.msplit > 1 ? ga.dx_splits + (size_t)blockIdx.z * a.B * a.C * a.H * a.W : ga.dx;
    const float *omax_r = a.omax + (size_t)r * n_mg * GM_TM, *orng_r = a.orng + (size_t)r * n_mg * GM_TM;
    // (everything the product form reads first is requested before the barriers that decide on it: the pixel, its
    // table entries, the first output value of the bound, the patch element records of this lane's gradients)
    const int lr = lane & 15, lq = lane >> 4;
    int4 kel[4];
#pragma unroll
    for (int v = 0; v < 4; ++v)
        kel[v] = a.ktab[min(k0 + wave * 16 + 4 * lq + v, a.K - 1)];
    const PixelRef px = locate(a, r, chunk * 64 + lane);
    const bool valid = px.out_off >= 0;
    if (wave == 0) {
        pb[lane] = valid ? px.b : -1;
        pc0[lane] = px.ci0; ph0[lane] = px.hi0; pw0[lane] = px.wi0;
        pout[lane] = px.out_off;
    }
    const size_t plane = (size_t)a.Co * a.Ho * a.Wo, gplane = pooled_g_plane(ga, plane);
    const float *gp = ga.g + (size_t)px.b * a.M * gplane + (valid ? pooled_g_offset(ga, px.out_off) : 0);
    const float *op = ga.out + (size_t)px.b * a.M * plane + (valid ? px.out_off : 0);
    const float o_first = op[(size_t)min(wave, a.M - 1) * plane];
    const float lo_first = omax_r[min(wave, a.M - 1)] - orng_r[min(wave, a.M - 1)];
    int roomy;  // some instance's offsets range is large enough for the choice of the bound to matter (below)
    {
        int wide = 0, big = 0;
        for (int m = tid; m < a.M; m += 256) {
            wide |= !(orng_r[m] <= kGradProductRange);
            big |= !(orng_r[m] <= kLooseBoundRange);
        }
        roomy = __syncthreads_or(big);
        if (__syncthreads_or(wide)) {
#pragma unroll
            for (int h = 0; h < GM_KT / (4 * GX_KT); ++h) {
                const int kk0 = k0 + (wave * (GM_KT / (4 * GX_KT)) + h) * GX_KT;
                if (kk0 < a.K)
                    mex_grad_input_wave(ga, r, chunk, kk0, lane, min(a.M, mg_begin * GM_TM), min(a.M, mg_end * GM_TM),
                                        dxo);
            }
            return;
        }
    }
    const bool buffered = ga.wbuf != nullptr;   // W and 2^(xs - a) come from mex_grad_factors_kernel
    const size_t row0 = (size_t)r * ga.slots_pad + (size_t)chunk * 64;
    // the pixel's bound a = min_m (outs_m - c0 - lo_m).  Every single term of the minimum is a valid bound
    // (>= every xs_k); with the minimum over all instances the exponent of W_m stays below the instance's own
    // offsets range, with the minimum over a few it stays below that range + the range of those few + log2 K.
    // While no range exceeds kLooseBoundRange that is far from overflow, and the first four instances (one
    // strided load per thread instead of M / 4) do.
    const int m_scan = buffered ? 0 : (roomy ? a.M : min(a.M, 4));
    float amin = INFINITY;
    for (int m = wave; m < m_scan; m += 4)
        amin = fminf(amin, m == wave ? __builtin_fmaf(o_first, a.c1, -(a.c0 + lo_first))
                                     : __builtin_fmaf(op[(size_t)m * plane], a.c1, -(a.c0 + (omax_r[m] - orng_r[m]))));
    pmn[wave * 64 + lane] = amin;
    __syncthreads();
    if (wave == 0)
        ap[lane] = valid ? fminf(fminf(pmn[lane], pmn[64 + lane]), fminf(pmn[128 + lane], pmn[192 + lane])) : 0.0f;
    __syncthreads();
    const float a_p = ap[lane];

    // where this lane's 16 gradients go (the pixel tables are in place behind the barriers above) and the input
    // values their factors 2^(xs_k - a) are made of: requested here, used after the matrix loop (a load in front of
    // each store made the lane wait for 16 memory round trips in turn, 45 % of the kernel on a 64 x 32 x 16 x 16 -> 64
    // layer)
    const size_t chw = (size_t)a.C * a.H * a.W;
    size_t at[4][4];
    float xin[4][4];
    bool ok[4][4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int k = k0 + wave * 16 + 4 * lq + v;
        const int dc = kel[v].y, dh = kel[v].z, dw = kel[v].w;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int p = t * 16 + lr;
            const int b = pb[p];
            const int ci = pc0[p] + dc, hi = ph0[p] + dh, wi = pw0[p] + dw;
            ok[v][t] = k < a.K && b >= 0 && ci >= 0 && ci < a.C && hi >= 0 && hi < a.H && wi >= 0 && wi < a.W;
            at[v][t] = ok[v][t] ? (size_t)b * chw + ((size_t)ci * a.H + hi) * a.W + wi : 0;
            if (buffered)
                xin[v][t] = ga.exbuf[ok[v][t] ? (row0 + p) * ga.Kp + k : 0];
            else
                xin[v][t] = a.in[at[v][t]];
        }
    }

    floatx4 acc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
        acc[t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    // operands of an instance group: the offsets tile (two float4 per thread) and, unless the pixel factors come from
    // the buffers, this thread's eight output and gradient values - requested a group ahead
    constexpr int EO4 = GM_KT * (GM_TM / 4) / 256;
    float4 eo_n[EO4];
    float ov_n[GM_TM / 4], gv_n[GM_TM / 4], om_n[GM_TM / 4];
    auto request = [&](int mg) {
        const float4 *src = reinterpret_cast<const float4 *>(a.offe + (((size_t)r * n_mg + mg) * a.K + k0) * GM_TM);
#pragma unroll
        for (int j = 0; j < EO4; ++j) {
            const int i = tid + j * 256;
            eo_n[j] = k0 + i / (GM_TM / 4) < a.K ? src[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
        if (!buffered) {
#pragma unroll
            for (int i = 0; i < GM_TM / 4; ++i) {
                const int m = min(mg * GM_TM + wave + 4 * i, a.M - 1);
                ov_n[i] = op[(size_t)m * plane];
                gv_n[i] = gp[(size_t)m * gplane];
                om_n[i] = omax_r[m];
            }
        }
    };
    if (mg_begin < mg_end)
        request(mg_begin);
    for (int mg = mg_begin; mg < mg_end; ++mg) {
        __syncthreads();  // the previous chunk's matrix instructions are done with eo / wt
#pragma unroll
        for (int j = 0; j < EO4; ++j) {
            const int i = tid + j * 256;
            const int row = i / (GM_TM / 4), c4 = i % (GM_TM / 4);
            const float4 v = eo_n[j];
            float *d = eo + row * (GM_TM + 1) + 4 * c4;
            d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
        }
        if (buffered) {
            // rows of 32 instances: thread (instance c, pixels pr, pr + 8, ...)
            const int c = tid & 31, pr = tid >> 5;
#pragma unroll
            for (int j = 0; j < 8; ++j)
                wt[c * 65 + pr + 8 * j] = ga.wbuf[(row0 + pr + 8 * j) * ga.Mp + mg * GM_TM + c];
        } else {
#pragma unroll
            for (int i = 0; i < GM_TM / 4; ++i) {
                const int mm = wave + 4 * i, m = mg * GM_TM + mm;
                float w = 0.0f;
                if (valid && m < a.M) {
                    // (a - outs) first: a small, once-rounded difference; the instance constant is added to that
                    const float e = __builtin_fmaf(-ov_n[i], a.c1, a_p) + (om_n[i] + a.c0);
                    w = gv_n[i] * __builtin_amdgcn_exp2f(e);
                }
                wt[mm * 65 + lane] = w;
            }
        }
        if (mg + 1 < mg_end)
            request(mg + 1);   // in flight during the matrix steps
        __syncthreads();
#pragma unroll
        for (int ms = 0; ms < GM_TM; ms += 4) {
            const float av = eo[(wave * 16 + lr) * (GM_TM + 1) + ms + lq];
#pragma unroll
            for (int t = 0; t < 4; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, wt[(ms + lq) * 65 + t * 16 + lr], acc[t], 0, 0, 0);
        }
    }
    // ---- d patch_k = 2^(xs_k - a) * acc, scattered to the input element the patch element is ----
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int k = k0 + wave * 16 + 4 * lq + v;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (!ok[v][t])
                continue;
            const int p = t * 16 + lr;
            const float val = acc[t][v] * (buffered ? xin[v][t]
                                                    : __builtin_amdgcn_exp2f(__builtin_fmaf(xin[v][t], a.c1, -ap[p])));
            if (ga.overlap)
                ga.col[((size_t)pb[p] * plane + pout[p]) * a.K + k] = val;
            else
                dxo[at[v][t]] = val;
        }
    }
}

// Instances split over several workgroups: input gradient = sum of their partial gradients, in split order.
__global__ __launch_bounds__(256) void mex_sum_splits_kernel(const float *__restrict__ parts, long long n, int splits,
                                                            float *__restrict__ dx)
{
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
        float s = parts[i];
        for (int z = 1; z < splits; ++z)
            s += parts[(size_t)z * n + i];
        dx[i] = s;
    }
}

// ... four elements per thread with all the splits' loads (at most 8) in flight together: n a multiple of 4, 16-byte
// aligned pointers.  The same additions in the same order.
__global__ __launch_bounds__(256) void mex_sum_splits4_kernel(const float4 *__restrict__ parts, long long n4, int splits,
                                                             float4 *__restrict__ dx)
{
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
    if (i >= n4)
        return;
    float4 v[8];
#pragma unroll
    for (int z = 0; z < 8; ++z)
        v[z] = parts[(size_t)min(z, splits - 1) * n4 + i];
    float4 s = v[0];
#pragma unroll
    for (int z = 1; z < 8; ++z)
        if (z < splits) {
            s.x += v[z].x; s.y += v[z].y; s.z += v[z].z; s.w += v[z].w;
        }
    dx[i] = s;
}

void launch_sum_splits(const float *parts, long long n, int splits, float *dx, hipStream_t s)
{
    if (splits <= 8 && n % 4 == 0 && reinterpret_cast<uintptr_t>(parts) % 16 == 0 &&
        reinterpret_cast<uintptr_t>(dx) % 16 == 0 && (n / 4 + 255) / 256 <= 0x7fffffffLL)
        hipLaunchKernelGGL(mex_sum_splits4_kernel, dim3((unsigned)((n / 4 + 255) / 256)), dim3(256), 0, s,
                           reinterpret_cast<const float4 *>(parts), n / 4, splits, reinterpret_cast<float4 *>(dx));
    else
        hipLaunchKernelGGL(mex_sum_splits_kernel, dim3((unsigned)std::min<long long>((n + 255) / 256, 65535)), dim3(256),
                           0, s, parts, n, splits, dx);
}

// Overlapping patches: input gradient = sum, over the patches that cover the element, of the patch-element
// gradients in `col` (the reference's col2im_3d, src/utils/im2col.cpp:297-328), patches in ascending (c, h, w)
// order.  One thread per input element; elements no patch covers get 0.
__global__ __launch_bounds__(256) void mex_col2im_kernel(const MexKernelArgs a, const float *__restrict__ col,
                                                         float *__restrict__ dx, long long n)
{
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n)
        return;
    const int w = (int)(idx % a.W);
    long long q = idx / a.W;
    const int h = (int)(q % a.H); q /= a.H;
    const int c = (int)(q % a.C);
    const long long b = q / a.C;
    // patches o along an axis that cover coordinate x: 0 <= x + pad - o * stride < block
    auto first = [](int x, int pad, int block, int stride) {
        const int lo = x + pad - block + 1;
        return lo <= 0 ? 0 : (lo + stride - 1) / stride;
    };
    const int co_lo = first(c, a.pc, a.bc, a.sc), co_hi = min(a.Co - 1, (c + a.pc) / a.sc);
    const int ho_lo = first(h, a.ph, a.bh, a.sh), ho_hi = min(a.Ho - 1, (h + a.ph) / a.sh);
    const int wo_lo = first(w, a.pw, a.bw, a.sw), wo_hi = min(a.Wo - 1, (w + a.pw) / a.sw);
    const float *cb = col + (size_t)b * a.Co * a.Ho * a.Wo * a.K;
    float acc = 0.0f;
    for (int co = co_lo; co <= co_hi; ++co) {
        const int dc = c + a.pc - co * a.sc;
        for (int ho = ho_lo; ho <= ho_hi; ++ho) {
            const int dh = h + a.ph - ho * a.sh;
            for (int wo = wo_lo; wo <= wo_hi; ++wo) {
                const int dw = w + a.pw - wo * a.sw;
                acc += cb[(((size_t)co * a.Ho + ho) * a.Wo + wo) * a.K + (dc * a.bh + dh) * a.bw + dw];
            }
        }
    }
    dx[idx] = acc;
}

constexpr int GO_MT = 4, GO_KT = 8;  // instances x patch elements per lane (offsets gradient)

// One wave: GO_MT instances from m0 x GO_KT patch elements from k0 over the 64*pxl pixel slots of (region r,
// chunk), term by term; writes its partial sums.
__device__ __forceinline__ void mex_grad_offsets_wave(const MexGradArgs &ga, int r, int chunk, int m0, int k0, int lane)
{
    const MexKernelArgs &a = ga.k;

    float acc[GO_MT][GO_KT];
#pragma unroll
    for (int i = 0; i < GO_MT; ++i)
#pragma unroll
        for (int j = 0; j < GO_KT; ++j)
            acc[i][j] = 0.0f;
    // the offsets of this wave's tile are the same for every pixel
    float of[GO_MT][GO_KT];
    const float SIMNETS_CONST_AS *off = (const float SIMNETS_CONST_AS *)(ga.off) + (size_t)r * a.M * a.K;
#pragma unroll
    for (int i = 0; i < GO_MT; ++i)
#pragma unroll
        for (int j = 0; j < GO_KT; ++j)
            of[i][j] = (m0 + i < a.M && k0 + j < a.K) ? to_vgpr(off[(size_t)(m0 + i) * a.K + k0 + j]) : 0.0f;

    const size_t plane = (size_t)a.Co * a.Ho * a.Wo;
    const bool finite = a.finite_eps != 0;
    for (int s = 0; s < ga.pxl; ++s) {
        const PixelRef px = locate(a, r, (chunk * ga.pxl + s) * 64 + lane);
        const bool valid = px.out_off >= 0;
        float xk[GO_KT];
#pragma unroll
        for (int j = 0; j < GO_KT; ++j) {
            ptrdiff_t unused;
            xk[j] = (k0 + j < a.K) ? patch_element(a, px, k0 + j, &unused) : 0.0f;
        }
        const size_t gplane = pooled_g_plane(ga, plane);
        const float *gp = ga.g + (size_t)px.b * a.M * gplane + (valid ? pooled_g_offset(ga, px.out_off) : 0);
        const float *op = ga.out + (size_t)px.b * a.M * plane + (valid ? px.out_off : 0);
        float gv[GO_MT], ov[GO_MT];
#pragma unroll
        for (int i = 0; i < GO_MT; ++i) {   // (all requests first, on clamped rows)
            const int mc = min(m0 + i, a.M - 1);
            gv[i] = gp[(size_t)mc * gplane];
            ov[i] = op[(size_t)mc * plane];
        }
#pragma unroll
        for (int i = 0; i < GO_MT; ++i) {
            const bool mok = valid && m0 + i < a.M;
            const float g = mok ? gv[i] : 0.0f;
            const float o = mok ? ov[i] : 0.0f;
#pragma unroll
            for (int j = 0; j < GO_KT; ++j) {
                const float e = mex_term(xk[j] + of[i][j], o, g, a.c1, a.c0, finite);
                acc[i][j] += mok ? e : 0.0f;
            }
        }
    }
    // sum over the 64 lanes; lane 0 holds the result
#pragma unroll
    for (int i = 0; i < GO_MT; ++i)
#pragma unroll
        for (int j = 0; j < GO_KT; ++j) {
            float v = acc[i][j];
            for (int d = 32; d > 0; d >>= 1)
                v += __shfl_xor(v, d, 64);
            acc[i][j] = v;
        }
    if (lane == 0) {
        float *dst = ga.partial + ((size_t)chunk * a.R + r) * a.M * a.K;
#pragma unroll
        for (int i = 0; i < GO_MT; ++i)
#pragma unroll
            for (int j = 0; j < GO_KT; ++j)
                if (m0 + i < a.M && k0 + j < a.K)
                    dst[(size_t)(m0 + i) * a.K + k0 + j] = acc[i][j];
    }
}

// grid.x: (region, pixel chunk of 64*pxl slots); grid.y: tile of 4*GO_MT instances (one GO_MT per wave);
// grid.z: tile of GO_KT patch elements
__global__ __launch_bounds__(256) void mex_grad_offsets_kernel(const MexGradArgs ga)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = blockIdx.x / ga.cpr;
    const int chunk = blockIdx.x - r * ga.cpr;
    const int m0 = (blockIdx.y * 4 + wave) * GO_MT;
    if (m0 < ga.k.M)
        mex_grad_offsets_wave(ga, r, chunk, m0, blockIdx.z * GO_KT, lane);
}

// Finite epsilon, product form (see mex_grad_input_mfma_kernel): d off_mk = 2^(os_mk - mo_m) * sum_px W_px,m 2^(xs_px,k - a_px)
// is a GEMM over the pixels.  The bound a of a pixel only has to hold for the instances of the workgroup's tile, so
// it is the minimum over those.  A workgroup owns 64 instances x 64 patch elements (wave: 16 x 64, four 16 x 16
// tiles) and walks its pxl groups of 64 pixel slots: pixel factors W [pixel][instance] and patch exponentials
// [pixel][k] go to LDS, 16 matrix steps of 4 pixels each.
// grid.x: (region, pixel chunk of 64*pxl slots); grid.y: tile of 64 instances; grid.z: tile of 64 patch elements
constexpr int GOM_MT = 64, GOM_KT = 64;

__global__ __launch_bounds__(256) void mex_grad_offsets_mfma_kernel(const MexGradArgs ga)
{
    const MexKernelArgs &a = ga.k;
    __shared__ float wt[64 * 65];   // [pixel][instance], padded rows
    __shared__ float ex[64 * 65];   // [pixel][k], padded rows
    __shared__ float pmn[4 * 64];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = blockIdx.x / ga.cpr;
    const int chunk = blockIdx.x - r * ga.cpr;
    const int m0 = blockIdx.y * GOM_MT, k0 = blockIdx.z * GOM_KT;
    const int n_mg = a.n_mgroups;
    const float *omax_r = a.omax + (size_t)r * n_mg * GM_TM, *orng_r = a.orng + (size_t)r * n_mg * GM_TM;
    {
        int wide = 0;
        for (int m = tid; m < a.M; m += 256)
            wide |= !(orng_r[m] <= kGradProductRange);
        if (__syncthreads_or(wide)) {
            // term by term: this workgroup's tile as GO_MT x GO_KT wave tiles
            for (int i = wave; i < (GOM_MT / GO_MT) * (GOM_KT / GO_KT); i += 4) {
                const int mm0 = m0 + (i / (GOM_KT / GO_KT)) * GO_MT, kk0 = k0 + (i % (GOM_KT / GO_KT)) * GO_KT;
                if (mm0 < a.M && kk0 < a.K)
                    mex_grad_offsets_wave(ga, r, chunk, mm0, kk0, lane);
            }
            return;
        }
    }
    const size_t plane = (size_t)a.Co * a.Ho * a.Wo, gplane = pooled_g_plane(ga, plane);
    const int lr = lane & 15, lq = lane >> 4;
    floatx4 acc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t)
        acc[t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    // this thread's instances when staging (16 of the tile, the same for the whole wave) and their constants
    const int ms0 = m0 + wave * 16;
    // the records of the wave's 16 patch elements: one vector load (lane i holds element i), read back lane by lane
    // where they are used - as 16 wave-uniform loads in front of the 16 gathers each was waited for on its own
    const int4 kl = a.ktab[min(k0 + wave * 16 + (lane & 15), a.K - 1)];
    const bool buffered = ga.wbuf != nullptr;   // W and 2^(xs - a) come from mex_grad_factors_kernel
    // global loads of a group of 64 pixel slots: this thread's pixel, its 16 instances' output and gradient values
    // and 16 of the tile's patch elements; the loads of group s + 1 are issued before group s is processed
    struct Group {
        bool valid;
        float ov[16], gv[16], xr[16];
    };
    auto load_group = [&](int s, Group &q) {
        const PixelRef px = locate(a, r, (chunk * ga.pxl + s) * 64 + lane);
        q.valid = px.out_off >= 0;
        const float *gp = ga.g + (size_t)px.b * a.M * gplane + (q.valid ? pooled_g_offset(ga, px.out_off) : 0);
        const float *op = ga.out + (size_t)px.b * a.M * plane + (q.valid ? px.out_off : 0);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int m = ms0 + i;
            q.ov[i] = 0.0f;
            q.gv[i] = 0.0f;
            if (m < a.M) {
                q.ov[i] = op[(size_t)m * plane];
                q.gv[i] = q.valid ? gp[(size_t)m * gplane] : 0.0f;
            }
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int k = k0 + wave * 16 + i;
            q.xr[i] = 0.0f;
            if (q.valid && k < a.K) {
                // {offset inside an image, dc, dh, dw} of element i
                const int kx = __builtin_amdgcn_readlane(kl.x, i), ky = __builtin_amdgcn_readlane(kl.y, i);
                const int kz = __builtin_amdgcn_readlane(kl.z, i), kw = __builtin_amdgcn_readlane(kl.w, i);
                const int ci = px.ci0 + ky, hi = px.hi0 + kz, wi = px.wi0 + kw;
                const bool ok = ci >= 0 && ci < a.C && hi >= 0 && hi < a.H && wi >= 0 && wi < a.W;
                q.xr[i] = ok ? px.base[kx] : a.oob;
            }
        }
    };
    Group cur;
    for (int s = 0; s < ga.pxl; ++s) {
        if (buffered) {
            // rows of the group's 64 pixel slots: thread (column cc of the tile, pixels pq, pq + 4, ...)
            const int grp = chunk * ga.pxl + s;
            if (grp * 64 >= ga.slots_pad)
                break;  // no slots left in the region (uniform)
            const size_t row0 = (size_t)r * ga.slots_pad + (size_t)grp * 64;
            const int cc = tid & 63, pq = tid >> 6;
            __syncthreads();  // the previous group's matrix instructions are done with wt / ex
            // (sixteen loads at a time, columns past the buffers' rows on a clamped address: inside the condition
            // each would be waited for in front of its LDS write)
            const int mcol_c = min(m0 + cc, ga.Mp - 1), kcol_c = min(k0 + cc, ga.Kp - 1);
#pragma unroll
            for (int j0 = 0; j0 < 16; j0 += 8) {
                float wv[8], ev[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int pp = pq + 4 * (j0 + j);
                    wv[j] = ga.wbuf[(row0 + pp) * ga.Mp + mcol_c];
                    ev[j] = ga.exbuf[(row0 + pp) * ga.Kp + kcol_c];
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int pp = pq + 4 * (j0 + j);
                    wt[pp * 65 + cc] = m0 + cc < ga.Mp ? wv[j] : 0.0f;
                    ex[pp * 65 + cc] = k0 + cc < ga.Kp ? ev[j] : 0.0f;
                }
            }
            __syncthreads();
#pragma unroll 4
            for (int ps = 0; ps < 64; ps += 4) {
                const float av = wt[(ps + lq) * 65 + wave * 16 + lr];
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, ex[(ps + lq) * 65 + t * 16 + lr], acc[t], 0, 0, 0);
            }
            continue;
        }
        if (s == 0)
            load_group(0, cur);
        Group nxt;
        if (s + 1 < ga.pxl)
            load_group(s + 1, nxt);   // in flight while this group is processed
        float amin = INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int m = ms0 + i;
            if (m < a.M)
                amin = fminf(amin, __builtin_fmaf(cur.ov[i], a.c1, -(a.c0 + (omax_r[m] - orng_r[m]))));
        }
        __syncthreads();  // the previous group's matrix instructions are done with wt / ex / ap
        pmn[wave * 64 + lane] = amin;
        __syncthreads();
        const float a_p = cur.valid ? fminf(fminf(pmn[lane], pmn[64 + lane]), fminf(pmn[128 + lane], pmn[192 + lane])) : 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int m = ms0 + i;
            // (an empty slot holds the values of another region's pixel: its exponent can be anything, and zero times
            // an overflowed factor would put NaN into the sums)
            float w = 0.0f;
            if (cur.valid && m < a.M)
                w = cur.gv[i] * __builtin_amdgcn_exp2f(__builtin_fmaf(-cur.ov[i], a.c1, a_p) + (omax_r[m] + a.c0));
            wt[lane * 65 + wave * 16 + i] = w;
        }
        // patch exponentials: this thread's pixel, 16 of the tile's patch elements
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int kk = wave * 16 + i, k = k0 + kk;
            float e = 0.0f;
            if (cur.valid && k < a.K)
                e = __builtin_amdgcn_exp2f(__builtin_fmaf(cur.xr[i], a.c1, -a_p));
            ex[lane * 65 + kk] = e;
        }
        __syncthreads();
#pragma unroll 4
        for (int ps = 0; ps < 64; ps += 4) {
            const float av = wt[(ps + lq) * 65 + wave * 16 + lr];
#pragma unroll
            for (int t = 0; t < 4; ++t)
                acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, ex[(ps + lq) * 65 + t * 16 + lr], acc[t], 0, 0, 0);
        }
        if (s + 1 < ga.pxl)
            cur = nxt;
    }
    // ---- partial sums of this pixel chunk: acc * 2^(os_mk - mo_m) ----
    float *dst = ga.partial + ((size_t)chunk * a.R + r) * a.M * a.K;
    // (the 16 offset exponentials first, on clamped indices, then the products and stores)
    float eov[4][4];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int m = min(m0 + wave * 16 + 4 * lq + v, a.M - 1);
        const float *eo = a.offe + (((size_t)r * n_mg + m / GM_TM) * a.K) * GM_TM + m % GM_TM;
#pragma unroll
        for (int t = 0; t < 4; ++t)
            eov[v][t] = eo[(size_t)min(k0 + t * 16 + lr, a.K - 1) * GM_TM];
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int m = m0 + wave * 16 + 4 * lq + v;
        if (m >= a.M)
            continue;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int k = k0 + t * 16 + lr;
            if (k < a.K)
                dst[(size_t)m * a.K + k] = acc[t][v] * eov[v][t];
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Row-wise forms of the two matrix kernels for the layers of the reference's networks: 2 x 2 unshared offsets over
// whole-channel patches (blocks [C, 1, 1], stride 1, no padding) on maps whose height and width are powers of two.
// There the pixel slots of a region are every other pixel of every other row.  A wave that walks one region's slots
// touches 16 to 64 separate 32-byte sectors per load and uses half of each or less, the four regions write the
// input gradient into each other's sectors at different times, and the address units, not the arithmetic, set the
// time of the kernels above.  Here a workgroup takes the 64 slots of a chunk for ALL four regions - 256 pixels that
// are whole rows of one image or whole small images - so that every plane (an instance of `out` / `g`, a channel
// of the input or of its gradient) is read and written as one run of 1 KB, or runs of whole images, with 16-byte
// accesses.  The values pass through LDS tiles [plane][column] with column = region * 64 + slot, and wave r does
// the matrix steps of region r on its 64 columns.
struct RowsArgs {
    int lgW, Ws, RS;   // log2(width), windows per row, windows per image
    int lgHW, HW;      // pixels of an image
    int nx, ty, tz;    // workgroup numbering (rows_block): pixel groups, tiles along the two other grid dimensions
};

// Workgroups that read the same rows - the tiles (y, z) of one pixel group x - get consecutive turns on ONE
// accelerator die (linear workgroup id mod 8), so that the rows come from memory once and from that die's L2 for the
// other tiles.  The launch is one-dimensional with 8 * ceil(nx / 8) * ty * tz workgroups; false: no such group.
__device__ __forceinline__ bool rows_block(const RowsArgs &g, int *x, int *y, int *z)
{
    const int l = blockIdx.x, tiles = g.ty * g.tz;
    const int j = l >> 3, tile = j % tiles;
    *x = (j / tiles) * 8 + (l & 7);
    *y = tile % g.ty;
    *z = tile / g.ty;
    return *x < g.nx;
}

// A thread's four neighbouring pixels (a 16-byte piece of a row; width >= 4, so they share the row) of the chunk's
// 256: image, first pixel, tile columns.  Pixels 0 and 2 belong to region rbase, 1 and 3 to rbase + 1.  A chunk
// starts on an even row (or a whole image), so the columns and rbase depend on the quad alone, not on the chunk.
struct RowsQuad {
    int img, pix0, rbase;
    bool img_ok;
    int col[4];
};

__device__ __forceinline__ RowsQuad rows_quad(const MexKernelArgs &a, const RowsArgs &g, int chunk, int quad)
{
    RowsQuad q;
    const int gpix = chunk * 256 + 4 * quad;
    q.img = gpix >> g.lgHW;
    q.pix0 = gpix & (g.HW - 1);
    q.img_ok = q.img < a.B;
    const int h = q.pix0 >> g.lgW, w0 = q.pix0 & ((1 << g.lgW) - 1);
    q.rbase = (h & 1) * 2;
    const int sl = q.img * g.RS + (h >> 1) * g.Ws + (w0 >> 1) - chunk * 64;
    q.col[0] = (q.rbase << 6) + sl;
    q.col[1] = q.col[0] + 64;
    q.col[2] = q.col[0] + 1;
    q.col[3] = q.col[1] + 1;
    return q;
}

// The output gradients of a thread's pixel quad for plane (img, m) as they come from memory: 16 bytes of g, or - g
// pooled - the two window gradients the quad's row lies in (x, y; each belongs to two pixels).  rows_quad_g expands
// them where they are used: expanding here would wait for the load where it is issued.
__device__ __forceinline__ float4 rows_load_g(const MexGradArgs &ga, const RowsArgs &g, const RowsQuad &q, size_t img,
                                              int m)
{
    if (!ga.gpool)
        return *reinterpret_cast<const float4 *>(ga.g + (img * ga.k.M + m) * (size_t)g.HW + q.pix0);
    const int h = q.pix0 >> g.lgW, w0 = q.pix0 & ((1 << g.lgW) - 1);
    const float2 v = *reinterpret_cast<const float2 *>(ga.g + (img * ga.k.M + m) * (size_t)(g.HW >> 2) +
                                                       (size_t)(h >> 1) * g.Ws + (w0 >> 1));
    return make_float4(v.x, v.y, 0.0f, 0.0f);
}

__device__ __forceinline__ void rows_quad_g(const MexGradArgs &ga, const float4 &v, float (&gg)[4])
{
    gg[0] = v.x;
    gg[1] = ga.gpool ? v.x : v.y;
    gg[2] = ga.gpool ? v.y : v.z;
    gg[3] = ga.gpool ? v.y : v.w;
}

// per region: is some instance's offsets range beyond kGradRowsRange or not finite (flags[r]: term by term); flags[4]:
// does some range exceed kLooseBoundRange; flags[5]: does some range exceed kGradProductRange.  All threads of the
// workgroup call it; the flags (six) are in place behind its last barrier.
// (All loads go out before the first is looked at.)
__device__ __forceinline__ void rows_ranges(const MexKernelArgs &a, int tid, int *flags)
{
    if (tid < 6)
        flags[tid] = 0;
    const int per = a.n_mgroups * GM_TM;
    int big = 0, mid = 0, wide[4] = {0, 0, 0, 0};
    for (int mb = 0; mb < a.M; mb += 1024) {
        float v[4][4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                v[u][r] = a.orng[r * per + min(mb + 256 * u + tid, a.M - 1)];
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (mb + 256 * u + tid < a.M) {
                    big |= !(v[u][r] <= kLooseBoundRange);
                    mid |= !(v[u][r] <= kGradProductRange);
                    wide[r] |= !(v[u][r] <= kGradRowsRange);
                }
    }
    __syncthreads();
    const bool first = (tid & 63) == 0;
#pragma unroll
    for (int r = 0; r < 4; ++r)
        if (__any(wide[r]) && first)
            flags[r] = 1;   // (every writer writes the same value)
    if (__any(mid) && first)
        flags[5] = 1;
    if (__any(big) && first)
        flags[4] = 1;
    __syncthreads();
}

// Input gradient.  Workgroup (rows_block) x: chunk of 256 pixels; y: tile of 16 * KSUB patch elements; z: split of the
// instance groups.  Per instance group the pixel factors W [32][256] are formed from rows of `out` and `g`, the four
// regions' offset exponentials [16 * KSUB][32] come from the packed offsets, and wave r accumulates region r's
// 16 * KSUB x 64 gradients; these leave through a tile [patch element][column], times 2^(xs - a) from rows of the
// input, as rows of the gradient.  A region with a wide offsets range is done term by term (the other three are not
// held up by it).
template <int KSUB>
__global__ __launch_bounds__(256, KSUB == 1 ? 3 : KSUB == 2 ? 2 : 1) void mex_grad_input_rows_kernel(const MexGradArgs ga, const RowsArgs g)
{
    const MexKernelArgs &a = ga.k;
    constexpr int KT = 16 * KSUB;
    constexpr int WP = 272, EP = 36, OP = 260;   // row pitches: the matrix steps' and the tile's accesses hit 64 banks
    constexpr int kWt = 32 * WP, kEo = 4 * KT * EP, kOt = KT * OP;
    constexpr int kTile = kWt + kEo > kOt ? kWt + kEo : kOt;
    __shared__ __attribute__((aligned(16))) float smem[kTile];
    __shared__ float ap[256];          // per column: the pixel's bound (0 for an empty slot)
    __shared__ float tab[2][128];      // per (region, instance of the group): omax + c0, for this group and the next
    __shared__ int wide_sh[6];         // per region: term by term; [4]: some range beyond the loose bound's
    float *wt = smem, *eo = smem + kWt, *ot = smem;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 15, lq = lane >> 4;
    int chunk, by, bz;
    if (!rows_block(g, &chunk, &by, &bz))
        return;
    const int k0 = by * KT;
    const int n_mg = a.n_mgroups, per = n_mg * GM_TM;
    const int mg_begin = bz * ga.mg_per_split, mg_end = min(n_mg, mg_begin + ga.mg_per_split);
    float *dxo = ga.msplit > 1 ? ga.dx_splits + (size_t)bz * a.B * a.C * a.H * a.W : ga.dx;
    const RowsQuad q = rows_quad(a, g, chunk, lane);
    const int pl0 = wave;              // this thread's planes of a block of 32: pl0, pl0 + 4, ...
    const size_t HW = (size_t)g.HW;
    const size_t img = q.img_ok ? q.img : 0;
    // operands of an instance group: this thread's eight rows pieces of `out` and `g`, its share of the four regions'
    // offset exponentials, the next group's instance constants - requested a group ahead (the first before the bound
    // is worked out, the others while the matrix steps run)
    float4 ov[8], gv[8], en[2 * KSUB];
    float tn = 0.0f;
    auto request = [&](int mg) {
        // (those past the last instance, image or patch element on a clamped address or skipped)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int m = min(mg * GM_TM + pl0 + 4 * j, a.M - 1);
            ov[j] = *reinterpret_cast<const float4 *>(ga.out + (img * a.M + m) * HW + q.pix0);
            gv[j] = rows_load_g(ga, g, q, img, m);
        }
#pragma unroll
        for (int j = 0; j < 2 * KSUB; ++j) {
            const int i = tid + 256 * j;
            const int r = i / (KT * 8), row = (i % (KT * 8)) >> 3, c4 = i & 7;
            en[j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (k0 + row < a.K)
                en[j] = *reinterpret_cast<const float4 *>(a.offe + (((size_t)r * n_mg + mg) * a.K + k0 + row) * GM_TM + 4 * c4);
        }
        if (tid < 128 && mg + 1 < mg_end)
            tn = a.omax[(tid >> 5) * per + (mg + 1) * GM_TM + (tid & 31)] + a.c0;
    };
    if (mg_begin < mg_end)
        request(mg_begin);
    // ---- the bound of every pixel: a = min over (a few) instances of outs_m - c0 - lo_m, see
    //      mex_grad_input_mfma_kernel.  The rows of the first four instances, which give it unless some offsets
    //      range is large, are requested before the ranges are looked at ----
    float4 bo[8];
    float lo_n = 0.0f;
    auto request_bound = [&](int mb, int m_scan) {
        if (tid < 128) {
            const int m = min(mb + (tid & 31), a.M - 1);
            lo_n = a.omax[(tid >> 5) * per + m] - a.orng[(tid >> 5) * per + m];
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int m = mb + pl0 + 4 * j;
            bo[j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (q.img_ok && m < m_scan)
                bo[j] = *reinterpret_cast<const float4 *>(ga.out + (img * a.M + m) * HW + q.pix0);
        }
    };
    request_bound(0, min(a.M, 4));
    rows_ranges(a, tid, wide_sh);
    const int roomy = wide_sh[4];
    const bool slot_ok = chunk * 64 + (tid & 63) < a.slots;
    // Large offsets ranges: the bound from `out` and the offsets' minima is loose by up to the range, which costs the
    // factors their precision (and, beyond kGradProductRange, the product form).  The pixel's own maximum over all of
    // K - one sweep over the rows of the input - is tight: the exponents then stay within the pixel's patch range, and
    // a region keeps the product form while those ranges are at most kGradPixelRange and its offsets span at most
    // kGradRowsRange.
    float amin = INFINITY;             // the bound of column tid
    if (roomy) {
        float amax = -INFINITY, alo = INFINITY;
        for (int kb = 0; kb < a.K; kb += 32) {
            float4 xr[8];
#pragma unroll
            for (int j = 0; j < 8; ++j)
                xr[j] = *reinterpret_cast<const float4 *>(a.in + (img * a.K + min(kb + pl0 + 4 * j, a.K - 1)) * HW + q.pix0);
            __syncthreads();           // the previous block's readers are done with the tile
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int pl = pl0 + 4 * j;
                const bool use = q.img_ok && kb + pl < a.K;
                const float v[4] = {xr[j].x, xr[j].y, xr[j].z, xr[j].w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    wt[pl * WP + q.col[e]] = use ? v[e] * a.c1 : __builtin_nanf("");   // (fmax / fmin skip NaN)
            }
            __syncthreads();
#pragma unroll 8
            for (int pl = 0; pl < 32; ++pl) {
                const float t = wt[pl * WP + tid];
                amax = fmaxf(amax, t);
                alo = fminf(alo, t);
            }
        }
        // a pixel with an infinite value, nothing finite, or a patch range beyond the bound sends its region term by term
        const bool px_ok = !slot_ok || (fabsf(amax) < INFINITY && amax - alo <= kGradPixelRange);
        const int bad = __any(!px_ok) ? 1 : 0;
        if (lane == 0)
            wide_sh[wave] |= bad;      // (columns of wave w belong to region w)
        amin = amax;
    }
    const int m_scan = roomy ? 0 : min(a.M, 4);
    for (int mb = 0; mb < m_scan; mb += 32) {
        if (tid < 128)
            tab[0][tid] = lo_n;
        __syncthreads();               // tab in place; the previous block's readers are done with the tile
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int pl = pl0 + 4 * j;
            const bool use = q.img_ok && mb + pl < m_scan;
            const float v[4] = {bo[j].x, bo[j].y, bo[j].z, bo[j].w};
#pragma unroll
            for (int e = 0; e < 4; ++e)
                wt[pl * WP + q.col[e]] =
                    use ? __builtin_fmaf(v[e], a.c1, -(a.c0 + tab[0][(q.rbase + (e & 1)) * 32 + pl])) : INFINITY;
        }
        __syncthreads();
#pragma unroll 8
        for (int pl = 0; pl < 32; ++pl)
            amin = fminf(amin, wt[pl * WP + tid]);
    }
    ap[tid] = slot_ok ? amin : 0.0f;
    if (tid < 128 && mg_begin < mg_end)   // (the loop above is done with the table: its last readers passed the
        tab[mg_begin & 1][tid] = a.omax[(tid >> 5) * per + mg_begin * GM_TM + (tid & 31)] + a.c0;   // barrier in front of the reduction)
    __syncthreads();
    const bool my_wide = wide_sh[wave] != 0;
    const bool any_wide = (wide_sh[0] | wide_sh[1] | wide_sh[2] | wide_sh[3]) != 0;
    float bound[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
        bound[e] = ap[q.col[e]];

    floatx4 acc[KSUB][4];
#pragma unroll
    for (int ks = 0; ks < KSUB; ++ks)
#pragma unroll
        for (int t = 0; t < 4; ++t)
            acc[ks][t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    constexpr int NJ = KT / 4;
    float4 xv[NJ];                     // the epilogue's rows of the input, requested during the last matrix steps
    for (int mg = mg_begin; mg < mg_end; ++mg) {
        __syncthreads();               // the previous group's matrix steps are done with wt / eo
        const float *tb = tab[mg & 1];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int pl = pl0 + 4 * j;
            const bool use = q.img_ok && mg * GM_TM + pl < a.M;
            const float o[4] = {ov[j].x, ov[j].y, ov[j].z, ov[j].w};
            float gg[4];
            rows_quad_g(ga, gv[j], gg);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                // (a - outs) first: a small, once-rounded difference; the instance constant is added to that (forming
                // a + mo first, about the size of outs, was tried for the tight bound: worse on half of the data)
                const float ex = __builtin_fmaf(-o[e], a.c1, bound[e]) + tb[(q.rbase + (e & 1)) * 32 + pl];
                wt[pl * WP + q.col[e]] = use ? gg[e] * __builtin_amdgcn_exp2f(ex) : 0.0f;
            }
        }
#pragma unroll
        for (int j = 0; j < 2 * KSUB; ++j) {
            const int i = tid + 256 * j;
            const int r = i / (KT * 8), row = (i % (KT * 8)) >> 3, c4 = i & 7;
            *reinterpret_cast<float4 *>(eo + (r * KT + row) * EP + 4 * c4) = en[j];
        }
        if (tid < 128)
            tab[(mg + 1) & 1][tid] = tn;
        if (mg + 1 < mg_end) {
            request(mg + 1);
        } else {
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const int k = min(k0 + pl0 + 4 * j, a.K - 1);
                xv[j] = *reinterpret_cast<const float4 *>(a.in + (img * a.K + k) * HW + q.pix0);
            }
        }
        __syncthreads();
        if (!my_wide) {
#pragma unroll
            for (int ms = 0; ms < GM_TM; ms += 4) {
                float bv[4];
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    bv[t] = wt[(ms + lq) * WP + wave * 64 + t * 16 + lr];
#pragma unroll
                for (int ks = 0; ks < KSUB; ++ks) {
                    const float av = eo[(wave * KT + ks * 16 + lr) * EP + ms + lq];
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        acc[ks][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv[t], acc[ks][t], 0, 0, 0);
                }
            }
        }
    }
    // ---- d patch_k = 2^(xs_k - a) * acc: through the tile [patch element][column] to rows of the gradient ----
    if (mg_begin >= mg_end) {
#pragma unroll
        for (int j = 0; j < NJ; ++j)
            xv[j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
    __syncthreads();                   // the last matrix steps are done with wt / eo, which the tile overlies
#pragma unroll
    for (int ks = 0; ks < KSUB; ++ks)
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v)
                ot[(ks * 16 + 4 * lq + v) * OP + wave * 64 + t * 16 + lr] = acc[ks][t][v];
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const int kl = pl0 + 4 * j, k = k0 + kl;
        if (!q.img_ok || k >= a.K)
            continue;
        const float x[4] = {xv[j].x, xv[j].y, xv[j].z, xv[j].w};
        float d[4];
#pragma unroll
        for (int e = 0; e < 4; ++e)
            d[e] = ot[kl * OP + q.col[e]] * __builtin_amdgcn_exp2f(__builtin_fmaf(x[e], a.c1, -bound[e]));
        float *dst = dxo + (img * a.K + k) * HW + q.pix0;
        if (!any_wide) {
            *reinterpret_cast<float4 *>(dst) = make_float4(d[0], d[1], d[2], d[3]);
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (!wide_sh[q.rbase + (e & 1)])
                    dst[e] = d[e];
        }
    }
    if (any_wide) {
        // the regions with a wide offsets range, term by term: GX_KT patch elements of a region per wave and turn
        constexpr int NSUB = KT / GX_KT;
        for (int u = wave; u < 4 * NSUB; u += 4) {
            const int r = u / NSUB, kk0 = k0 + (u % NSUB) * GX_KT;
            if (wide_sh[r] && kk0 < a.K)
                mex_grad_input_wave(ga, r, chunk, kk0, lane, min(a.M, mg_begin * GM_TM), min(a.M, mg_end * GM_TM), dxo);
        }
    }
}

// Offsets gradient.  Workgroup (rows_block) x: group of ga.pxl chunks of 256 pixels; y: tile of 32 instances; z: tile
// of 32 patch elements.  Per chunk the tile's pixel factors W [32][256] and patch exponentials [32][256] are formed from
// rows of `out`, `g` and the input - relative to the bound over the tile's own instances, which the rows just read
// give - and wave r adds region r's 32 x 32 products over its 64 columns.  Partial sums [chunk group][region][M][K]
// like mex_grad_offsets_mfma_kernel's.
__global__ __launch_bounds__(256, 2) void mex_grad_offsets_rows_kernel(const MexGradArgs ga, const RowsArgs g)
{
    const MexKernelArgs &a = ga.k;
    constexpr int TP = 260;
    __shared__ float wt[32 * TP];      // [instance][column]
    __shared__ float ex[32 * TP];      // [patch element][column]
    __shared__ float pm[4 * 256];      // per column: the four waves' minima
    __shared__ int wide_sh[6];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lr = lane & 15, lq = lane >> 4;
    int bx, by, bz;
    if (!rows_block(g, &bx, &by, &bz))
        return;
    const int m0 = by * 32, k0 = bz * 32;
    const int n_mg = a.n_mgroups, per = n_mg * GM_TM;
    const int pl0 = wave;
    const size_t HW = (size_t)g.HW;
    // the constants of this thread's planes for its two regions (the same in every chunk)
    const RowsQuad q0 = rows_quad(a, g, 0, lane);   // (the columns and regions are the same in every chunk)
    const int rbase = q0.rbase;
    float lo[8][2], omc[8][2];
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int par = 0; par < 2; ++par) {
            const int idx = (rbase + par) * per + min(m0 + pl0 + 4 * j, a.M - 1);
            const float om = a.omax[idx];
            lo[j][par] = a.c0 + (om - a.orng[idx]);
            omc[j][par] = om + a.c0;
        }
    floatx4 acc[2][2];
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
            acc[mt][kt] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
    // the rows of a chunk: this thread's pieces of eight instances of `out` and `g` and of eight channels of the
    // input; those of chunk s + 1 are requested as soon as chunk s has gone to LDS, in front of its matrix steps
    float4 ov[8], gv[8], xv[8];
    bool img_ok = false;
    auto request = [&](int s) {
        const RowsQuad q = rows_quad(a, g, bx * ga.pxl + s, lane);
        img_ok = q.img_ok;
        const size_t img = q.img_ok ? q.img : 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int m = min(m0 + pl0 + 4 * j, a.M - 1), k = min(k0 + pl0 + 4 * j, a.K - 1);
            ov[j] = *reinterpret_cast<const float4 *>(ga.out + (img * a.M + m) * HW + q.pix0);
            gv[j] = rows_load_g(ga, g, q, img, m);
            xv[j] = *reinterpret_cast<const float4 *>(a.in + (img * a.K + k) * HW + q.pix0);
        }
    };
    // chunks of this workgroup that hold pixels (uniform)
    const int n_steps = min(ga.pxl, ga.slots_pad / 64 - bx * ga.pxl);
    if (n_steps > 0)
        request(0);
    rows_ranges(a, tid, wide_sh);      // (behind the requests above: one wait for everything)
    // Some range beyond kGradProductRange: the bound of every pixel is its own maximum over all of K (a sweep over the
    // rows of the input per chunk, see mex_grad_input_rows_kernel); a region then keeps the product form unless a range
    // of its offsets is beyond kGradRowsRange (or not finite) or one of its pixels spans more than kGradPixelRange
    // (found while sweeping: `bad`, which discards the region's sums at the end).
    const bool sweep = wide_sh[5] != 0;
    const bool unbounded = wide_sh[wave] != 0;   // (or beyond kGradRowsRange: term by term whatever the pixels)
    int bad = unbounded ? 1 : 0;
    // the offset exponentials of the epilogue: requested in front of the last matrix steps
    float eov[2][2][4];
    for (int s = 0; s < n_steps; ++s) {
        const bool cur_ok = img_ok;
        float cand[4] = {INFINITY, INFINITY, INFINITY, INFINITY};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (m0 + pl0 + 4 * j >= a.M)
                continue;
            const float o[4] = {ov[j].x, ov[j].y, ov[j].z, ov[j].w};
#pragma unroll
            for (int e = 0; e < 4; ++e)
                cand[e] = fminf(cand[e], __builtin_fmaf(o[e], a.c1, -lo[j][e & 1]));
        }
        float bound[4];
        if (sweep) {
            const RowsQuad q = rows_quad(a, g, bx * ga.pxl + s, lane);
            const size_t img = q.img_ok ? q.img : 0;
            float amax = -INFINITY, alo = INFINITY;
            for (int kb = 0; kb < a.K; kb += 32) {
                __syncthreads();       // the previous matrix steps / the previous block's readers are done with the tile
                // (two rows at a time: the chunk's own operands stay in their registers meanwhile)
#pragma unroll
                for (int h = 0; h < 4; ++h) {
                    float4 xr[2];
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        xr[j] = *reinterpret_cast<const float4 *>(
                            a.in + (img * a.K + min(kb + pl0 + 4 * (2 * h + j), a.K - 1)) * HW + q.pix0);
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const int pl = pl0 + 4 * (2 * h + j);
                        const bool use = q.img_ok && kb + pl < a.K;
                        const float v[4] = {xr[j].x, xr[j].y, xr[j].z, xr[j].w};
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            wt[pl * TP + q0.col[e]] = use ? v[e] * a.c1 : __builtin_nanf("");   // (fmax / fmin skip NaN)
                    }
                }
                __syncthreads();
#pragma unroll 8
                for (int pl = 0; pl < 32; ++pl) {
                    const float t = wt[pl * TP + tid];
                    amax = fmaxf(amax, t);
                    alo = fminf(alo, t);
                }
            }
            const bool slot_ok = (bx * ga.pxl + s) * 64 + (tid & 63) < a.slots;
            const bool px_ok = !slot_ok || (fabsf(amax) < INFINITY && amax - alo <= kGradPixelRange);
            bad |= __any(!px_ok) ? 1 : 0;          // (columns of wave w belong to region w)
            pm[tid] = slot_ok ? amax : 0.0f;
            __syncthreads();
#pragma unroll
            for (int e = 0; e < 4; ++e)
                bound[e] = cur_ok ? pm[q0.col[e]] : 0.0f;
        } else {
            __syncthreads();           // the previous chunk's matrix steps are done with wt / ex, its readers with pm
#pragma unroll
            for (int e = 0; e < 4; ++e)
                pm[pl0 * 256 + q0.col[e]] = cand[e];
            __syncthreads();
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int c = q0.col[e];
                bound[e] = cur_ok ? fminf(fminf(pm[c], pm[256 + c]), fminf(pm[512 + c], pm[768 + c])) : 0.0f;
            }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int pl = pl0 + 4 * j;
            const bool use_m = cur_ok && m0 + pl < a.M, use_k = cur_ok && k0 + pl < a.K;
            const float o[4] = {ov[j].x, ov[j].y, ov[j].z, ov[j].w};
            float gg[4];
            rows_quad_g(ga, gv[j], gg);
            const float x[4] = {xv[j].x, xv[j].y, xv[j].z, xv[j].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float we = __builtin_fmaf(-o[e], a.c1, bound[e]) + omc[j][e & 1];
                wt[pl * TP + q0.col[e]] = use_m ? gg[e] * __builtin_amdgcn_exp2f(we) : 0.0f;
                ex[pl * TP + q0.col[e]] = use_k ? __builtin_amdgcn_exp2f(__builtin_fmaf(x[e], a.c1, -bound[e])) : 0.0f;
            }
        }
        if (s + 1 < n_steps) {
            request(s + 1);
        } else {
#pragma unroll
            for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int m = min(m0 + mt * 16 + 4 * lq + v, a.M - 1);
                    const float *eo = a.offe + (((size_t)wave * n_mg + m / GM_TM) * a.K) * GM_TM + m % GM_TM;
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt)
                        eov[mt][kt][v] = eo[(size_t)min(k0 + kt * 16 + lr, a.K - 1) * GM_TM];
                }
        }
        __syncthreads();
        if (!unbounded) {
#pragma unroll 4
            for (int ps = 0; ps < 64; ps += 4) {
                float wa[2], xb[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    wa[i] = wt[(i * 16 + lr) * TP + wave * 64 + ps + lq];
                    xb[i] = ex[(i * 16 + lr) * TP + wave * 64 + ps + lq];
                }
#pragma unroll
                for (int mt = 0; mt < 2; ++mt)
#pragma unroll
                    for (int kt = 0; kt < 2; ++kt)
                        acc[mt][kt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wa[mt], xb[kt], acc[mt][kt], 0, 0, 0);
            }
        }
    }
    // ---- partial sums of this chunk group: acc * 2^(os_mk - mo_m) ----
    if (sweep) {
        __syncthreads();               // (everyone has read the flags)
        if (lane == 0)
            wide_sh[wave] = bad;
        __syncthreads();
    }
    const bool my_wide = wide_sh[wave] != 0;
    const bool any_wide = (wide_sh[0] | wide_sh[1] | wide_sh[2] | wide_sh[3]) != 0;
    if (!my_wide) {
        float *dst = ga.partial + ((size_t)bx * a.R + wave) * a.M * a.K;
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int m = m0 + mt * 16 + 4 * lq + v;
                if (m >= a.M)
                    continue;
#pragma unroll
                for (int kt = 0; kt < 2; ++kt) {
                    const int k = k0 + kt * 16 + lr;
                    if (k < a.K)
                        dst[(size_t)m * a.K + k] = acc[mt][kt][v] * eov[mt][kt][v];
                }
            }
    }
    if (any_wide) {
        // the regions with a wide offsets range, term by term: this workgroup's tile as GO_MT x GO_KT wave tiles
        constexpr int NU = (32 / GO_MT) * (32 / GO_KT);
        for (int u = wave; u < 4 * NU; u += 4) {
            const int r = u / NU, i = u % NU;
            const int mm0 = m0 + (i / (32 / GO_KT)) * GO_MT, kk0 = k0 + (i % (32 / GO_KT)) * GO_KT;
            if (wide_sh[r] && mm0 < a.M && kk0 < a.K)
                mex_grad_offsets_wave(ga, r, bx, mm0, kk0, lane);
        }
    }
}

// dOff[r,m,k] = sum over pixel chunks, in a fixed order (reproducible): a workgroup takes 32 consecutive elements,
// its 8 groups of 32 threads each sum every 8th chunk in chunk order, and the 8 sums are added in group order.
__global__ __launch_bounds__(256) void mex_grad_offsets_finish_kernel(const float *__restrict__ partial, long long n,
                                                                     int chunks, float *__restrict__ doff)
{
    __shared__ float sm[8][32];
    const int e = threadIdx.x & 31, sub = threadIdx.x >> 5;
    for (long long i0 = (long long)blockIdx.x * 32; i0 < n; i0 += (long long)gridDim.x * 32) {
        const long long i = i0 + e;
        float s = 0.0f;
        if (i < n)
            for (int c = sub; c < chunks; c += 8)
                s += partial[(size_t)c * n + i];
        sm[sub][e] = s;
        __syncthreads();
        if (sub == 0 && i < n) {
            float t = sm[0][e];
#pragma unroll
            for (int j = 1; j < 8; ++j)
                t += sm[j][e];
            doff[i] = t;
        }
        __syncthreads();
    }
}

// One wave per (region, instance) row: n = o - logsumexp(o)  (python/simnets/keras.py:155-160).
__global__ __launch_bounds__(256) void mex_normalize_rows_kernel(const float *__restrict__ src, long long rows, int K,
                                                                float *__restrict__ dst)
{
    const int lane = threadIdx.x & 63;
    const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows)
        return;
    const float *s = src + (size_t)row * K;
    float mxv = -INFINITY;
    for (int k = lane; k < K; k += 64)
        mxv = fmaxf(mxv, s[k]);
    for (int d = 32; d > 0; d >>= 1)
        mxv = fmaxf(mxv, __shfl_xor(mxv, d, 64));
    if (!(fabsf(mxv) < INFINITY))
        mxv = 0.0f;
    float sum = 0.0f;
    for (int k = lane; k < K; k += 64)
        sum += mex_exp_term(s[k] - mxv);   // (the pack kernel's arithmetic: both write the same normalised rows)
    for (int d = 32; d > 0; d >>= 1)
        sum += __shfl_xor(sum, d, 64);
    const float lse = mex_lse_of(sum, mxv);
    for (int k = lane; k < K; k += 64)
        dst[(size_t)row * K + k] = s[k] - lse;
}

// Chain rule through the normalisation n = o - logsumexp(o): d/do_j = G_j - exp(n_j) * sum_k G_k, in place.
__global__ __launch_bounds__(256) void mex_normalize_rows_backward_kernel(const float *__restrict__ normalized,
                                                                         long long rows, int K, float *__restrict__ grad)
{
    const int lane = threadIdx.x & 63;
    const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows)
        return;
    float *gr = grad + (size_t)row * K;
    const float *n = normalized + (size_t)row * K;
    float sum = 0.0f;
    for (int k = lane; k < K; k += 64)
        sum += gr[k];
    for (int d = 32; d > 0; d >>= 1)
        sum += __shfl_xor(sum, d, 64);
    for (int k = lane; k < K; k += 64)
        gr[k] -= expf(n[k]) * sum;
}

// Elements lane, lane + 64, ... of one row of the offsets gradient from its partial sums (eight interleaved sums in
// chunk order, added in order), E elements at a time; returns the lane's share of the row sum (in element order).
// (NB: rounds of eight chunks requested together; the additions keep the order of one round at a time)
template <int E, int STRIDE = 64, int NB = 1>
__device__ __forceinline__ float finish_long_row(const float *__restrict__ pr, float *__restrict__ gr, long long n,
                                                 int chunks, int K, int lane)
{
    float sum = 0.0f;
    for (int k0 = lane; k0 < K; k0 += STRIDE * E) {
        float s8[E][8];
#pragma unroll
        for (int e = 0; e < E; ++e)
#pragma unroll
            for (int j = 0; j < 8; ++j)
                s8[e][j] = 0.0f;
        for (int c0 = 0; c0 < chunks; c0 += 8 * NB) {
            // all requests first, those past the last chunk or the row's end on a valid address (a load inside the
            // condition would be waited for before the next one is issued)
            float v[NB][E][8];
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int e = 0; e < E; ++e)
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        v[b][e][j] = pr[(size_t)min(c0 + 8 * b + j, chunks - 1) * n + min(k0 + STRIDE * e, K - 1)];
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int e = 0; e < E; ++e)
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        s8[e][j] = c0 + 8 * b + j < chunks ? s8[e][j] + v[b][e][j] : s8[e][j];
        }
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float t = s8[e][0];
#pragma unroll
            for (int j = 1; j < 8; ++j)
                t += s8[e][j];
            if (k0 + STRIDE * e < K) {
                gr[k0 + STRIDE * e] = t;
                sum += t;
            }
        }
    }
    return sum;
}

// Both of the above for short rows, one wave per (region, instance) row: element k of the row is the sum of its
// partial sums in the order of mex_grad_offsets_finish_kernel (eight interleaved sums in chunk order, added in
// order), then, if `normalized` is given, the chain rule of mex_normalize_rows_backward_kernel with the same
// reduction over the row: the same values as the two launches, in one.
constexpr int kFinishRowsMaxK = 1024;
__global__ __launch_bounds__(256) void mex_grad_offsets_finish_rows_kernel(const float *__restrict__ partial, long long n,
                                                                          int chunks, long long rows, int K,
                                                                          const float *__restrict__ normalized,
                                                                          float *__restrict__ doff)
{
    const int lane = threadIdx.x & 63;
    const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows)
        return;
    float *gr = doff + (size_t)row * K;
    const float *pr = partial + (size_t)row * K;
    float sum = 0.0f;
    if (K <= 32 && (K & 3) == 0) {
        // short rows of whole 16-byte pieces: lane (q, j) = (lane & 7, lane >> 3) takes piece q (elements 4 q ... 4 q + 3)
        // of the chunks j, j + 8, ... - the interleaved sum j -, eight of them requested at a time; lane (q, 0) then
        // adds the eight sums in order.  The values are those of the loops below.
        const int Kq = K >> 2, q = lane & 7, j = lane >> 3, qc = min(q, Kq - 1);
        const long long n4 = n >> 2;
        const float4 *pr4 = reinterpret_cast<const float4 *>(pr) + qc;
        float4 sj = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        for (int c0 = j; c0 < chunks; c0 += 64) {
            float4 v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                v[u] = pr4[(size_t)min(c0 + 8 * u, chunks - 1) * n4];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (c0 + 8 * u < chunks) {
                    sj.x += v[u].x; sj.y += v[u].y; sj.z += v[u].z; sj.w += v[u].w;
                }
        }
        float4 t4 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
        for (int jj = 0; jj < 8; ++jj) {
            const float4 val = make_float4(__shfl(sj.x, q + 8 * jj, 64), __shfl(sj.y, q + 8 * jj, 64),
                                           __shfl(sj.z, q + 8 * jj, 64), __shfl(sj.w, q + 8 * jj, 64));
            if (jj == 0)
                t4 = val;
            else {
                t4.x += val.x; t4.y += val.y; t4.z += val.z; t4.w += val.w;
            }
        }
        if (normalized == nullptr) {
            if (j == 0 && q < Kq) {
                if ((reinterpret_cast<uintptr_t>(gr) & 15) == 0)
                    reinterpret_cast<float4 *>(gr)[q] = t4;
                else {
                    gr[4 * q] = t4.x; gr[4 * q + 1] = t4.y; gr[4 * q + 2] = t4.z; gr[4 * q + 3] = t4.w;
                }
            }
            return;
        }
        // element k to lane k (it lives in lane k / 4), then the row sum and the chain rule as below
        const int k = lane & 31;
        const float a0 = __shfl(t4.x, k >> 2, 64), a1 = __shfl(t4.y, k >> 2, 64), a2 = __shfl(t4.z, k >> 2, 64),
                    a3 = __shfl(t4.w, k >> 2, 64);
        const float t = (k & 3) == 0 ? a0 : (k & 3) == 1 ? a1 : (k & 3) == 2 ? a2 : a3;
        const bool owner = lane < K;
        sum = owner ? t : 0.0f;
        for (int d = 32; d > 0; d >>= 1)
            sum += __shfl_xor(sum, d, 64);
        if (owner)
            gr[k] = t - expf(normalized[(size_t)row * K + k]) * sum;
        return;
    }
    if (K <= 32) {
        // rows shorter than a wave: the lanes form 64 / Kp groups (Kp = 8, 16 or 32 >= K) that each take 8 / groups
        // of the eight interleaved sums, four rounds of chunks requested at a time; every lane then adds the eight
        // sums in order (read from the lanes that hold them), so the values are those of the loop below
        const int lg = K <= 8 ? 3 : K <= 16 ? 4 : 5, Kp = 1 << lg;
        const int per = 8 >> (6 - lg);               // sums per group: 1, 2 or 4
        const int gi = lane >> lg, k = lane & (Kp - 1), kc = min(k, K - 1);
        float sj[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int c0 = 0; c0 < chunks; c0 += 32) {
            float v[4][4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (i < per)
                        v[u][i] = pr[(size_t)min(c0 + 8 * u + gi * per + i, chunks - 1) * n + kc];
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (i < per && c0 + 8 * u + gi * per + i < chunks)
                        sj[i] += v[u][i];
        }
        float t = 0.0f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int i = j & (per - 1), src = ((j >> (lg - 3)) << lg) + k;   // sum j lives in group j / per, slot j % per
            const float mine = i == 0 ? sj[0] : i == 1 ? sj[1] : i == 2 ? sj[2] : sj[3];
            const float val = __shfl(mine, src, 64);
            t = j == 0 ? val : t + val;
        }
        const bool owner = gi == 0 && k < K;
        if (owner)
            gr[k] = t;
        if (normalized == nullptr)
            return;
        sum = owner ? t : 0.0f;
        for (int d = 32; d > 0; d >>= 1)
            sum += __shfl_xor(sum, d, 64);
        if (owner)
            gr[k] = t - expf(normalized[(size_t)row * K + k]) * sum;
        return;
    }
    // up to four elements of the row per lane at a time (64 apart): 8 requests each in flight
    if (K <= 64)
        sum = finish_long_row<1>(pr, gr, n, chunks, K, lane);
    else if (K <= 128)
        sum = finish_long_row<2>(pr, gr, n, chunks, K, lane);
    else
        sum = finish_long_row<4>(pr, gr, n, chunks, K, lane);
    if (normalized == nullptr)
        return;
    for (int d = 32; d > 0; d >>= 1)
        sum += __shfl_xor(sum, d, 64);
    const float *nr = normalized + (size_t)row * K;
    for (int k = lane; k < K; k += 64)
        gr[k] -= expf(nr[k]) * sum;   // reads back what this lane stored above
}

// The same for few long rows (a classifier head: 10 rows of 512): one workgroup per row, the four waves split its
// elements (thread t takes t, t + 256, ...), the row sum of the chain rule goes through LDS.
__global__ __launch_bounds__(256) void mex_grad_offsets_finish_wide_rows_kernel(const float *__restrict__ partial,
                                                                               long long n, int chunks, int K,
                                                                               const float *__restrict__ normalized,
                                                                               float *__restrict__ doff)
{
    __shared__ float ws[4];
    const long long row = blockIdx.x;
    float *gr = doff + (size_t)row * K;
    const float *pr = partial + (size_t)row * K;
    const int tid = threadIdx.x;
    float sum = K <= 256 ? finish_long_row<1, 256, 4>(pr, gr, n, chunks, K, tid)
                         : (K <= 512 ? finish_long_row<2, 256, 2>(pr, gr, n, chunks, K, tid)
                                     : finish_long_row<4, 256, 1>(pr, gr, n, chunks, K, tid));
    if (normalized == nullptr)
        return;
    for (int d = 32; d > 0; d >>= 1)
        sum += __shfl_xor(sum, d, 64);
    if ((tid & 63) == 0)
        ws[tid >> 6] = sum;
    __syncthreads();
    sum = (ws[0] + ws[1]) + (ws[2] + ws[3]);
    const float *nr = normalized + (size_t)row * K;
    for (int k = tid; k < K; k += 256)
        gr[k] -= expf(nr[k]) * sum;   // reads back what this thread stored above
}

// Few instances over long patches on few pixels (a network's classifier head: 10 instances x 512 channels on one
// pixel per image): the tiled kernels above would run a handful of workgroups in long serial chains, in three
// launches.  Here a thread owns one patch element k (a workgroup spans K) and keeps the region's offsets for that
// element in registers; the workgroup walks its share of the pixels, four at a time (their loads in flight
// together), and forms every term as the reference does (mex_term: either epsilon, any offsets range): summed over
// the instances it is the input gradient of (pixel, k), summed over the pixels - in registers - the offsets gradient
// of (instance, k).  No LDS, no barriers; one partial sum [M][K] per workgroup for the finish kernel.
constexpr int kHeadMaxM = 16, kHeadPixels = 4;
template <int MH, bool FINITE>
__global__ __launch_bounds__(1024) void mex_grad_head_kernel(const MexGradArgs ga, int wgs_per_region, int want_input,
                                                             int want_offsets)
{
    static_assert(MH <= 16, "one lane per instance in the load of the gradients and outputs");
    const MexKernelArgs &a = ga.k;
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x / wgs_per_region, wg = blockIdx.x - r * wgs_per_region;
    const int k = threadIdx.x;
    const bool kv = k < a.K;
    const int kk = kv ? k : 0;
    const int bhw = a.bh * a.bw;
    const int dc = kk / bhw, rem = kk - dc * bhw, dh = rem / a.bw, dw = rem - dh * a.bw;
    float of[MH], acc[MH];
#pragma unroll
    for (int m = 0; m < MH; ++m) {
        of[m] = ga.off[((size_t)r * a.M + min(m, a.M - 1)) * a.K + kk];
        acc[m] = 0.0f;
    }
    const size_t plane = (size_t)a.Co * a.Ho * a.Wo, gplane = pooled_g_plane(ga, plane);
    const int ml = min(lane & 15, a.M - 1);
    for (int s0 = wg * kHeadPixels; s0 < a.slots; s0 += wgs_per_region * kHeadPixels) {
        float x[kHeadPixels], go[kHeadPixels];
        int io[kHeadPixels];
        bool valid[kHeadPixels];
        size_t img[kHeadPixels], col[kHeadPixels];
#pragma unroll
        for (int p = 0; p < kHeadPixels; ++p) {
            const int slot = s0 + p;
            const PixelRef px = locate(a, r, min(slot, a.slots - 1));   // (the same pixel for the whole workgroup)
            valid[p] = slot < a.slots && px.out_off >= 0;
            const int ci = px.ci0 + dc, hi = px.hi0 + dh, wi = px.wi0 + dw;
            const bool ok = kv && ci >= 0 && ci < a.C && hi >= 0 && hi < a.H && wi >= 0 && wi < a.W;
            io[p] = ok ? (ci * a.H + hi) * a.W + wi : -1;
            img[p] = (size_t)px.b * a.C * a.H * a.W;
            // (loads on addresses that are always valid, the choice made afterwards: a load inside a condition is
            // waited for before the next one is issued)
            const float xv = a.in[img[p] + (ok ? io[p] : 0)];
            x[p] = ok ? xv : a.oob;
            const int oo = valid[p] ? px.out_off : 0;
            // every instance's gradient (lanes 0 ... 15) and output value (lanes 16 ... 31) through one load, read back
            // lane by lane below
            const float *src = (lane & 16) ? ga.out + ((size_t)px.b * a.M + ml) * plane + oo
                                           : ga.g + ((size_t)px.b * a.M + ml) * gplane + pooled_g_offset(ga, oo);
            go[p] = *src;
            col[p] = ((size_t)px.b * plane + oo) * a.K;
        }
        // Straight-line arithmetic: instances past the last one repeat it with a zero gradient (their sums are never
        // stored), threads past the last patch element compute on the out-of-bounds value (nothing of theirs is
        // stored either); only an empty pixel slot is skipped.
#pragma unroll
        for (int p = 0; p < kHeadPixels; ++p) {
            if (!valid[p])
                continue;
            float dxa = 0.0f;
#pragma unroll
            for (int m = 0; m < MH; ++m) {
                float gm = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, go[p]), m));
                const float om = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, go[p]), 16 + m));
                gm = m < a.M ? gm : 0.0f;
                const float e = mex_term(x[p] + of[m], om, gm, a.c1, a.c0, FINITE);
                dxa += e;
                acc[m] += e;
            }
            if (want_input && io[p] >= 0) {
                if (ga.overlap)
                    ga.col[col[p] + k] = dxa;
                else
                    ga.dx[img[p] + io[p]] = dxa;
            }
        }
    }
    if (!want_offsets || !kv)
        return;
    float *part = ga.partial + ((size_t)wg * a.R + r) * a.M * a.K + k;
#pragma unroll
    for (int m = 0; m < MH; ++m)
        if (m < a.M)
            part[(size_t)m * a.K] = acc[m];
}

__global__ void mex_fill_zero_kernel(float *__restrict__ p, long long n)
{
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
        p[i] = 0.0f;
}

struct MexGradTiling {
    int pxl, cpr_offsets;
    bool head;           // few instances over long patches on few pixels: mex_grad_head_kernel, both gradients
    int head_wgs;        // ... with this many workgroups per region (= partial sums per region)
    bool mfma;           // finite epsilon: the matrix-core kernels, fed by the forward pass's packed offsets
    size_t norm_bytes, partial_bytes, packed_bytes;
    bool overlap;        // input gradient: patches overlap
    size_t col_bytes;    // ... and their per-patch gradients pass through a [B][Co*Ho*Wo][K] buffer
    bool tiles_input;    // patches tile the input exactly: every element is written by exactly one patch
    int msplit, mg_per_split;  // input gradient, matrix form: instance groups split over gridDim.z workgroups
    size_t split_bytes;  // ... whose partial gradients [split][input] are added by mex_sum_splits_kernel
    // factor buffers of mex_grad_factors_kernel: used when a matrix kernel would otherwise form the same factors
    // in several workgroups (more than one tile along the dimension it does not contract)
    bool factors_input, factors_offsets;
    int slots_pad, Mp, Kp;
    size_t factor_bytes;
    // the row-wise kernels (mex_grad_input_rows_kernel, mex_grad_offsets_rows_kernel): the layer qualifies (the
    // pointers are checked at the launch), and their tiling
    bool rows;
    int rows_ksub;                        // input gradient: 16 * ksub patch elements per workgroup
    int rows_msplit, rows_mg_per_split;   // ... and the split of its instance groups
    int rows_pxl, rows_cpr;               // offsets gradient: chunks per workgroup, workgroups along the pixels
};

inline int log2_exact(int v)   // log2 of a power of two, -1 otherwise
{
    int l = 0;
    while ((1 << l) < v)
        ++l;
    return v > 0 && (1 << l) == v ? l : -1;
}

// 2 x 2 unshared offsets over whole-channel patches on a map with power-of-two sides: see the row-wise kernels.
// A chunk of 256 pixels must be whole images or an even number of whole rows (width <= 128), so that it holds
// exactly the 64 slots [64 chunk, 64 chunk + 64) of each of the four regions; a 16-byte piece lies in one row
// (width >= 4).
bool rows_geometry(const MexPlan &p)
{
    const simnets_mex_dims &d = p.d;
    return std::isfinite(p.epsilon) && p.use_unshared && d.offsets_c == 1 && d.offsets_h == 2 && d.offsets_w == 2 &&
           d.channels_out == 1 && d.block_c == p.C && d.block_h == 1 && d.block_w == 1 && d.stride_h == 1 &&
           d.stride_w == 1 && d.pad_c == 0 && d.pad_h == 0 && d.pad_w == 0 && d.height_out == p.H &&
           d.width_out == p.W && log2_exact(p.H) >= 1 && log2_exact(p.W) >= 2 && p.W <= 128 &&
           d.region_size == (p.H / 2) * (p.W / 2) && (long long)p.B * p.H * p.W <= 0x3fffffffLL;
}

MexGradTiling mex_grad_tiling(const MexPlan &p)
{
    const simnets_mex_dims &d = p.d;
    MexGradTiling t;
    const long long slots = (long long)p.B * d.region_size;
    t.mfma = std::isfinite(p.epsilon);
    const long long mk = t.mfma ? 4LL * ((d.M + GOM_MT - 1) / GOM_MT) * ((d.K + GOM_KT - 1) / GOM_KT)
                                : (long long)((d.M + GO_MT - 1) / GO_MT) * ((d.K + GO_KT - 1) / GO_KT);
    auto waves = [&](int pxl) { return d.num_regions * ((slots + 64LL * pxl - 1) / (64LL * pxl)) * mk; };
    t.pxl = 16;
    while (t.pxl > 1 && waves(t.pxl) < (t.mfma ? 2048 : 4096))
        t.pxl >>= 1;
    t.cpr_offsets = (int)((slots + 64LL * t.pxl - 1) / (64LL * t.pxl));
    const size_t rmk = (size_t)d.num_regions * d.M * d.K * sizeof(float);
    t.norm_bytes = p.normalize_offsets ? align_up(rmk, 256) : 0;
    t.partial_bytes = align_up(rmk * t.cpr_offsets, 256);
    t.packed_bytes = t.mfma ? mex_packed_bytes(p, GM_TM, (d.M + GM_TM - 1) / GM_TM) : 0;
    t.overlap = (d.block_c > d.stride_c && d.channels_out > 1) || (d.block_h > d.stride_h && d.height_out > 1) ||
                (d.block_w > d.stride_w && d.width_out > 1);
    t.col_bytes = t.overlap ? align_up((size_t)p.B * d.channels_out * d.height_out * d.width_out * d.K * sizeof(float),
                                       256) : 0;
    t.tiles_input = d.pad_c == 0 && d.pad_h == 0 && d.pad_w == 0 && d.stride_c == d.block_c &&
                    d.stride_h == d.block_h && d.stride_w == d.block_w && d.channels_out * d.block_c == p.C &&
                    d.height_out * d.block_h == p.H && d.width_out * d.block_w == p.W;
    // Few pixels and many instances (deep layers on small maps): a workgroup would walk all instance groups alone
    // while most of the chip idles.  Then the groups are split over up to 8 workgroups (two groups each at least)
    // until the launch has about two workgroups per compute unit.
    t.msplit = 1;
    const int n_mg = (d.M + GM_TM - 1) / GM_TM;
    const long long wgs = (long long)d.num_regions * ((slots + 63) / 64) * ((d.K + GM_KT - 1) / GM_KT);
    if (t.mfma && t.tiles_input && wgs <= 256 && n_mg >= 4)
        t.msplit = (int)std::max<long long>(1, std::min<long long>(std::min(8, n_mg / 2), 512 / std::max<long long>(wgs, 1)));
    t.mg_per_split = (n_mg + t.msplit - 1) / t.msplit;
    t.msplit = (n_mg + t.mg_per_split - 1) / t.mg_per_split;
    t.split_bytes = t.msplit > 1 ? align_up((size_t)t.msplit * p.B * p.C * p.H * p.W * sizeof(float), 256) : 0;
    t.slots_pad = (int)((slots + 63) / 64 * 64);
    t.Mp = n_mg * GM_TM;
    t.Kp = (d.K + 31) / 32 * 32;
    const int k_tiles = (d.K + GM_KT - 1) / GM_KT, m_tiles = (d.M + GOM_MT - 1) / GOM_MT;
    // (the extra launch and the round trip through memory cost about 10 us: measured to pay from 4 tiles of patch
    // elements and 128 instances on for the input gradient and from 16 tiles on for the offsets gradient)
    t.factors_input = t.mfma && k_tiles >= 4 && d.M >= 128;
    t.factors_offsets = t.mfma && m_tiles * ((d.K + GOM_KT - 1) / GOM_KT) >= 16;
    t.factor_bytes = align_up((size_t)d.num_regions * t.slots_pad * ((size_t)t.Mp + t.Kp) * sizeof(float), 256);
    // Row-wise kernels: about two workgroups per compute unit at least.  The input gradient takes as many patch
    // elements per workgroup as that allows (each tile of them reads all of `out` and `g`), then splits the instance
    // groups; the offsets gradient walks as many chunks per workgroup as that allows (each workgroup writes a
    // partial sum of its tile).
    // The head kernel: terms few enough for one exponential each (a classifier head has 512 x 10 x 512 of them)
    t.head = d.M <= kHeadMaxM && d.K >= 64 && d.K <= 1024 && slots >= 1 &&
             (long long)d.num_regions * slots * d.M * d.K <= (16LL << 20) && (long long)p.C * p.H * p.W <= 0x7fffffffLL;
    // (about 8 pixels per workgroup, at most 64 partial sums per region for the finish kernel)
    t.head_wgs = (int)std::max<long long>(1, std::min<long long>((slots + 7) / 8, std::max(1, 64 / d.num_regions)));
    if (t.head)
        t.partial_bytes = std::max(t.partial_bytes, align_up(rmk * t.head_wgs, 256));
    t.rows = rows_geometry(p);
    t.rows_ksub = 1; t.rows_msplit = 1; t.rows_mg_per_split = n_mg; t.rows_pxl = 1; t.rows_cpr = 0;
    if (t.rows) {
        const long long chunks = t.slots_pad / 64;
        auto ktiles = [&](int ksub) { return (long long)((d.K + 16 * ksub - 1) / (16 * ksub)); };
        t.rows_ksub = std::min(4, (d.K + 15) / 16);
        if (t.rows_ksub == 3)
            t.rows_ksub = 4;
        while (t.rows_ksub > 1 && chunks * ktiles(t.rows_ksub) < 512)
            t.rows_ksub >>= 1;
        const long long wgs_in = chunks * ktiles(t.rows_ksub);
        if (wgs_in < 512 && n_mg >= 4)
            t.rows_msplit = (int)std::max<long long>(1, std::min<long long>(std::min(8, n_mg / 2), 512 / std::max<long long>(wgs_in, 1)));
        t.rows_mg_per_split = (n_mg + t.rows_msplit - 1) / t.rows_msplit;
        t.rows_msplit = (n_mg + t.rows_mg_per_split - 1) / t.rows_mg_per_split;
        if (t.rows_msplit > 1)
            t.split_bytes = std::max(t.split_bytes, align_up((size_t)t.rows_msplit * p.B * p.C * p.H * p.W * sizeof(float), 256));
        const long long tiles = (long long)((d.M + 31) / 32) * ((d.K + 31) / 32);
        t.rows_pxl = 16;
        while (t.rows_pxl > 1 && (chunks + t.rows_pxl - 1) / t.rows_pxl * tiles < 512)
            t.rows_pxl >>= 1;
        t.rows_cpr = (int)((chunks + t.rows_pxl - 1) / t.rows_pxl);
        t.partial_bytes = std::max(t.partial_bytes, align_up(rmk * t.rows_cpr, 256));
    }
    return t;
}

// offsets as the forward op used them: the caller's, or their normalised copy in the workspace
int prepare_offsets(const MexPlan &p, const float *offsets, void *workspace, hipStream_t s, const float **used)
{
    *used = offsets;
    if (!p.normalize_offsets)
        return SIMNETS_OK;
    float *norm = reinterpret_cast<float *>(workspace);
    const long long rows = (long long)p.d.num_regions * p.d.M;
    hipLaunchKernelGGL(mex_normalize_rows_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, offsets, rows,
                       p.d.K, norm);
    *used = norm;
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

// Launches mex_grad_factors_kernel into `buffers` and points ga at them (ga.k must hold the packed offsets).
int launch_factors(const MexPlan &p, const MexGradTiling &t, MexGradArgs &ga, void *buffers, hipStream_t s)
{
    ga.slots_pad = t.slots_pad; ga.Mp = t.Mp; ga.Kp = t.Kp;
    ga.wbuf = reinterpret_cast<float *>(buffers);
    ga.exbuf = ga.wbuf + (size_t)p.d.num_regions * t.slots_pad * t.Mp;
    MexGradArgs fa = ga;
    fa.cpr = t.slots_pad / 64;
    const long long gx = (long long)p.d.num_regions * fa.cpr;
    if (gx > 0x7fffffffLL)
        return SIMNETS_ERR_TOO_LARGE;
    const int gy = t.Mp / GM_TM + t.Kp / 32;
    if (gy > 65535)
        return SIMNETS_ERR_TOO_LARGE;
    if (gx > 0)
        hipLaunchKernelGGL(mex_grad_factors_kernel, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, fa);
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

}  // namespace

namespace {

// Scratch of a gradient call, in this order: normalised offsets | packed offsets | offsets-gradient partial sums |
// patch gradients of overlapping patches | partial input gradients of the instance split | factor buffers.
struct MexGradScratch {
    size_t norm, packed, partial, col, split, factors, total;
    bool use_factors;
};

MexGradScratch mex_grad_scratch(const MexGradTiling &t, bool want_input, bool want_offsets)
{
    MexGradScratch w;
    // both gradients in one call: the factors are formed once for the kernels that want them
    w.use_factors = (want_input && t.factors_input) || (want_offsets && t.factors_offsets);
    size_t at = 0;
    w.norm = at;    at += t.norm_bytes;
    w.packed = at;  at += t.packed_bytes;
    w.partial = at; at += want_offsets ? t.partial_bytes : 0;
    w.col = at;     at += want_input ? t.col_bytes : 0;
    w.split = at;   at += want_input ? t.split_bytes : 0;
    w.factors = at; at += w.use_factors ? t.factor_bytes : 0;
    w.total = at;
    return w;
}

}  // namespace

size_t mex_grads_workspace_bytes(const MexPlan &p, bool want_input, bool want_offsets)
{
    return mex_grad_scratch(mex_grad_tiling(p), want_input, want_offsets).total;
}

size_t mex_grad_input_workspace_bytes(const MexPlan &p) { return mex_grads_workspace_bytes(p, true, false); }

size_t mex_grad_offsets_workspace_bytes(const MexPlan &p) { return mex_grads_workspace_bytes(p, false, true); }

// Either gradient or both (a null pointer skips one).  The offsets as the forward op used them, their packed form
// and, where used, the factor buffers are prepared once and shared.
bool mex_grads_take_pooled(const MexPlan &p, const float *input, const float *output, const float *pooled_grad,
                           const float *input_grad)
{
    (void)input; (void)output; (void)pooled_grad; (void)input_grad;   // (any alignment: only the row-wise kernels care)
    // every kernel maps an output pixel to its window (pooled_g_offset): one output channel per instance and no
    // trailing row or column that the pooling dropped
    return p.d.channels_out == 1 && p.d.height_out % 2 == 0 && p.d.width_out % 2 == 0;
}

bool mex_grads_read_packed(const MexPlan &p)
{
    const MexGradTiling t = mex_grad_tiling(p);
    return t.mfma && !t.head;
}

int mex_grad_pack_launch(const MexPlan &p, const float *offsets, void *buffer, void *stream)
{
    MexPlan q = p;
    q.grad_pack = nullptr;
    MexPackTwin tw;
    float *norm;
    mex_grad_pack_layout(q, buffer, &tw, &norm);
    if (tw.offp == nullptr) {   // only the normalised copy is kept
        const float *used;
        return prepare_offsets(q, offsets, norm, reinterpret_cast<hipStream_t>(stream), &used);
    }
    MexKernelArgs a = mex_kernel_args(q);
    return mex_pack_offsets(q, offsets, GM_TM, tw.n_mgroups, buffer, &a, stream, nullptr, true, norm, true);
}

int mex_grads(const MexPlan &p, const float *input, const float *offsets, const float *output,
              const float *output_grad, float *input_grad, float *offsets_grad, void *workspace,
              size_t workspace_bytes, void *stream, bool grad_is_pooled, const void *saved)
{
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const bool want_input = input_grad != nullptr, want_offsets = offsets_grad != nullptr;
    const MexGradTiling t = mex_grad_tiling(p);
    const MexGradScratch w = mex_grad_scratch(t, want_input, want_offsets);
    if (workspace_bytes < w.total)
        return SIMNETS_ERR_WORKSPACE;
    const simnets_mex_dims &d = p.d;
    const long long n_in = (long long)p.B * p.C * p.H * p.W;
    const long long n_off = (long long)d.num_regions * d.M * d.K;
    if (p.B == 0) {  // an empty batch has an empty input gradient and a zero offsets gradient
        if (want_offsets) {
            hipLaunchKernelGGL(mex_fill_zero_kernel, dim3((unsigned)std::min<long long>((n_off + 255) / 256, 65535)),
                               dim3(256), 0, s, offsets_grad, n_off);
            return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
        }
        return SIMNETS_OK;
    }
    if ((n_in + 255) / 256 > 0x7fffffffLL)
        return SIMNETS_ERR_TOO_LARGE;
    char *ws = reinterpret_cast<char *>(workspace);

    MexGradArgs ga;
    ga.k = mex_kernel_args(p);
    ga.k.in = input;
    // the offsets as the forward op used them: with the matrix kernels the pack launch below writes the normalised
    // copy as well, otherwise a launch of its own does
    const bool pack_normalizes = t.mfma && p.normalize_offsets;
    // ... or the forward call left them (and their packed form) in `saved`
    const bool packed_already = saved != nullptr && t.mfma;
    char *packed_at = ws + w.packed;
    float *norm_at = reinterpret_cast<float *>(ws + w.norm);
    if (packed_already) {
        MexPackTwin tw;
        packed_at = reinterpret_cast<char *>(const_cast<void *>(saved));
        mex_grad_pack_layout(p, packed_at, &tw, &norm_at);
    }
    int rc = SIMNETS_OK;
    if (pack_normalizes)
        ga.off = norm_at;
    else
        rc = prepare_offsets(p, offsets, ws + w.norm, s, &ga.off);
    if (rc)
        return rc;
    ga.out = output; ga.g = output_grad;
    ga.gpool = grad_is_pooled ? 1 : 0;
    ga.dx = input_grad;
    ga.partial = reinterpret_cast<float *>(ws + w.partial);
    ga.overlap = 0;
    ga.col = reinterpret_cast<float *>(ws + w.col);
    if (grad_is_pooled && !mex_grads_take_pooled(p, input, output, output_grad, input_grad))
        return SIMNETS_ERR_ALGO;   // (the callers ask first)
    if (t.head) {
        // one launch for both gradients, on the offsets as they are (or their normalised copy): nothing is packed
        if (pack_normalizes && !packed_already) {
            rc = prepare_offsets(p, offsets, ws + w.norm, s, &ga.off);
            if (rc)
                return rc;
        }
        ga.overlap = t.overlap ? 1 : 0;
        if (want_input && !t.overlap && !t.tiles_input) {
            hipLaunchKernelGGL(mex_fill_zero_kernel, dim3((unsigned)std::min<long long>((n_in + 255) / 256, 65535)),
                               dim3(256), 0, s, input_grad, n_in);
            if (hipGetLastError() != hipSuccess)
                return SIMNETS_ERR_HIP;
        }
        const dim3 grid((unsigned)(d.num_regions * t.head_wgs)), block((unsigned)((d.K + 63) / 64 * 64));
        const int wi = want_input ? 1 : 0, wo = want_offsets ? 1 : 0;
#define SIMNETS_HEAD_LAUNCH(MH)                                                                                      \
    if (t.mfma)                                                                                                      \
        hipLaunchKernelGGL((mex_grad_head_kernel<MH, true>), grid, block, 0, s, ga, t.head_wgs, wi, wo);              \
    else                                                                                                             \
        hipLaunchKernelGGL((mex_grad_head_kernel<MH, false>), grid, block, 0, s, ga, t.head_wgs, wi, wo)
        if (d.M <= 4) {
            SIMNETS_HEAD_LAUNCH(4);
        } else if (d.M <= 8) {
            SIMNETS_HEAD_LAUNCH(8);
        } else if (d.M <= 12) {
            SIMNETS_HEAD_LAUNCH(12);
        } else {
            SIMNETS_HEAD_LAUNCH(kHeadMaxM);
        }
#undef SIMNETS_HEAD_LAUNCH
        if (hipGetLastError() != hipSuccess)
            return SIMNETS_ERR_HIP;
        if (want_input && t.overlap) {
            hipLaunchKernelGGL(mex_col2im_kernel, dim3((unsigned)((n_in + 255) / 256)), dim3(256), 0, s, ga.k, ga.col,
                               input_grad, n_in);
            if (hipGetLastError() != hipSuccess)
                return SIMNETS_ERR_HIP;
        }
        if (want_offsets) {
            const long long rows = (long long)d.num_regions * d.M;
            hipLaunchKernelGGL(mex_grad_offsets_finish_wide_rows_kernel, dim3((unsigned)rows), dim3(256), 0, s, ga.partial,
                               n_off, t.head_wgs, d.K, p.normalize_offsets ? ga.off : nullptr, offsets_grad);
            if (hipGetLastError() != hipSuccess)
                return SIMNETS_ERR_HIP;
        }
        return SIMNETS_OK;
    }
    ga.msplit = 1; ga.mg_per_split = (d.M + GM_TM - 1) / GM_TM;
    ga.dx_splits = reinterpret_cast<float *>(ws + w.split);
    ga.wbuf = nullptr; ga.exbuf = nullptr; ga.slots_pad = 0; ga.Mp = 0; ga.Kp = 0;
    ga.pxl = 1;
    ga.cpr = (ga.k.slots + 63) / 64;
    // the row-wise kernels read and write 16 bytes at a time
    auto aligned16 = [](const void *q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; };
    // (of a pooled gradient they read a window row's two values: 8 bytes)
    const bool g_aligned = grad_is_pooled ? (reinterpret_cast<uintptr_t>(output_grad) & 7) == 0 : aligned16(output_grad);
    const bool use_rows = t.mfma && t.rows && aligned16(input) && aligned16(output) && g_aligned &&
                          (!want_input || aligned16(input_grad));
    if (t.mfma) {
        rc = mex_pack_offsets(p, offsets, GM_TM, (d.M + GM_TM - 1) / GM_TM, packed_at, &ga.k, stream, nullptr,
                              !packed_already, pack_normalizes ? norm_at : nullptr, true);
        if (rc)
            return rc;
        if (w.use_factors && !use_rows) {
            rc = launch_factors(p, t, ga, ws + w.factors, s);
            if (rc)
                return rc;
        }
    }
    RowsArgs rg;
    rg.lgW = log2_exact(p.W); rg.Ws = p.W / 2; rg.RS = d.region_size; rg.HW = p.H * p.W; rg.lgHW = log2_exact(rg.HW);
    if (use_rows)
        ga.slots_pad = t.slots_pad;

    if (want_input) {
        MexGradArgs gi = ga;
        gi.overlap = t.overlap ? 1 : 0;
        gi.msplit = t.msplit; gi.mg_per_split = t.mg_per_split;
        gi.pxl = 1;
        gi.cpr = (ga.k.slots + 63) / 64;
        if (!t.factors_input)
            gi.wbuf = gi.exbuf = nullptr;  // (each gradient forms its factors as it does in a call of its own)
        if (!t.overlap && !t.tiles_input) {
            // every element belongs to at most one patch, which stores its gradient; the others keep 0 (patches
            // that tile the input exactly write every element; overlapping ones go through mex_col2im_kernel)
            hipLaunchKernelGGL(mex_fill_zero_kernel, dim3((unsigned)std::min<long long>((n_in + 255) / 256, 65535)),
                               dim3(256), 0, s, input_grad, n_in);
            if (hipGetLastError() != hipSuccess)
                return SIMNETS_ERR_HIP;
        }
        const long long gx = (long long)d.num_regions * gi.cpr;
        if (use_rows) {
            gi.wbuf = gi.exbuf = nullptr;
            gi.msplit = t.rows_msplit; gi.mg_per_split = t.rows_mg_per_split;
            const int kt = 16 * t.rows_ksub, gy = (d.K + kt - 1) / kt;
            if (gy > 65535)
                return SIMNETS_ERR_TOO_LARGE;
            rg.nx = t.slots_pad / 64; rg.ty = gy; rg.tz = t.rows_msplit;
            const long long wgs = (long long)((rg.nx + 7) / 8 * 8) * gy * t.rows_msplit;
            if (wgs > 0x7fffffffLL)
                return SIMNETS_ERR_TOO_LARGE;
            const dim3 grid((unsigned)wgs);
            if (t.rows_ksub == 4)
                hipLaunchKernelGGL(mex_grad_input_rows_kernel<4>, grid, dim3(256), 0, s, gi, rg);
            else if (t.rows_ksub == 2)
                hipLaunchKernelGGL(mex_grad_input_rows_kernel<2>, grid, dim3(256), 0, s, gi, rg);
            else
                hipLaunchKernelGGL(mex_grad_input_rows_kernel<1>, grid, dim3(256), 0, s, gi, rg);
            if (t.rows_msplit > 1) {
                if (hipGetLastError() != hipSuccess)
                    return SIMNETS_ERR_HIP;
                launch_sum_splits(gi.dx_splits, n_in, t.rows_msplit, input_grad, s);
            }
        } else if (t.mfma) {
            const int gy = (d.K + GM_KT - 1) / GM_KT;
            if (gx > 0x7fffffffLL || gy > 65535)
                return SIMNETS_ERR_TOO_LARGE;
            if (gx > 0)
                hipLaunchKernelGGL(mex_grad_input_mfma_kernel, dim3((unsigned)gx, (unsigned)gy, (unsigned)t.msplit),
                                   dim3(256), 0, s, gi);
            if (gx > 0 && t.msplit > 1) {
                if (hipGetLastError() != hipSuccess)
                    return SIMNETS_ERR_HIP;
                launch_sum_splits(gi.dx_splits, n_in, t.msplit, input_grad, s);
            }
        } else {
            const int gy = (d.K + 4 * GX_KT - 1) / (4 * GX_KT);
            if (gx > 0x7fffffffLL || gy > 65535)
                return SIMNETS_ERR_TOO_LARGE;
            if (gx > 0)
                hipLaunchKernelGGL(mex_grad_input_kernel, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, gi);
        }
        if (hipGetLastError() != hipSuccess)
            return SIMNETS_ERR_HIP;
        if (t.overlap) {
            hipLaunchKernelGGL(mex_col2im_kernel, dim3((unsigned)((n_in + 255) / 256)), dim3(256), 0, s, gi.k, gi.col,
                               input_grad, n_in);
            if (hipGetLastError() != hipSuccess)
                return SIMNETS_ERR_HIP;
        }
    }

    if (want_offsets) {
        MexGradArgs go = ga;
        go.dx = nullptr; go.col = nullptr; go.dx_splits = nullptr;
        go.overlap = 0; go.msplit = 1;
        go.pxl = t.pxl;
        go.cpr = t.cpr_offsets;
        if (!t.factors_offsets)
            go.wbuf = go.exbuf = nullptr;
        const long long gx = (long long)d.num_regions * go.cpr;
        if (use_rows) {
            go.wbuf = go.exbuf = nullptr;
            go.pxl = t.rows_pxl;
            go.cpr = t.rows_cpr;
            const int gy = (d.M + 31) / 32, gz = (d.K + 31) / 32;
            if (gy > 65535 || gz > 65535)
                return SIMNETS_ERR_TOO_LARGE;
            rg.nx = t.rows_cpr; rg.ty = gy; rg.tz = gz;
            const long long wgs = (long long)((rg.nx + 7) / 8 * 8) * gy * gz;
            if (wgs > 0x7fffffffLL)
                return SIMNETS_ERR_TOO_LARGE;
            hipLaunchKernelGGL(mex_grad_offsets_rows_kernel, dim3((unsigned)wgs), dim3(256), 0, s, go, rg);
        } else if (t.mfma) {
            const int gy = (d.M + GOM_MT - 1) / GOM_MT, gz = (d.K + GOM_KT - 1) / GOM_KT;
            if (gx > 0x7fffffffLL || gy > 65535 || gz > 65535)
                return SIMNETS_ERR_TOO_LARGE;
            hipLaunchKernelGGL(mex_grad_offsets_mfma_kernel, dim3((unsigned)gx, (unsigned)gy, (unsigned)gz), dim3(256),
                               0, s, go);
        } else {
            const int gy = (d.M + 4 * GO_MT - 1) / (4 * GO_MT);
            const int gz = (d.K + GO_KT - 1) / GO_KT;
            if (gx > 0x7fffffffLL || gy > 65535 || gz > 65535)
                return SIMNETS_ERR_TOO_LARGE;
            hipLaunchKernelGGL(mex_grad_offsets_kernel, dim3((unsigned)gx, (unsigned)gy, (unsigned)gz), dim3(256), 0, s,
                               go);
        }
        if (hipGetLastError() != hipSuccess)
            return SIMNETS_ERR_HIP;
        const long long rows = (long long)d.num_regions * d.M;
        if (rows <= 64 && d.K >= 256 && d.K <= kFinishRowsMaxK) {
            // few long rows: a workgroup per row
            hipLaunchKernelGGL(mex_grad_offsets_finish_wide_rows_kernel, dim3((unsigned)rows), dim3(256), 0, s, go.partial,
                               n_off, go.cpr, d.K, p.normalize_offsets ? go.off : nullptr, offsets_grad);
            return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
        }
        if (d.K <= kFinishRowsMaxK && (rows + 3) / 4 <= 0x7fffffffLL) {
            // short rows: the sum over the pixel chunks and the chain rule through the normalisation in one launch
            hipLaunchKernelGGL(mex_grad_offsets_finish_rows_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s,
                               go.partial, n_off, go.cpr, rows, d.K, p.normalize_offsets ? go.off : nullptr,
                               offsets_grad);
            return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
        }
        hipLaunchKernelGGL(mex_grad_offsets_finish_kernel,
                           dim3((unsigned)std::min<long long>((n_off + 31) / 32, 65535)), dim3(256), 0, s, go.partial,
                           n_off, go.cpr, offsets_grad);
        if (hipGetLastError() != hipSuccess)
            return SIMNETS_ERR_HIP;
        if (p.normalize_offsets) {
            hipLaunchKernelGGL(mex_normalize_rows_backward_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s,
                               go.off, rows, d.K, offsets_grad);
            if (hipGetLastError() != hipSuccess)
                return SIMNETS_ERR_HIP;
        }
    }
    return SIMNETS_OK;
}

int mex_grad_input(const MexPlan &p, const float *input, const float *offsets, const float *output,
                   const float *output_grad, float *input_grad, void *workspace, size_t workspace_bytes, void *stream)
{
    return mex_grads(p, input, offsets, output, output_grad, input_grad, nullptr, workspace, workspace_bytes, stream);
}

int mex_grad_offsets(const MexPlan &p, const float *input, const float *offsets, const float *output,
                     const float *output_grad, float *offsets_grad, void *workspace, size_t workspace_bytes,
                     void *stream)
{
    return mex_grads(p, input, offsets, output, output_grad, nullptr, offsets_grad, workspace, workspace_bytes, stream);
}

}  // namespace simnets
