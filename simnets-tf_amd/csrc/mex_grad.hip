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
//   d patch(px)[k]  = sum_m e(px, m, k)          (then scattered to the input element the patch element is)
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
    float *dx;             // input gradient
    float *partial;        // offsets gradient partial sums [chunk][R][M][K]
    int overlap;           // patches overlap: the scatter must add atomically
    int cpr;               // pixel chunks per region
    int pxl;               // pixel slots per lane (offsets gradient)
};

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
    return ok ? a.in[(size_t)px.b * a.C * a.H * a.W + o] : a.oob;
}

__device__ __forceinline__ float mex_term(float x_plus_off, float out, float g, float c1, float c0, bool finite)
{
    if (finite)
        return g * __builtin_amdgcn_exp2f(__builtin_fmaf(x_plus_off - out, c1, c0));
    return x_plus_off == out ? g : 0.0f;
}

constexpr int GX_KT = 8;   // patch elements per lane (input gradient)

// grid.x: (region, pixel chunk of 64 slots); grid.y: tile of 4*GX_KT patch elements (one GX_KT per wave)
__global__ __launch_bounds__(256) void mex_grad_input_kernel(const MexGradArgs ga)
{
    const MexKernelArgs &a = ga.k;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = blockIdx.x / ga.cpr;
    const int chunk = blockIdx.x - r * ga.cpr;
    const int k0 = (blockIdx.y * 4 + wave) * GX_KT;
    if (k0 >= a.K)
        return;
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
    const float *gp = ga.g + (size_t)px.b * a.M * plane + (valid ? px.out_off : 0);
    const float *op = ga.out + (size_t)px.b * a.M * plane + (valid ? px.out_off : 0);
    const float SIMNETS_CONST_AS *off = (const float SIMNETS_CONST_AS *)(ga.off) + (size_t)r * a.M * a.K + k0;
    const bool finite = a.finite_eps != 0;
    for (int m = 0; m < a.M; ++m) {
        const float g = valid ? gp[(size_t)m * plane] : 0.0f;
        const float o = op[(size_t)m * plane];
#pragma unroll
        for (int j = 0; j < GX_KT; ++j) {
            const float of = (k0 + j < a.K) ? off[(size_t)m * a.K + j] : 0.0f;
            acc[j] += mex_term(xk[j] + of, o, g, a.c1, a.c0, finite);
        }
    }
    if (!valid)
        return;
    float *dimg = ga.dx + (size_t)px.b * a.C * a.H * a.W;
#pragma unroll
    for (int j = 0; j < GX_KT; ++j) {
        if (io[j] < 0)
            continue;
        if (ga.overlap)
            unsafeAtomicAdd(dimg + io[j], acc[j]);
        else
            dimg[io[j]] = acc[j];
    }
}

constexpr int GO_MT = 4, GO_KT = 8;  // instances x patch elements per lane (offsets gradient)

// grid.x: (region, pixel chunk of 64*pxl slots); grid.y: tile of 4*GO_MT instances (one GO_MT per wave);
// grid.z: tile of GO_KT patch elements
__global__ __launch_bounds__(256) void mex_grad_offsets_kernel(const MexGradArgs ga)
{
    const MexKernelArgs &a = ga.k;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int r = blockIdx.x / ga.cpr;
    const int chunk = blockIdx.x - r * ga.cpr;
    const int m0 = (blockIdx.y * 4 + wave) * GO_MT;
    const int k0 = blockIdx.z * GO_KT;
    if (m0 >= a.M)
        return;

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
        const float *gp = ga.g + (size_t)px.b * a.M * plane + (valid ? px.out_off : 0);
        const float *op = ga.out + (size_t)px.b * a.M * plane + (valid ? px.out_off : 0);
#pragma unroll
        for (int i = 0; i < GO_MT; ++i) {
            const bool mok = valid && m0 + i < a.M;
            const float g = mok ? gp[(size_t)(m0 + i) * plane] : 0.0f;
            const float o = mok ? op[(size_t)(m0 + i) * plane] : 0.0f;
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

// dOff[r,m,k] = sum over pixel chunks, in chunk order
__global__ void mex_grad_offsets_finish_kernel(const float *__restrict__ partial, long long n, int chunks,
                                               float *__restrict__ doff)
{
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) {
        float s = 0.0f;
        for (int c = 0; c < chunks; ++c)
            s += partial[(size_t)c * n + i];
        doff[i] = s;
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
        sum += expf(s[k] - mxv);
    for (int d = 32; d > 0; d >>= 1)
        sum += __shfl_xor(sum, d, 64);
    const float lse = logf(sum) + mxv;
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

__global__ void mex_fill_zero_kernel(float *__restrict__ p, long long n)
{
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x)
        p[i] = 0.0f;
}

struct MexGradTiling {
    int pxl, cpr_offsets;
    size_t norm_bytes, partial_bytes;
};

MexGradTiling mex_grad_tiling(const MexPlan &p)
{
    const simnets_mex_dims &d = p.d;
    MexGradTiling t;
    const long long slots = (long long)p.B * d.region_size;
    const long long mk = (long long)((d.M + GO_MT - 1) / GO_MT) * ((d.K + GO_KT - 1) / GO_KT);
    auto waves = [&](int pxl) { return d.num_regions * ((slots + 64LL * pxl - 1) / (64LL * pxl)) * mk; };
    t.pxl = 16;
    while (t.pxl > 1 && waves(t.pxl) < 4096)
        t.pxl >>= 1;
    t.cpr_offsets = (int)((slots + 64LL * t.pxl - 1) / (64LL * t.pxl));
    const size_t rmk = (size_t)d.num_regions * d.M * d.K * sizeof(float);
    t.norm_bytes = p.normalize_offsets ? align_up(rmk, 256) : 0;
    t.partial_bytes = align_up(rmk * t.cpr_offsets, 256);
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

}  // namespace

size_t mex_grad_input_workspace_bytes(const MexPlan &p) { return mex_grad_tiling(p).norm_bytes; }

size_t mex_grad_offsets_workspace_bytes(const MexPlan &p)
{
    const MexGradTiling t = mex_grad_tiling(p);
    return t.norm_bytes + t.partial_bytes;
}

int mex_grad_input(const MexPlan &p, const float *input, const float *offsets, const float *output,
                          const float *output_grad, float *input_grad, void *workspace, size_t workspace_bytes,
                          void *stream)
{
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (workspace_bytes < mex_grad_input_workspace_bytes(p))
        return SIMNETS_ERR_WORKSPACE;
    const simnets_mex_dims &d = p.d;
    MexGradArgs ga;
    ga.k = mex_kernel_args(p);
    ga.k.in = input;
    int rc = prepare_offsets(p, offsets, workspace, s, &ga.off);
    if (rc)
        return rc;
    ga.out = output; ga.g = output_grad; ga.dx = input_grad; ga.partial = nullptr;
    ga.overlap = (d.block_c > d.stride_c && d.channels_out > 1) || (d.block_h > d.stride_h && d.height_out > 1) ||
                 (d.block_w > d.stride_w && d.width_out > 1);
    ga.pxl = 1;
    ga.cpr = (ga.k.slots + 63) / 64;

    // elements no patch covers keep gradient 0; overlapping patches add into it
    const long long n_in = (long long)p.B * p.C * p.H * p.W;
    hipLaunchKernelGGL(mex_fill_zero_kernel, dim3((unsigned)std::min<long long>((n_in + 255) / 256, 65535)), dim3(256),
                       0, s, input_grad, n_in);
    if (hipGetLastError() != hipSuccess)
        return SIMNETS_ERR_HIP;
    const long long gx = (long long)d.num_regions * ga.cpr;
    const int gy = (d.K + 4 * GX_KT - 1) / (4 * GX_KT);
    if (gx > 0x7fffffffLL || gy > 65535)
        return SIMNETS_ERR_TOO_LARGE;
    hipLaunchKernelGGL(mex_grad_input_kernel, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, s, ga);
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

int mex_grad_offsets(const MexPlan &p, const float *input, const float *offsets, const float *output,
                            const float *output_grad, float *offsets_grad, void *workspace, size_t workspace_bytes,
                            void *stream)
{
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (workspace_bytes < mex_grad_offsets_workspace_bytes(p))
        return SIMNETS_ERR_WORKSPACE;
    const simnets_mex_dims &d = p.d;
    if (p.B == 0) {  // an empty batch has a zero gradient
        const long long n = (long long)d.num_regions * d.M * d.K;
        hipLaunchKernelGGL(mex_fill_zero_kernel, dim3((unsigned)std::min<long long>((n + 255) / 256, 65535)), dim3(256),
                           0, s, offsets_grad, n);
        return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
    }
    const MexGradTiling t = mex_grad_tiling(p);
    MexGradArgs ga;
    ga.k = mex_kernel_args(p);
    ga.k.in = input;
    int rc = prepare_offsets(p, offsets, workspace, s, &ga.off);
    if (rc)
        return rc;
    ga.out = output; ga.g = output_grad; ga.dx = nullptr;
    ga.partial = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + t.norm_bytes);
    ga.overlap = 0;
    ga.pxl = t.pxl;
    ga.cpr = t.cpr_offsets;

    const long long gx = (long long)d.num_regions * ga.cpr;
    const int gy = (d.M + 4 * GO_MT - 1) / (4 * GO_MT);
    const int gz = (d.K + GO_KT - 1) / GO_KT;
    if (gx > 0x7fffffffLL || gy > 65535 || gz > 65535)
        return SIMNETS_ERR_TOO_LARGE;
    hipLaunchKernelGGL(mex_grad_offsets_kernel, dim3((unsigned)gx, (unsigned)gy, (unsigned)gz), dim3(256), 0, s, ga);
    if (hipGetLastError() != hipSuccess)
        return SIMNETS_ERR_HIP;
    const long long n = (long long)d.num_regions * d.M * d.K;
    hipLaunchKernelGGL(mex_grad_offsets_finish_kernel, dim3((unsigned)std::min<long long>((n + 255) / 256, 65535)),
                       dim3(256), 0, s, ga.partial, n, ga.cpr, offsets_grad);
    if (hipGetLastError() != hipSuccess)
        return SIMNETS_ERR_HIP;
    if (p.normalize_offsets) {
        const long long rows = (long long)d.num_regions * d.M;
        hipLaunchKernelGGL(mex_normalize_rows_backward_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, ga.off,
                           rows, d.K, offsets_grad);
        if (hipGetLastError() != hipSuccess)
            return SIMNETS_ERR_HIP;
    }
    return SIMNETS_OK;
}

}  // namespace simnets
