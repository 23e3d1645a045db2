// MEX forward (gfx950): out = (1/eps) * log( [1/K] * sum_k exp(eps * (patch_k + offset_k)) ).
//
// Replaces, for the whole batch in one launch, the reference's per-image sequence
// (src/kernels/mex_kernel_gpu.cu:60-159): offsets copy, im2col_3d_gpu_kernel
// (src/utils/im2col.cu:546-585), split_patches_kernel forward (include/utils/ggemm.cuh:660-708),
// ggemm_kernel max pass and ggemm_readc_kernel exp/sum/log pass (mex_kernel_gpu.cu:12-39),
// split_patches_kernel reverse.
//
// Work split
//   * output pixels are enumerated region-major: slot s of region r is image s / region_size,
//     position s % region_size inside the region (the order split_patches lays them out in,
//     include/utils/mex_utils.hpp:69-116).  A wave takes 64 consecutive slots of ONE region, so
//     the offsets it needs, offsets[r, m, k], are the same for all its lanes and are read with
//     scalar loads into SGPRs; nothing is regrouped in memory, each lane maps its slot straight
//     to the (c, h, w) it belongs to for either region flavour (contiguous "shared" tiles or
//     interleaved "unshared" ones).
//   * a lane gathers its patch element k from the input with the im2col_3d index rule (out of
//     image -> blocks_out_of_bounds_value) and combines it with MTX instances at once;
//   * two sweeps over k like the reference (max, then exp-sum relative to the max), with the
//     2*MTX running values in VGPRs; exp is v_exp_f32 on a pre-scaled argument.
//   The four waves of a workgroup share the pixels and split the instances, so the second to
//   fourth gather of an element hit L1.
#include <hip/hip_runtime.h>

#include <cmath>

#include "internal.h"

namespace simnets {

#define SIMNETS_CONST_AS __attribute__((address_space(4)))

namespace {

constexpr int MTX = 16;  // instances per wave

struct MexKernelArgs {
    const float *in;
    float *out;
    const float *offp;  // [R][mtile][K][MTX]
    int B, C, H, W;
    int Co, Ho, Wo;
    int bc, bh, bw, sc, sh, sw, pc, ph, pw;
    int Cg, Hg, Wg;     // offsets_c/h/w: number of regions along each axis
    int Cs, Hs, Ws;     // shared_region_c/h/w: extent of a region along each axis
    int unshared;
    int RS;             // region_size
    int slots;          // B * RS
    int cpr;            // 64-slot chunks per region
    int M, K, n_mtiles;
    float c1;           // eps * log2(e)
    float c0;           // (softmax ? 0 : -log K) * log2(e)
    float eps;
    int finite_eps;
    float oob;
};

template <bool NEG, bool CHECK>
__global__ __launch_bounds__(256) void mex_fwd_kernel(const MexKernelArgs a)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int mtile = blockIdx.y * 4 + wave;
    if (mtile >= a.n_mtiles)
        return;
    const int r = blockIdx.x / a.cpr;
    const int chunk = blockIdx.x - r * a.cpr;

    // region coordinates: r = (c_g * Hg + h_g) * Wg + w_g
    const int w_g = r % a.Wg;
    const int h_g = (r / a.Wg) % a.Hg;
    const int c_g = r / (a.Wg * a.Hg);

    const int slot = chunk * 64 + lane;
    bool valid = slot < a.slots;
    const int sl = valid ? slot : 0;
    const int b = sl / a.RS;
    const int q = sl - b * a.RS;
    const int i = q % a.Ws;
    const int j = (q / a.Ws) % a.Hs;
    const int l = q / (a.Ws * a.Hs);
    int c, h, w;
    if (a.unshared) {
        c = c_g + l * a.Cg; h = h_g + j * a.Hg; w = w_g + i * a.Wg;
    } else {
        c = c_g * a.Cs + l; h = h_g * a.Hs + j; w = w_g * a.Ws + i;
    }
    valid = valid && c < a.Co && h < a.Ho && w < a.Wo;
    if (!valid) {
        c = 0; h = 0; w = 0;
    }
    const int ci0 = c * a.sc - a.pc, hi0 = h * a.sh - a.ph, wi0 = w * a.sw - a.pw;
    const float *img = a.in + (size_t)(valid ? b : 0) * a.C * a.H * a.W;
    const float *base = img + ((ptrdiff_t)ci0 * a.H + hi0) * a.W + wi0;  // only dereferenced in range

    const float SIMNETS_CONST_AS *offp =
        (const float SIMNETS_CONST_AS *)(a.offp) + ((size_t)r * a.n_mtiles + mtile) * a.K * MTX;

    float mx[MTX];
#pragma unroll
    for (int m = 0; m < MTX; ++m)
        mx[m] = NEG ? INFINITY : -INFINITY;

    auto gather = [&](int dc, int dh, int dw) -> float {
        if (CHECK) {
            const int ci = ci0 + dc, hi = hi0 + dh, wi = wi0 + dw;
            if (ci >= 0 && ci < a.C && hi >= 0 && hi < a.H && wi >= 0 && wi < a.W)
                return base[((ptrdiff_t)dc * a.H + dh) * a.W + dw];
            return a.oob;
        }
        return base[((ptrdiff_t)dc * a.H + dh) * a.W + dw];
    };

    // ---- sweep 1: running max (min for negative epsilon) of patch + offset ----
    {
        const float SIMNETS_CONST_AS *op = offp;
        for (int dc = 0; dc < a.bc; ++dc)
            for (int dh = 0; dh < a.bh; ++dh)
                for (int dw = 0; dw < a.bw; ++dw) {
                    const float x = gather(dc, dh, dw);
#pragma unroll
                    for (int m = 0; m < MTX; ++m) {
                        const float v = x + op[m];
                        mx[m] = NEG ? __builtin_fminf(mx[m], v) : __builtin_fmaxf(mx[m], v);
                    }
                    op += MTX;
                }
    }
    float res[MTX];
    if (a.finite_eps) {
        // ---- sweep 2: sum of exp(eps * (v - max) + ey), evaluated as exp2 of the scaled argument ----
        float s[MTX];
#pragma unroll
        for (int m = 0; m < MTX; ++m)
            s[m] = 0.0f;
        const float SIMNETS_CONST_AS *op = offp;
        for (int dc = 0; dc < a.bc; ++dc)
            for (int dh = 0; dh < a.bh; ++dh)
                for (int dw = 0; dw < a.bw; ++dw) {
                    const float x = gather(dc, dh, dw);
#pragma unroll
                    for (int m = 0; m < MTX; ++m) {
                        const float v = x + op[m];
                        s[m] += __builtin_amdgcn_exp2f(__builtin_fmaf(v - mx[m], a.c1, a.c0));
                    }
                    op += MTX;
                }
#pragma unroll
        for (int m = 0; m < MTX; ++m)
            res[m] = mx[m] + logf(s[m]) / a.eps;
    } else {
#pragma unroll
        for (int m = 0; m < MTX; ++m)
            res[m] = mx[m];
    }
    if (!valid)
        return;
    // output channel = instance * channels_out + c  (src/kernels/mex_kernel_cpu.cpp:113-115)
    const size_t plane = (size_t)a.Ho * a.Wo;
    float *o = a.out + ((size_t)b * a.M * a.Co + c) * plane + (size_t)h * a.Wo + w;
#pragma unroll
    for (int m = 0; m < MTX; ++m) {
        const int mm = mtile * MTX + m;
        if (mm < a.M)
            o[(size_t)mm * a.Co * plane] = res[m];
    }
}

// One wave per (region, instance) row of the offsets: optional logsumexp normalisation
// (python/simnets/keras.py:155-160), then the row is scattered into the k-major packed layout.
__global__ __launch_bounds__(256) void mex_pack_offsets_kernel(const float *__restrict__ offsets, int R, int M, int K,
                                                              int n_mtiles, int normalize, float *__restrict__ offp)
{
    const int lane = threadIdx.x & 63;
    const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    const long long rows = (long long)R * n_mtiles * MTX;
    if (row >= rows)
        return;
    const int mi = (int)(row % MTX);
    const long long t = row / MTX;
    const int mtile = (int)(t % n_mtiles);
    const int r = (int)(t / n_mtiles);
    const int m = mtile * MTX + mi;
    float *dst = offp + ((size_t)r * n_mtiles + mtile) * K * MTX + mi;
    if (m >= M) {
        for (int k = lane; k < K; k += 64)
            dst[(size_t)k * MTX] = 0.0f;
        return;
    }
    const float *src = offsets + ((size_t)r * M + m) * K;
    float lse = 0.0f;
    if (normalize) {
        float mxv = -INFINITY;
        for (int k = lane; k < K; k += 64)
            mxv = fmaxf(mxv, src[k]);
        for (int d = 32; d > 0; d >>= 1)
            mxv = fmaxf(mxv, __shfl_xor(mxv, d, 64));
        if (!(fabsf(mxv) < INFINITY))
            mxv = 0.0f;
        float sum = 0.0f;
        for (int k = lane; k < K; k += 64)
            sum += expf(src[k] - mxv);
        for (int d = 32; d > 0; d >>= 1)
            sum += __shfl_xor(sum, d, 64);
        lse = logf(sum) + mxv;
    }
    for (int k = lane; k < K; k += 64)
        dst[(size_t)k * MTX] = src[k] - lse;
}

}  // namespace

size_t mex_workspace_bytes(const MexPlan &p)
{
    const size_t n_mtiles = (p.d.M + MTX - 1) / MTX;
    return align_up(((size_t)p.d.num_regions * n_mtiles * p.d.K + 1) * MTX * sizeof(float), 256);
}

int mex_launch(const MexPlan &p, const float *input, const float *offsets, float *output, void *workspace,
               size_t workspace_bytes, void *stream)
{
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const simnets_mex_dims &d = p.d;
    if (workspace_bytes < mex_workspace_bytes(p))
        return SIMNETS_ERR_WORKSPACE;
    const int n_mtiles = (d.M + MTX - 1) / MTX;
    float *offp = reinterpret_cast<float *>(workspace);

    const long long rows = (long long)d.num_regions * n_mtiles * MTX;
    hipLaunchKernelGGL(mex_pack_offsets_kernel, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, offsets,
                       d.num_regions, d.M, d.K, n_mtiles, p.normalize_offsets, offp);
    if (hipGetLastError() != hipSuccess)
        return SIMNETS_ERR_HIP;

    MexKernelArgs a;
    a.in = input; a.out = output; a.offp = offp;
    a.B = p.B; a.C = p.C; a.H = p.H; a.W = p.W;
    a.Co = d.channels_out; a.Ho = d.height_out; a.Wo = d.width_out;
    a.bc = d.block_c; a.bh = d.block_h; a.bw = d.block_w;
    a.sc = d.stride_c; a.sh = d.stride_h; a.sw = d.stride_w;
    a.pc = d.pad_c; a.ph = d.pad_h; a.pw = d.pad_w;
    a.Cg = d.offsets_c; a.Hg = d.offsets_h; a.Wg = d.offsets_w;
    a.Cs = d.shared_region_c; a.Hs = d.shared_region_h; a.Ws = d.shared_region_w;
    a.unshared = p.use_unshared;
    a.RS = d.region_size;
    a.slots = p.B * d.region_size;
    a.cpr = (a.slots + 63) / 64;
    a.M = d.M; a.K = d.K; a.n_mtiles = n_mtiles;
    const double log2e = 1.4426950408889634;
    a.finite_eps = std::isfinite(p.epsilon);
    a.eps = p.epsilon;
    a.c1 = a.finite_eps ? (float)((double)p.epsilon * log2e) : 0.0f;
    // ey = softmax ? 0 : (float)-log(K)   (src/kernels/mex_kernel_cpu.cpp:36)
    const float ey = p.softmax_mode ? 0.0f : (float)-std::log((double)d.K);
    a.c0 = (float)((double)ey * log2e);
    a.oob = p.oob;

    // bounds checks are needed unless every patch lies inside the image
    const bool inside = d.pad_c == 0 && d.pad_h == 0 && d.pad_w == 0 &&
                        (d.channels_out - 1) * d.stride_c + d.block_c <= p.C &&
                        (d.height_out - 1) * d.stride_h + d.block_h <= p.H &&
                        (d.width_out - 1) * d.stride_w + d.block_w <= p.W;
    const long long gx = (long long)d.num_regions * a.cpr;
    if (gx > 0x7fffffffLL)
        return SIMNETS_ERR_TOO_LARGE;
    dim3 grid((unsigned)gx, (unsigned)((n_mtiles + 3) / 4));
    const bool neg = p.epsilon < 0;
    if (neg && inside)
        hipLaunchKernelGGL((mex_fwd_kernel<true, false>), grid, dim3(256), 0, s, a);
    else if (neg)
        hipLaunchKernelGGL((mex_fwd_kernel<true, true>), grid, dim3(256), 0, s, a);
    else if (inside)
        hipLaunchKernelGGL((mex_fwd_kernel<false, false>), grid, dim3(256), 0, s, a);
    else
        hipLaunchKernelGGL((mex_fwd_kernel<false, true>), grid, dim3(256), 0, s, a);
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

namespace {
__global__ void sum_pool_kernel(const float *__restrict__ in, float *__restrict__ out, long long total, int H, int W,
                                int Ho, int Wo, int ph, int pw)
{
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
         idx += (long long)gridDim.x * blockDim.x) {
        const int wo = (int)(idx % Wo);
        const long long t = idx / Wo;
        const int ho = (int)(t % Ho);
        const long long bc = t / Ho;
        const float *src = in + (bc * H + (long long)ho * ph) * W + (long long)wo * pw;
        float acc = 0.0f;
        for (int i = 0; i < ph; ++i)
            for (int j = 0; j < pw; ++j)
                acc += src[(long long)i * W + j];
        out[idx] = acc;
    }
}
}  // namespace

int sum_pool_launch(int B, int C, int H, int W, int ph, int pw, const float *input, float *output, void *stream)
{
    const int Ho = H / ph, Wo = W / pw;
    const long long total = (long long)B * C * Ho * Wo;
    if (total == 0)
        return SIMNETS_OK;
    const int blocks = (int)std::min<long long>((total + 255) / 256, 65535);
    hipLaunchKernelGGL(sum_pool_kernel, dim3(blocks), dim3(256), 0, reinterpret_cast<hipStream_t>(stream), input,
                       output, total, H, W, Ho, Wo, ph, pw);
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

}  // namespace simnets
