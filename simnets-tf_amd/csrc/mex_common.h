// Argument block and pixel enumeration shared by the MEX forward and backward kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cmath>

#include "fast_div.h"
#include "internal.h"

namespace simnets {

struct MexKernelArgs {
    const float *in;
    float *out;
    const float *offp;  // [R][mgroup][K][TM]  offsets * scale
    const float *offe;  // [R][mgroup][K][TM]  exp2(offsets * scale - row maximum)   (finite epsilon only)
    const float *omax;  // [R][mgroup][TM]     row maximum of offsets * scale
    const float *orng;  // [R][mgroup][TM]     row maximum - row minimum of offsets * scale
    const int4 *ktab;   // [K] patch element k -> {offset (dc*H + dh)*W + dw inside an image, dc, dh, dw}
    int B, C, H, W;
    int Co, Ho, Wo;
    int bc, bh, bw, sc, sh, sw, pc, ph, pw;
    int Cg, Hg, Wg;     // offsets_c/h/w: number of regions along each axis
    int Cs, Hs, Ws;     // shared_region_c/h/w: extent of a region along each axis
    int unshared;
    int R;              // num_regions
    int RS;             // region_size
    FastDiv dRS, dWs, dWsHs, dWg, dWgHg;  // divisions of locate()
    FastDiv dSuper;     // by 8 * R: workgroup numbering of the forward kernel
    int slots;          // B * RS
    int cpr;            // pixel chunks (64*PX slots) per region
    int M, K, n_mgroups;
    float c1;           // eps * log2(e)
    float scale;        // what the tiled kernel multiplies patch values and offsets by: c1 for finite eps, else 1
    float c0;           // (softmax ? 0 : -log K) * log2(e)
    float ln2_over_eps; // log(2) / eps
    int finite_eps;
    float inf_sign;     // infinite eps: +1 (maximum) or -1 (minimum), else 0
    int kgather;        // tiled kernel: gather patch elements with lanes along k (pixels of a chunk lie an image apart)
    float oob;
};

// The forward kernels' product form sum_k exp2(x_k - max x) * exp2(o_k - max o): its largest term is at least
// exp2(-range of the row's scaled offsets) (take k where the patch peaks) and at least exp2(-range of the pixel's scaled
// patch) (take k where the offsets peak).  While one of the two ranges is at most this many exponents of two the sum
// stays far inside the normal range and the terms that underflow lie below its last bit.  Every forward kernel
// decides on the offsets' ranges first (known from the pack) and, in a workgroup that has a wide but finite row, on
// its pixels' patch ranges: the panel and the wave-per-pixel kernel hold the whole patch anyway, the fused and the
// tiled kernel sweep the patches once more for it (not the tiled kernel's k-oriented gather, which keeps the first rule).
constexpr float kProductRange = 90.0f;

struct PixelRef {
    const float *base;  // &input[b][c*sc-pc][h*sh-ph][w*sw-pw] (only dereferenced inside the image)
    int ci0, hi0, wi0;
    int out_off;        // offset of out[b][c][h][w] within image b's output, -1 if the slot is empty
    int b;
};

// slot of region r -> pixel; empty slots (beyond the batch or past a ragged region edge) get
// out_off = -1 and read pixel (0,0,0) of image 0.
__device__ __forceinline__ PixelRef locate(const MexKernelArgs &a, int r, int slot)
{
    const int rw = (int)fast_div((unsigned)r, a.dWg);
    const int w_g = r - rw * a.Wg;
    const int c_g = (int)fast_div((unsigned)r, a.dWgHg);
    const int h_g = rw - c_g * a.Hg;
    bool valid = slot < a.slots;
    const int sl = valid ? slot : 0;
    const int b = (int)fast_div((unsigned)sl, a.dRS);
    const int q = sl - b * a.RS;
    const int qw = (int)fast_div((unsigned)q, a.dWs);
    const int i = q - qw * a.Ws;
    const int l = (int)fast_div((unsigned)q, a.dWsHs);
    const int j = qw - l * a.Hs;
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
    PixelRef p;
    p.b = valid ? b : 0;
    p.ci0 = c * a.sc - a.pc; p.hi0 = h * a.sh - a.ph; p.wi0 = w * a.sw - a.pw;
    p.base = a.in + (size_t)p.b * a.C * a.H * a.W + ((ptrdiff_t)p.ci0 * a.H + p.hi0) * a.W + p.wi0;
    p.out_off = valid ? (c * a.Ho + h) * a.Wo + w : -1;
    return p;
}

// Everything of the argument block that follows from the plan alone (pointers and tiling are the
// caller's).
inline MexKernelArgs mex_kernel_args(const MexPlan &p)
{
    const simnets_mex_dims &d = p.d;
    MexKernelArgs a;
    a.in = nullptr; a.out = nullptr; a.offp = nullptr; a.offe = nullptr; a.omax = nullptr; a.orng = nullptr; a.ktab = nullptr;
    a.B = p.B; a.C = p.C; a.H = p.H; a.W = p.W;
    a.Co = d.channels_out; a.Ho = d.height_out; a.Wo = d.width_out;
    a.bc = d.block_c; a.bh = d.block_h; a.bw = d.block_w;
    a.sc = d.stride_c; a.sh = d.stride_h; a.sw = d.stride_w;
    a.pc = d.pad_c; a.ph = d.pad_h; a.pw = d.pad_w;
    a.Cg = d.offsets_c; a.Hg = d.offsets_h; a.Wg = d.offsets_w;
    a.Cs = d.shared_region_c; a.Hs = d.shared_region_h; a.Ws = d.shared_region_w;
    a.unshared = p.use_unshared;
    a.R = d.num_regions;
    a.RS = d.region_size;
    a.slots = p.B * d.region_size;
    a.dRS = make_fast_div((unsigned)a.RS); a.dWs = make_fast_div((unsigned)a.Ws);
    a.dWsHs = make_fast_div((unsigned)(a.Ws * a.Hs));
    a.dWg = make_fast_div((unsigned)a.Wg); a.dWgHg = make_fast_div((unsigned)(a.Wg * a.Hg));
    a.dSuper = make_fast_div(8u * (unsigned)a.R);
    a.cpr = 0;
    a.M = d.M; a.K = d.K; a.n_mgroups = 0;
    const double log2e = 1.4426950408889634;
    a.finite_eps = std::isfinite(p.epsilon);
    a.inf_sign = a.finite_eps ? 0.0f : (p.epsilon < 0 ? -1.0f : 1.0f);
    a.c1 = a.finite_eps ? (float)((double)p.epsilon * log2e) : 0.0f;
    a.scale = a.finite_eps ? a.c1 : 1.0f;
    a.ln2_over_eps = a.finite_eps ? (float)(0.6931471805599453 / (double)p.epsilon) : 0.0f;
    // ey = softmax ? 0 : (float)-log(K)   (src/kernels/mex_kernel_cpu.cpp:36)
    const float ey = p.softmax_mode ? 0.0f : (float)-std::log((double)d.K);
    a.c0 = (float)((double)ey * log2e);
    a.oob = p.oob;
    a.kgather = 0;
    return a;
}

// The scaled, normalised offset every packing path stores (and exponentiates relative to its row maximum): kept out of
// the compiler's multiply-add fusion so that the pack kernel and the kernels that pack for themselves agree bit for bit.
__device__ __forceinline__ float mex_scaled_offset(float x, float lse, float scale)
{
#pragma clang fp contract(off)
    return (x - lse) * scale;
}

// The exponent of a packed offset's exponential, 2^(scaled offset - row maximum), from the offsets themselves: the
// difference to the row's extreme element first, then the scale - one rounding at the size of the difference instead of
// two at the size of the offsets (xh: the element whose scaled value is the row maximum).
__device__ __forceinline__ float mex_offset_exponent(float x, float xh, float lse, float scale)
{
#pragma clang fp contract(off)
    return ((x - lse) - (xh - lse)) * scale;
}

// exp(d) for d <= 0 and the row's logsumexp from the sum of such terms, as the packing paths compute them for
// normalize_offsets: one v_exp_f32 / v_log_f32 each (results within about an ulp of the library functions', at a
// tenth of their instructions: a workgroup that packs for itself evaluates 32 of them per thread), in one place so
// that every path rounds alike.  Terms below 2^-126 of the largest come out as 0.
__device__ __forceinline__ float mex_exp_term(float d)
{
#pragma clang fp contract(off)
    return __builtin_amdgcn_exp2f(d * 1.44269504088896341f);
}
__device__ __forceinline__ float mex_lse_of(float sum, float mxv)
{
#pragma clang fp contract(off)
    return __builtin_amdgcn_logf(sum) * 0.693147180559945309f + mxv;
}

// Packs the offsets for the forward kernels (k-major tiles of tm instances per group: scaled values, their
// exponentials relative to the row maximum, row maxima and ranges) and the patch element table into `workspace`
// (mex_packed_bytes), and points the argument block at them.
// `job` (optional): the parameters of a Similarity layer, packed by extra workgroups of the same launch
// (sim_pack_element) for the kernel that evaluates that layer inside the MEX staging: channels in chunks of 32,
// pa[chunk][k % 4][tap][k / 4 % 8] = (template, scaled negative weight), pc likewise.
struct SimPackJob {
    const float *templates, *weights;  // [O][K]
    float *pa, *pc;                    // (O rounded up to 32) * K pairs / values
    int O, K, mode;
    float fudge;
};
size_t mex_packed_bytes(const MexPlan &p, int tm, int n_mgroups);
// A second packed layout written by the same launch: what the gradient kernels read (groups of kGradPackTm instances:
// the exponentials, row maxima and ranges - the scaled values, which those kernels do not take, stay unwritten - and
// the normalised offsets when the layer normalises them), kept by a forward call for the gradient call that
// follows it.  A plan whose grad_pack is set makes the forward's pack launch write it (and say so in `written`; a
// forward that packs inside its own kernel does not).
constexpr int kGradPackTm = 32;
// The gradient kernels' product form builds its exponents from the scaled offsets, `out` and the bound, i.e. from values
// of the size of the offsets: a term's relative error is about the last bit of such a value, 4e-6 at 64 exponents of two
// and 1.5e-5 from 128 on - an order above the reference's, which subtracts `out` from patch + offset (exactly, for the
// terms that matter) before it scales.  A row with a scaled offset beyond this size therefore gets an infinite range in
// the arrays those kernels read, which sends its region to their term-by-term form (the reference's arithmetic).
// Normalised offsets (log-probabilities) get there through their range first.
constexpr float kGradOffsetsSize = 64.0f;
struct MexPackTwin {
    float *offp, *offe, *omax, *orng;
    int4 *ktab;
    int tm, n_mgroups;
};
void mex_grad_pack_layout(const MexPlan &p, void *buffer, MexPackTwin *tw, float **normalized);
// launch = false: the arrays were packed by an earlier call with the same arguments; only the pointers are set.
// normalized_out: if not null, the launch also writes the offsets minus their rows' logsumexp there, [region][M][K]
// (what the gradient kernels' term-by-term path and the chain rule through the normalisation read).
// for_gradients: the ranges written are the gradient kernels' (kGradOffsetsSize), as in the layout a forward call keeps.
int mex_pack_offsets(const MexPlan &p, const float *offsets, int tm, int n_mgroups, void *workspace, MexKernelArgs *a,
                     void *stream, const SimPackJob *job = nullptr, bool launch = true,
                     float *normalized_out = nullptr, bool for_gradients = false);


// Panel form of the tiled forward kernel (csrc/mex_pool.hip) for layers with 2x2 unshared offsets over whole-channel
// patches of 32 (small grids), 64, 128 or 256 channels: mex_panel_geometry says whether a layer has its geometry (its offsets are then
// packed in groups of 64 instances); mex_panel_launch runs it on offsets packed that way, or returns
// SIMNETS_PANEL_NOT_TAKEN without launching anything (input not 16-byte aligned).
constexpr int SIMNETS_PANEL_NOT_TAKEN = 1;
bool mex_panel_geometry(const MexPlan &p);
int mex_panel_launch(const MexPlan &p, const MexKernelArgs &a, const float *input, float *output, void *stream);
// The whole self-packing call of such a layer as ONE launch when its patches are a single chunk (32 channels) and the
// grid is small: every workgroup packs the offsets rows it needs (4 regions x 64 instances, one row per thread) into
// its LDS tile itself, with the pack kernel's arithmetic in the pack kernel's order (bit-identical results).  Returns
// SIMNETS_PANEL_NOT_TAKEN without launching anything when the layer or the pointers do not qualify.
int mex_panel_launch_selfpack(const MexPlan &p, const MexKernelArgs &a, const float *input, const float *offsets,
                              float *output, void *stream);

}  // namespace simnets
