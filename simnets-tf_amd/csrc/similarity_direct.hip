// Similarity forward, direct evaluation on the vector ALU (gfx950).
//
// Replaces, for the whole batch in one launch, what the reference does per image with three
// kernels: interlace_kernel (include/utils/ggemm.cuh:70-87), im2col_3d_gpu_kernel
// (src/utils/im2col.cu:546-585) and ggemm_kernel (include/utils/ggemm.cuh:108-185) with the
// combines of include/utils/similarity_utils.hpp:17-80.
//
// Shape of the computation
//   out[b, m, h, w] = sum_k comb(t[m,k], w[m,k], patch[b,h,w][k]),  k = (c*bh + dh)*bw + dw
// Work split
//   * a lane owns PT consecutive output columns of one output row ("pixel group") and MT
//     output channels: PT*MT accumulators in VGPRs, summed over k in the reference's order;
//   * the MT (template, weight) pairs of a k are the same for all 64 lanes; they come from a packed,
//     k-major copy of the parameters through vector loads with a lane-uniform address, one step
//     ahead, so that the arithmetic reads VGPRs only (SGPR operands halve the VALU issue rate here);
//     the gather fallback fetches them with scalar loads and moves each to a VGPR once;
//   * a workgroup (4 waves) stages the rows of the input image its pixel groups touch, a few
//     channels at a time, into LDS with coalesced loads; out-of-image positions are written as
//     the out_of_bounds_value bit pattern there, so the inner loop has no bounds checks and NaN
//     padding behaves exactly like NaN data.
//   The inner loop is VALU bound: per k and lane PT/2 ds_read2_b32 and 4 global_load_dwordx4 against
//   3*PT*MT VALU ops (L2).
#include <hip/hip_runtime.h>

#include <cmath>

#include "internal.h"
#include "stage.h"
#include "valu_tile.h"
#include "sim_step.h"

namespace simnets {

namespace {

constexpr int kWaves = 4;                 // waves per workgroup
constexpr int kThreads = 64 * kWaves;
constexpr int kLdsBudgetFloats = 16384;   // 64 KiB of input tile per workgroup
constexpr int kStagePos = 6;              // tile elements per thread and channel (a channel's tile holds at most
                                          // kStagePos * kThreads floats; larger geometries use the gather kernel)
constexpr int kStageChan = 6;             // channels whose loads are in flight at once while staging

struct SimKernelArgs {
    const float *in;
    float *out;
    const float *pa;   // [mtile][K][MT][2]  (template, scaled negative weight)
    const float *pc;   // [mtile][K][MT]     per-(m,k) additive constant (normalized modes)
    const int *koff;   // [K + 2] LDS offset of patch element k inside the staged chunk: (c % CC) * TRmax*TC + dh*TC + dw
    int B, C, H, W, O, oh, ow;
    int bh, bw, sh, sw, ph, pw, K;
    int G;             // pixel groups per output row = ceil(ow / PT)
    int gpi;           // pixel groups per image = oh * G
    int tiles;         // workgroup tiles per image
    int nws;           // spatial waves per workgroup (1, 2 or 4); kWaves / nws waves split the templates
    int nws_log2;
    int n_mtiles;      // ceil(O / MT)
    int TC;            // LDS tile row pitch (floats)
    int TRmax;         // LDS rows reserved per channel
    int CC;            // channels staged per chunk
    float oob;
    float norm_const;  // -0.5*K*log(2 pi) for SIM_MODE_L2_NORM, else 0
    int norm_every_iteration;
    int vec_store;     // output rows are 16-byte aligned: store float4
    int fast_stage;    // the channel tile has at most kStagePos * kThreads elements: division-free staging
    // sqrt-weight form only (see sim_guard_fix_kernel)
    const float *templates, *weights;  // the caller's arrays [O][K]
    const float *thr;  // [O] outputs of template m above -thr[m] are recomputed exactly
    int *flags;        // [workgroups * kWaves] set by a wave that wrote such an output
};

// Output positions of a lane: the mapping shared by sim_direct_kernel and sim_guard_fix_kernel.
struct LanePos {
    int b, tile, ws, mtile;
    int g_first, g_last, row_first;
    int h, gw;
    bool wave_active, lane_valid;
};

__device__ __forceinline__ LanePos lane_pos(const SimKernelArgs &a, int wave, int lane)
{
    LanePos q;
    q.b = blockIdx.x / a.tiles;
    q.tile = blockIdx.x - q.b * a.tiles;
    q.ws = wave & (a.nws - 1);                   // which 64 pixel groups of the tile
    const int wm = wave >> a.nws_log2;           // which MT templates
    const int nwm = kWaves >> a.nws_log2;
    q.mtile = blockIdx.y * nwm + wm;
    q.wave_active = q.mtile < a.n_mtiles;
    q.g_first = q.tile * 64 * a.nws;
    q.g_last = min(q.g_first + 64 * a.nws, a.gpi) - 1;
    q.row_first = q.g_first / a.G;
    int g = q.g_first + q.ws * 64 + lane;
    q.lane_valid = g <= q.g_last;
    g = min(g, q.g_last);
    q.h = g / a.G;
    q.gw = g - q.h * a.G;
    return q;
}

// Wave-uniform parameter fetch of the gather fallback: the address is the same in every lane, so these
// become scalar loads (s_load_dwordx8/x16) and the values live in SGPRs.
template <int MODE, int MT>
__device__ __forceinline__ void load_params(float (&pa)[2 * MT], float (&pc)[MT], const float SIMNETS_CONST_AS *ppa,
                                            const float SIMNETS_CONST_AS *ppc)
{
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i)
        pa[i] = ppa[i];
#pragma unroll
    for (int i = 0; i < MT; ++i)
        pc[i] = (MODE == SIM_MODE_L2_NORM || MODE == SIM_MODE_L2_NORM_IGNORE_NAN) ? ppc[i] : 0.0f;
}

// Lane tile of the wide-image variant, and of the narrow one.
#ifndef SIMNETS_BIG_PT
#define SIMNETS_BIG_PT 16
#endif
#ifndef SIMNETS_BIG_MT
#define SIMNETS_BIG_MT 8
#endif
constexpr int kBigPT = SIMNETS_BIG_PT, kBigMT = SIMNETS_BIG_MT;
constexpr int kSmallPT = 4, kSmallMT = 8;
// waves per SIMD the register budget is sized for: 64 accumulators leave room for 4, 128 for 2
constexpr int waves_per_simd(int pt, int mt) { return pt * mt <= 64 ? 4 : 2; }
constexpr int lds_budget_floats(int pt, int mt) { return pt * mt <= 64 ? kLdsBudgetFloats / 2 : kLdsBudgetFloats; }

template <int MODE, int PT, int MT, int SWT>
__global__ __launch_bounds__(kThreads, waves_per_simd(PT, MT)) void sim_direct_kernel(const SimKernelArgs a)
{
    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int sw = SWT > 0 ? SWT : a.sw;

    const LanePos lp = lane_pos(a, wave, lane);
    const int b = lp.b, mtile = lp.mtile, h = lp.h, gw = lp.gw;
    const bool wave_active = lp.wave_active, lane_valid = lp.lane_valid;

    // pixel groups of this workgroup and the input rows they need
    const int row_first = lp.row_first;
    const int nrows = lp.g_last / a.G - row_first + 1;
    const int TR = (nrows - 1) * a.sh + a.bh;
    const int in_row0 = row_first * a.sh - a.ph;
    const int lds_base = (h - row_first) * a.sh * a.TC + gw * PT * sw;

    float acc[MT][PT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int p = 0; p < PT; ++p)
            acc[m][p] = 0.0f;

    // Parameter stream of this wave's templates.  Every lane reads the same address, but through vector
    // loads (the zero below is opaque to the compiler, so the address counts as lane-dependent): the
    // values arrive in VGPRs, which is where the arithmetic wants them (VALU instructions with SGPR
    // operands issue at half rate), at the cost of 4 load instructions per k instead of one scalar load
    // plus 16 moves; they use the vector-memory counter, so waiting for LDS data never waits for them.
    unsigned zero_v;
    asm volatile("v_mov_b32 %0, 0" : "=v"(zero_v));
    constexpr bool HAS_PC = MODE == SIM_MODE_L2_NORM || MODE == SIM_MODE_L2_NORM_IGNORE_NAN;
    const char *pa_base = reinterpret_cast<const char *>(a.pa + (size_t)(wave_active ? mtile : 0) * a.K * MT * 2);
    const char *pc_base = reinterpret_cast<const char *>(a.pc + (size_t)(wave_active ? mtile : 0) * a.K * MT);
    unsigned pa_off = zero_v, pc_off = zero_v;  // byte offsets of the NEXT k
    auto fetch_params = [&](float (&pav)[2 * MT], float (&pcv)[MT]) {
#pragma unroll
        for (int i = 0; i < 2 * MT / 4; ++i) {
            const float4 v = *reinterpret_cast<const float4 *>(pa_base + pa_off + 16 * i);
            pav[4 * i] = v.x; pav[4 * i + 1] = v.y; pav[4 * i + 2] = v.z; pav[4 * i + 3] = v.w;
        }
        pa_off += 2 * MT * sizeof(float);
        if (HAS_PC) {
#pragma unroll
            for (int i = 0; i < MT / 4; ++i) {
                const float4 v = *reinterpret_cast<const float4 *>(pc_base + pc_off + 16 * i);
                pcv[4 * i] = v.x; pcv[4 * i + 1] = v.y; pcv[4 * i + 2] = v.z; pcv[4 * i + 3] = v.w;
            }
            pc_off += MT * sizeof(float);
        } else {
#pragma unroll
            for (int i = 0; i < MT; ++i)
                pcv[i] = 0.0f;
        }
    };
    const float *img = a.in + (size_t)b * a.C * a.H * a.W;
    const int chan_lds = a.TRmax * a.TC;
    float pa0[2 * MT], pc0[MT], pa1[2 * MT], pc1[MT];
    fetch_params(pa0, pc0);
    TilePositions<kStagePos> tp;
    tp.template init<kThreads>(a.H, a.W, TR, a.TC, in_row0, a.pw);
    // LDS offsets of the patch elements, one scalar load per k, fetched two steps ahead
    const int SIMNETS_CONST_AS *kt = (const int SIMNETS_CONST_AS *)(a.koff);

    for (int ch0 = 0; ch0 < a.C; ch0 += a.CC) {
        const int ccn = min(a.CC, a.C - ch0);
        __syncthreads();
        // ---- stage ccn channels x TR rows x TC columns; out-of-image -> oob ----
        if (a.fast_stage)
            stage_input_tile_fast<kStagePos, kStageChan>(lds, img, a.H, a.W, ch0, ccn, ccn, chan_lds, a.oob, nullptr, tp);
        else  // tiles with more elements per channel than the precomputed positions cover
            stage_input_tile<kThreads, 8>(lds, img, a.H, a.W, ch0, ccn, ccn, TR, a.TC, chan_lds, in_row0, a.pw, a.oob,
                                          nullptr);
        __syncthreads();
        if (!wave_active)
            continue;
        // ---- accumulate over the k of these channels, in k order.  Software pipeline: the pixel
        //      values and the parameters of step k+1 are requested before the arithmetic of step k,
        //      ping-ponging between two register sets (no copies) ----
        const int nk = ccn * a.bh * a.bw;
        int off_next = kt[1];  // offset of step k+1 (the entries behind the last k are 0)
        auto step = [&](const float (&xc)[PT], const float (&pac)[2 * MT], const float (&pcc)[MT], float (&xnx)[PT],
                        float (&panx)[2 * MT], float (&pcnx)[MT]) {
            // everything outstanding on the LDS / scalar counter was issued a whole step ago
            __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int p = 0; p < PT; ++p)
                xnx[p] = lds[lds_base + off_next + p * sw];
            kt += 1;
            off_next = kt[1];
            fetch_params(panx, pcnx);  // one k of slack exists behind the arrays
            __builtin_amdgcn_sched_barrier(0);
            sim_step<MODE, PT, MT, true>(acc, xc, pac, pcc);
            __builtin_amdgcn_sched_barrier(0);
        };
        float x0[PT], x1[PT];
        {
            const int off0 = kt[0];
#pragma unroll
            for (int p = 0; p < PT; ++p)
                x0[p] = lds[lds_base + off0 + p * sw];
        }
        int kk = 0;
        for (; kk + 2 <= nk; kk += 2) {
            step(x0, pa0, pc0, x1, pa1, pc1);
            step(x1, pa1, pc1, x0, pa0, pc0);
        }
        if (kk < nk) {
            step(x0, pa0, pc0, x1, pa1, pc1);
#pragma unroll
            for (int i = 0; i < 2 * MT; ++i)
                pa0[i] = pa1[i];
#pragma unroll
            for (int i = 0; i < MT; ++i)
                pc0[i] = pc1[i];
        }
    }

    if (!wave_active || !lane_valid)
        return;
    // ---- epilogue ----
    int reps = 0;
    if (MODE == SIM_MODE_L2_NORM)
        reps = a.norm_every_iteration ? (a.B - b) : 1;
    const int w0 = gw * PT;
    bool suspect = false;  // sqrt-weight form: an output so close to zero that its rounding error may show
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int mm = mtile * MT + m;
        if (mm >= a.O)
            break;
        float v[PT];
#pragma unroll
        for (int p = 0; p < PT; ++p) {
            v[p] = acc[m][p];
            for (int r = 0; r < reps; ++r)
                v[p] += a.norm_const;
        }
        if (MODE == SIM_MODE_L2_SQRTW) {
            const float thr = a.thr[mm];
#pragma unroll
            for (int p = 0; p < PT; ++p)
                suspect |= w0 + p < a.ow && !(-v[p] >= thr);  // (also catches NaN)
        }
        float *o = a.out + (((size_t)b * a.O + mm) * a.oh + h) * a.ow + w0;
        if (a.vec_store && PT % 4 == 0) {
#pragma unroll
            for (int q = 0; q < PT / 4; ++q)
                if (w0 + 4 * q < a.ow)
                    *reinterpret_cast<float4 *>(o + 4 * q) = make_float4(v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]);
        } else {
#pragma unroll
            for (int p = 0; p < PT; ++p)
                if (w0 + p < a.ow)
                    o[p] = v[p];
        }
    }
    if (MODE == SIM_MODE_L2_SQRTW && suspect)
        a.flags[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * kWaves + wave] = 1;
}

// Second pass of the sqrt-weight form (plain L2 evaluated as -(sqrt(w) t - sqrt(w) x)^2: 2 instead of 3 VALU
// instructions per term).  Its rounding differs from the reference's w (t - x)^2 only inside d = sqrt(w)(t - x):
// |err(d)| <= eps (|sqrt(w) t| + |d|), so by Cauchy-Schwarz the relative error of an output `out` of template m is
// at most 2 eps sqrt(T_m / out) + O(eps) with T_m = sum_k w t^2: below 4e-6 unless out < T_m / 1024.  The main
// kernel flags the waves that wrote such an output (exact matches of a patch and a template, in practice); this
// kernel, launched with the same grid, returns at once for the others and recomputes the flagged waves' small
// outputs with the reference's arithmetic (d = t - x; acc = fma(-w d, d, acc), k ascending: bit-identical to the
// direct kernel).  thr[m] = T_m / 1024, or +inf for a template with a negative or NaN weight (sqrt undefined):
// all outputs of such a template are recomputed.
template <int PT, int MT>
__global__ __launch_bounds__(kThreads) void sim_guard_fix_kernel(const SimKernelArgs a)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (a.flags[((size_t)blockIdx.y * gridDim.x + blockIdx.x) * kWaves + wave] == 0)
        return;
    const LanePos lp = lane_pos(a, wave, lane);
    if (!lp.wave_active || !lp.lane_valid)
        return;
    const int w0 = lp.gw * PT, bhw = a.bh * a.bw;
    const float *img = a.in + (size_t)lp.b * a.C * a.H * a.W;
    for (int m = 0; m < MT; ++m) {
        const int mm = lp.mtile * MT + m;
        if (mm >= a.O)
            break;
        const float thr = a.thr[mm];
        const float *tp = a.templates + (size_t)mm * a.K, *wp = a.weights + (size_t)mm * a.K;
        float *o = a.out + (((size_t)lp.b * a.O + mm) * a.oh + lp.h) * a.ow + w0;
        for (int p = 0; p < PT && w0 + p < a.ow; ++p) {
            if (-o[p] >= thr)
                continue;
            const int hi0 = lp.h * a.sh - a.ph, wi0 = (w0 + p) * a.sw - a.pw;
            float acc = 0.0f;
            for (int k = 0; k < a.K; ++k) {
                const int c = k / bhw, rem = k - c * bhw;
                const int hi = hi0 + rem / a.bw, wi = wi0 + rem % a.bw;
                const bool inside = hi >= 0 && hi < a.H && wi >= 0 && wi < a.W;
                const float x = inside ? img[((size_t)c * a.H + hi) * a.W + wi] : a.oob;
                const float d = tp[k] - x;
                acc = __builtin_fmaf(-wp[k] * d, d, acc);
            }
            o[p] = acc;
        }
    }
}

// Thresholds of the sqrt-weight form (one wave per template) and the cleared flags.
__global__ __launch_bounds__(256) void sim_guard_prep_kernel(const float *__restrict__ templates,
                                                            const float *__restrict__ weights, int O, int K,
                                                            float *__restrict__ thr, int *__restrict__ flags,
                                                            long long n_flags)
{
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n_flags; i += (long long)gridDim.x * 256)
        flags[i] = 0;
    const int lane = threadIdx.x & 63;
    for (int m = blockIdx.x * 4 + (threadIdx.x >> 6); m < O; m += gridDim.x * 4) {
        float t2 = 0.0f;
        bool bad = false;
        for (int k = lane; k < K; k += 64) {
            const float t = templates[(size_t)m * K + k], w = weights[(size_t)m * K + k];
            t2 = __builtin_fmaf(w * t, t, t2);
            bad |= !(w >= 0.0f);
        }
        for (int d = 32; d > 0; d >>= 1)
            t2 += __shfl_xor(t2, d, 64);
        const bool any_bad = __any(bad);
        if (lane == 0)
            thr[m] = (any_bad || !(t2 >= 0.0f)) ? INFINITY : t2 * (1.0f / 1024.0f);
    }
}

// Fallback for geometries whose input rows do not fit the LDS budget: one output pixel per
// lane, patch elements gathered straight from global memory with bounds checks.
template <int MODE, int MT>
__global__ __launch_bounds__(256) void sim_gather_kernel(const SimKernelArgs a)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const long long pix0 = ((long long)blockIdx.x * kWaves + wave) * 64;
    const long long npix = (long long)a.B * a.oh * a.ow;
    if (pix0 >= npix)
        return;
    long long pix = pix0 + lane;
    const bool lane_valid = pix < npix;
    if (!lane_valid)
        pix = npix - 1;
    const int b = (int)(pix / (a.oh * a.ow));
    const int rem = (int)(pix - (long long)b * a.oh * a.ow);
    const int h = rem / a.ow, w = rem - h * a.ow;
    const int mtile = blockIdx.y;
    const float *img = a.in + (size_t)b * a.C * a.H * a.W;
    const float SIMNETS_CONST_AS *pa = (const float SIMNETS_CONST_AS *)(a.pa) + (size_t)mtile * a.K * MT * 2;
    const float SIMNETS_CONST_AS *pc = (const float SIMNETS_CONST_AS *)(a.pc) + (size_t)mtile * a.K * MT;
    float acc[MT][1];
#pragma unroll
    for (int m = 0; m < MT; ++m)
        acc[m][0] = 0.0f;
    for (int c = 0; c < a.C; ++c)
        for (int dh = 0; dh < a.bh; ++dh) {
            const int ih = h * a.sh - a.ph + dh;
            for (int dw = 0; dw < a.bw; ++dw) {
                const int iw = w * a.sw - a.pw + dw;
                float x[1] = {a.oob};
                if (ih >= 0 && ih < a.H && iw >= 0 && iw < a.W)
                    x[0] = img[((size_t)c * a.H + ih) * a.W + iw];
                float pav[2 * MT], pcv[MT];
                load_params<MODE, MT>(pav, pcv, pa, pc);
                sim_step<MODE, 1, MT>(acc, x, pav, pcv);
                pa += 2 * MT;
                pc += MT;
            }
        }
    if (!lane_valid)
        return;
    int reps = 0;
    if (MODE == SIM_MODE_L2_NORM)
        reps = a.norm_every_iteration ? (a.B - b) : 1;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int mm = mtile * MT + m;
        if (mm >= a.O)
            break;
        float v = acc[m][0];
        for (int r = 0; r < reps; ++r)
            v += a.norm_const;
        a.out[(((size_t)b * a.O + mm) * a.oh + h) * a.ow + w] = v;
    }
}

// Packs (template, weight) into the k-major, MT-interleaved layout the parameter loads walk, with
// the sign and the 1/2 of the normalized modes folded into the weight, and precomputes the
// per-(m,k) logarithm term.  Replaces interlace_kernel (include/utils/ggemm.cuh:70-87).
__global__ void sim_pack_params_kernel(const float *__restrict__ templates, const float *__restrict__ weights, int O,
                                       int K, int MT, int n_mtiles, int mode, float fudge, float *__restrict__ pa,
                                       float *__restrict__ pc, int *__restrict__ koff, int taps, int bw, int CC,
                                       int chan_pitch, int TC)
{
    // LDS offset of patch element k inside a staged chunk of CC channels; 0 behind the last k
    for (int k = blockIdx.x * blockDim.x + threadIdx.x; k < K + 2; k += gridDim.x * blockDim.x) {
        int off = 0;
        if (k < K) {
            const int c = k / taps, rem = k - c * taps;
            const int dh = rem / bw, dw = rem - dh * bw;
            off = (c % CC) * chan_pitch + dh * TC + dw;
        }
        koff[k] = off;
    }
    const long long total = (long long)n_mtiles * K * MT;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (long long)gridDim.x * blockDim.x) {
        const int mi = (int)(i % MT);
        const long long r = i / MT;
        const int k = (int)(r % K);
        const int mtile = (int)(r / K);
        const int m = mtile * MT + mi;
        float t = 0.0f, w = 0.0f;
        if (m < O) {
            t = templates[(size_t)m * K + k];
            w = weights[(size_t)m * K + k];
        }
        sim_pack_element(mode, m < O, t, w, fudge, pa[2 * i], pa[2 * i + 1], pc[i]);
    }
}

struct Tiling {
    int PT, MT, nws, G, gpi, tiles, TC, TRmax, CC;
    bool lds_ok;       // the rows of a workgroup's pixel groups fit the LDS tile (else: gather kernel)
    bool fast_stage;   // ... and the division-free staging (at most kStagePos elements per thread and channel)
};

// One candidate: lane tile (PT, MT) with `nws` spatial waves per workgroup.
Tiling try_tiling(const SimPlan &p, int PT, int MT, int nws)
{
    Tiling t;
    t.PT = PT; t.MT = MT; t.nws = nws;
    const int budget = lds_budget_floats(PT, MT);
    t.G = (p.ow + PT - 1) / PT;
    t.gpi = p.oh * t.G;
    t.tiles = (t.gpi + 64 * nws - 1) / (64 * nws);
    t.TC = (t.G * PT - 1) * p.sw + p.bw;
    t.TC |= 1;  // odd pitch spreads rows over LDS banks
    const int max_rows = std::min(p.oh, (64 * nws + t.G - 1) / t.G + 1);
    t.TRmax = (max_rows - 1) * p.sh + p.bh;
    const long long per_chan = 1LL * t.TRmax * t.TC;
    t.lds_ok = per_chan <= budget;
    t.fast_stage = per_chan <= kStagePos * kThreads;
    t.CC = 1;
    if (t.lds_ok) {
        const int cc_max = (int)std::min<long long>(p.C, budget / per_chan);
        const int chunks = (p.C + cc_max - 1) / cc_max;
        t.CC = (p.C + chunks - 1) / chunks;
    }
    return t;
}

// Lane tile and workgroup shape for a problem.
Tiling choose_tiling(const SimPlan &p)
{
    auto pick = [&](int PT, int MT) {
        const int n_mtiles = (p.O + MT - 1) / MT;
        const int G = (p.ow + PT - 1) / PT, gpi = p.oh * G;
        // spatial waves per workgroup: as many as the template tiles leave free, if the image has the groups;
        // fewer if the rows of that many groups do not fit the LDS tile (or its fast staging)
        int nws = 1;
        if (n_mtiles <= 2 && gpi >= 128)
            nws = 2;
        if (n_mtiles <= 1 && gpi >= 256)
            nws = 4;
        Tiling t = try_tiling(p, PT, MT, nws);
        while (nws > 1 && !(t.lds_ok && t.fast_stage)) {
            nws >>= 1;
            t = try_tiling(p, PT, MT, nws);
        }
        return t;
    };
    auto waves = [&](const Tiling &t) {
        const int n_mtiles = (p.O + t.MT - 1) / t.MT, nwm = kWaves / t.nws;
        return (long long)p.B * t.tiles * ((n_mtiles + nwm - 1) / nwm) * kWaves;
    };
    // Wide rows and many templates: 16 pixels x 8 templates per lane (128 accumulators, two waves per SIMD; 8x8
    // and 16x4 tiles measured slower on the 256x64x32x32 / 128-template case) - provided the grid then still
    // gives the SIMDs about two waves each (1.5 on average): a SIMD with a single wave issues at half rate.  Otherwise 4 x 8, which
    // keeps narrow images, small template counts and small batches from idling lanes, waves and CUs.
    if (p.ow >= 32 && p.O >= 32) {
        const Tiling big = pick(kBigPT, kBigMT);
        if (big.lds_ok && waves(big) >= 1536)
            return big;
    }
    return pick(kSmallPT, kSmallMT);
}

template <int MODE, int PT, int MT>
hipError_t launch_direct(const SimKernelArgs &a, dim3 grid, size_t lds_bytes, hipStream_t s)
{
    if (a.sw == 1)
        hipLaunchKernelGGL((sim_direct_kernel<MODE, PT, MT, 1>), grid, dim3(kThreads), lds_bytes, s, a);
    else if (a.sw == 2)
        hipLaunchKernelGGL((sim_direct_kernel<MODE, PT, MT, 2>), grid, dim3(kThreads), lds_bytes, s, a);
    else
        hipLaunchKernelGGL((sim_direct_kernel<MODE, PT, MT, 0>), grid, dim3(kThreads), lds_bytes, s, a);
    return hipGetLastError();
}

template <int MODE>
hipError_t launch_mode(const SimKernelArgs &a, const Tiling &t, hipStream_t s)
{
    if (!t.lds_ok) {
        const long long npix = (long long)a.B * a.oh * a.ow;
        dim3 grid((unsigned)((npix + 255) / 256), (unsigned)a.n_mtiles);
        if (t.MT == 4)
            hipLaunchKernelGGL((sim_gather_kernel<MODE, 4>), grid, dim3(256), 0, s, a);
        else if (t.MT == 16)
            hipLaunchKernelGGL((sim_gather_kernel<MODE, 16>), grid, dim3(256), 0, s, a);
        else
            hipLaunchKernelGGL((sim_gather_kernel<MODE, 8>), grid, dim3(256), 0, s, a);
        return hipGetLastError();
    }
    const int nwm = kWaves / a.nws;
    dim3 grid((unsigned)(a.B * a.tiles), (unsigned)((a.n_mtiles + nwm - 1) / nwm));
    const size_t lds_bytes = (size_t)a.CC * a.TRmax * a.TC * sizeof(float);
    if (t.PT == kBigPT && t.MT == kBigMT)
        return launch_direct<MODE, kBigPT, kBigMT>(a, grid, lds_bytes, s);
    return launch_direct<MODE, kSmallPT, kSmallMT>(a, grid, lds_bytes, s);
}

// the sqrt-weight form runs on the tiled kernel only; its thresholds [O] and wave flags
bool use_sqrtw(const SimPlan &p, const Tiling &t) { return p.algo == SIMNETS_ALGO_SQRTW && t.lds_ok; }

long long guard_flags(const SimPlan &p, const Tiling &t)
{
    const int n_mtiles = (p.O + t.MT - 1) / t.MT, nwm = kWaves / t.nws;
    return (long long)p.B * t.tiles * ((n_mtiles + nwm - 1) / nwm) * kWaves;
}

size_t guard_bytes(const SimPlan &p, const Tiling &t)
{
    if (!use_sqrtw(p, t))
        return 0;
    return align_up((size_t)p.O * sizeof(float), 256) + align_up((size_t)guard_flags(p, t) * sizeof(int), 256);
}

}  // namespace

size_t sim_direct_workspace_bytes(const SimPlan &p)
{
    const Tiling t = choose_tiling(p);
    const size_t n_mtiles = (p.O + t.MT - 1) / t.MT;
    // one extra k of slack behind each array: the parameter loads are issued one step ahead
    const size_t pa = align_up((n_mtiles * p.K + 1) * t.MT * 2 * sizeof(float), 256);
    const size_t pc = align_up((n_mtiles * p.K + 1) * t.MT * sizeof(float), 256);
    const size_t koff = align_up(((size_t)p.K + 2) * sizeof(int), 256);
    return pa + pc + koff + guard_bytes(p, t);
}

int sim_direct_launch(const SimPlan &p, const float *input, const float *templates, const float *weights,
                      float *output, void *workspace, size_t workspace_bytes, hipStream_t s)
{
    const Tiling t = choose_tiling(p);
    const int n_mtiles = (p.O + t.MT - 1) / t.MT;
    const size_t pa_bytes = align_up(((size_t)n_mtiles * p.K + 1) * t.MT * 2 * sizeof(float), 256);
    if (workspace_bytes < sim_direct_workspace_bytes(p))
        return SIMNETS_ERR_WORKSPACE;
    float *pa = reinterpret_cast<float *>(workspace);
    const size_t pc_bytes = align_up(((size_t)n_mtiles * p.K + 1) * t.MT * sizeof(float), 256);
    float *pc = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + pa_bytes);
    int *koff = reinterpret_cast<int *>(reinterpret_cast<char *>(workspace) + pa_bytes + pc_bytes);

    const long long total = (long long)n_mtiles * p.K * t.MT;
    const int pack_blocks = (int)std::min<long long>((total + 255) / 256, 4096);
    const bool sqrtw = use_sqrtw(p, t);
    const int mode = sqrtw ? (int)SIM_MODE_L2_SQRTW : p.mode;
    const size_t koff_bytes = align_up(((size_t)p.K + 2) * sizeof(int), 256);
    float *thr = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + pa_bytes + pc_bytes + koff_bytes);
    int *flags = reinterpret_cast<int *>(reinterpret_cast<char *>(thr) + align_up((size_t)p.O * sizeof(float), 256));
    if (sqrtw) {
        const long long n_flags = guard_flags(p, t);
        const int blocks = (int)std::min<long long>(std::max<long long>((p.O + 3) / 4, (n_flags + 255) / 256), 1024);
        hipLaunchKernelGGL(sim_guard_prep_kernel, dim3(blocks), dim3(256), 0, s, templates, weights, p.O, p.K, thr,
                           flags, n_flags);
        if (hipGetLastError() != hipSuccess)
            return SIMNETS_ERR_HIP;
    }
    hipLaunchKernelGGL(sim_pack_params_kernel, dim3(pack_blocks), dim3(256), 0, s, templates, weights, p.O, p.K, t.MT,
                       n_mtiles, mode, p.fudge, pa, pc, koff, p.bh * p.bw, p.bw, t.CC, t.TRmax * t.TC, t.TC);
    if (hipGetLastError() != hipSuccess)
        return SIMNETS_ERR_HIP;

    SimKernelArgs a;
    a.in = input; a.out = output; a.pa = pa; a.pc = pc; a.koff = koff;
    a.B = p.B; a.C = p.C; a.H = p.H; a.W = p.W; a.O = p.O; a.oh = p.oh; a.ow = p.ow;
    a.bh = p.bh; a.bw = p.bw; a.sh = p.sh; a.sw = p.sw; a.ph = p.ph; a.pw = p.pw; a.K = p.K;
    a.G = t.G; a.gpi = t.gpi; a.tiles = t.tiles; a.nws = t.nws; a.n_mtiles = n_mtiles;
    a.nws_log2 = t.nws == 4 ? 2 : (t.nws == 2 ? 1 : 0);
    a.vec_store = (p.ow % 4 == 0) && ((reinterpret_cast<uintptr_t>(output) & 15) == 0);
    a.TC = t.TC; a.TRmax = t.TRmax; a.CC = t.CC; a.fast_stage = t.fast_stage;
    a.oob = p.oob;
    // Dtype(-0.5) * Dtype(K_) * std::log(2.0 * M_PI), rounded to float by Eigen's constant()
    a.norm_const = (p.mode == SIM_MODE_L2_NORM) ? (float)((double)(-0.5f * (float)p.K) * std::log(2.0 * M_PI)) : 0.0f;
    a.norm_every_iteration = p.norm_const_every_iteration;
    a.templates = templates; a.weights = weights; a.thr = thr; a.flags = flags;

    hipError_t e;
    switch (mode) {
    case SIM_MODE_L1: e = launch_mode<SIM_MODE_L1>(a, t, s); break;
    case SIM_MODE_L2: e = launch_mode<SIM_MODE_L2>(a, t, s); break;
    case SIM_MODE_L2_NORM: e = launch_mode<SIM_MODE_L2_NORM>(a, t, s); break;
    case SIM_MODE_L2_NORM_IGNORE_NAN: e = launch_mode<SIM_MODE_L2_NORM_IGNORE_NAN>(a, t, s); break;
    default: e = launch_mode<SIM_MODE_L2_SQRTW>(a, t, s); break;
    }
    if (e == hipSuccess && sqrtw) {
        // same grid as the main kernel: a wave looks at its flag and, almost always, returns
        const int nwm = kWaves / a.nws;
        dim3 grid((unsigned)(a.B * a.tiles), (unsigned)((a.n_mtiles + nwm - 1) / nwm));
        if (t.PT == kBigPT && t.MT == kBigMT)
            hipLaunchKernelGGL((sim_guard_fix_kernel<kBigPT, kBigMT>), grid, dim3(kThreads), 0, s, a);
        else
            hipLaunchKernelGGL((sim_guard_fix_kernel<kSmallPT, kSmallMT>), grid, dim3(kThreads), 0, s, a);
        e = hipGetLastError();
    }
    return e == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

}  // namespace simnets
