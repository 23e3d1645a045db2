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

#include "fast_div.h"
#include "internal.h"
#include "stage.h"
#include "valu_tile.h"
#include "sim_step.h"

namespace simnets {

namespace {

constexpr int kWaves = 4;                 // waves per workgroup
constexpr int kThreads = 64 * kWaves;
constexpr int kLdsBudgetFloats = 16384;   // 64 KiB of input tile per workgroup
constexpr int kSmWaves = 4;   // the small-map kernel's workgroup: four waves, eight when the grid would otherwise give the
                              // SIMDs at most one wave each (with more waves in the grid, eight measured slower)
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
    int NI, img_lds;   // small-map kernel: images per workgroup and LDS floats of one image's tile (one channel)
    FastDiv d_chan, d_img, d_tc;   // ... divisions of its staging loop: by NI * img_lds, img_lds, TC
    int plds_off;      // PLDS variants: where the workgroup's parameter copy starts in LDS (floats, multiple of 4)
    int xcd_group;     // tiled kernel: number the workgroups so that the template groups of one pixel tile share an XCD
    // sqrt-weight form only (see the guard in sim_direct_kernel)
    const float *pa2;  // [mtile][K][MT][2]  (template, negative weight): what the recomputing pass reads
    const float *thr;  // [O] a partial sum of template m above -thr[m] sends its wave to the recomputing pass
    int *flags;        // [workgroups * kWaves] 1: the wave left its outputs to the recomputing pass
    // self-packing gather kernel only: the parameters as the caller holds them, [O][K] each
    const float *raw_t, *raw_w;
    float fudge;
};

// Output positions of a lane.
struct LanePos {
    int bx, by;        // the workgroup's (pixel tile over the batch, template group)
    int b, tile, ws, mtile;
    int g_first, g_last, row_first;
    int h, gw;
    bool wave_active, lane_valid;
};

__device__ __forceinline__ LanePos lane_pos(const SimKernelArgs &a, int wave, int lane)
{
    LanePos q;
    q.bx = blockIdx.x;
    q.by = blockIdx.y;
    if (a.xcd_group) {
        // Workgroups are handed to the 8 XCDs in turn by their linear number.  The gridDim.y template groups that
        // stage the same pixel tile take numbers a multiple of 8 apart and next to each other in time, so they run on
        // one XCD in the same round and the tile is fetched from HBM once: linear number = ((tile / 8) * gridDim.y +
        // group) * 8 + tile % 8.  (gridDim.x is a multiple of 8 when the host sets this.)
        const unsigned l = blockIdx.x + gridDim.x * blockIdx.y;
        const unsigned j = l >> 3;
        const unsigned q8 = j / gridDim.y;
        q.by = (int)(j - q8 * gridDim.y);
        q.bx = (int)(q8 * 8 + (l & 7));
    }
    q.b = q.bx / a.tiles;
    q.tile = q.bx - q.b * a.tiles;
    q.ws = wave & (a.nws - 1);                   // which 64 pixel groups of the tile
    const int wm = wave >> a.nws_log2;           // which MT templates
    const int nwm = kWaves >> a.nws_log2;
    q.mtile = q.by * nwm + wm;
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
constexpr int kGatherMaxK = 12;            // patch lengths up to which the gather kernel replaces the tiled ones
constexpr int kSmStageGroups = 2;   // small-map kernel: channel groups whose loads are in flight at once while staging
// waves per SIMD the register budget is sized for: 64 accumulators leave room for 4, 128 for 2
constexpr int waves_per_simd(int pt, int mt) { return pt * mt <= 64 ? 4 : 2; }
constexpr int lds_budget_floats(int pt, int mt) { return pt * mt <= 64 ? kLdsBudgetFloats / 2 : kLdsBudgetFloats; }

// GATED: the recomputing pass of the sqrt-weight form, run by a workgroup with a flagged wave behind the main pass:
//        the flagged waves recompute their outputs (MODE = SIM_MODE_L2 on the second packed copy, bit-identical to
//        SIMNETS_ALGO_DIRECT), the others only help staging.
// PLDS:  the workgroup's packed parameters (all K) are copied to LDS once and read from there by broadcast:
//        for short K the step-ahead global loads would cost one memory latency per k.
// ROW3:  3 x 3 templates at stride 1 (the convolution-like layers): the k loop walks (channel, dh) rows of the
//        staged tile; a lane reads the PT + 2 values of a row once and the three taps of the row take their
//        operands from those registers (x of tap dw, pixel p = value dw + p), instead of PT LDS values per tap
//        through a table of offsets: a third of the LDS instructions, no per-k address arithmetic.
// The kernel's body.  wave_bail: sqrt-weight form - out: this wave's guard flag; GATED - in: the flag that selects the
// waves to recompute.
template <int MODE, int PT, int MT, int SWT, bool GATED, bool PLDS, bool ROW3>
__device__ __forceinline__ void sim_direct_body(const SimKernelArgs &a, float *lds, int &wave_bail)
{
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int sw = SWT > 0 ? SWT : a.sw;

    const LanePos lp = lane_pos(a, wave, lane);
    const int b = lp.b, mtile = lp.mtile, h = lp.h, gw = lp.gw;
    const bool lane_valid = lp.lane_valid;
    bool wave_active = lp.wave_active;
    if (GATED)
        wave_active = wave_active && wave_bail != 0;  // the other waves only help staging

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
    // PLDS: the same stream out of the LDS copy (every lane one address: a broadcast read).
    unsigned zero_v;
    asm volatile("v_mov_b32 %0, 0" : "=v"(zero_v));
    constexpr bool HAS_PC = MODE == SIM_MODE_L2_NORM || MODE == SIM_MODE_L2_NORM_IGNORE_NAN;
    const int mtile_c = lp.wave_active ? mtile : 0;
    const int wm = wave >> a.nws_log2;
    const int pk = (a.K + 1) * MT;  // floats of one wave's pc block in LDS (its pa block: twice that), one k of slack
    const char *pa_base = PLDS ? reinterpret_cast<const char *>(lds + a.plds_off + wm * 3 * pk)
                               : reinterpret_cast<const char *>((GATED ? a.pa2 : a.pa) + (size_t)mtile_c * a.K * MT * 2);
    const char *pc_base = PLDS ? reinterpret_cast<const char *>(lds + a.plds_off + wm * 3 * pk + 2 * pk)
                               : reinterpret_cast<const char *>(a.pc + (size_t)mtile_c * a.K * MT);
    if (PLDS) {
        // copy the parameters of the workgroup's template tiles: [wm][pa: K*MT*2 | slack | pc: K*MT | slack]
        const int nwm = kWaves >> a.nws_log2;
        for (int j = 0; j < nwm; ++j) {
            const int mt = min(lp.by * nwm + j, a.n_mtiles - 1);
            const float *ga = a.pa + (size_t)mt * a.K * MT * 2;
            float *la = lds + a.plds_off + j * 3 * pk;
            for (int i = tid; i < a.K * MT * 2; i += kThreads)
                la[i] = ga[i];
            if (HAS_PC) {
                const float *gc = a.pc + (size_t)mt * a.K * MT;
                for (int i = tid; i < a.K * MT; i += kThreads)
                    la[2 * pk + i] = gc[i];
            }
        }
    }
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
    if (!PLDS)
        fetch_params(pa0, pc0);
    TilePositions<kStagePos> tp;
    tp.template init<kThreads>(a.H, a.W, TR, a.TC, in_row0, a.pw);
    // LDS offsets of the patch elements, one scalar load per k, fetched two steps ahead
    const int SIMNETS_CONST_AS *kt = (const int SIMNETS_CONST_AS *)(a.koff);
    // sqrt-weight form: the thresholds of the wave's MT templates, one per lane (lane % MT), requested now and
    // read after the first chunk
    float thr_lane = 0.0f;
    if (MODE == SIM_MODE_L2_SQRTW)
        thr_lane = a.thr[min(mtile_c * MT + (lane % MT), a.O - 1)];

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
        if (PLDS && ch0 == 0)
            fetch_params(pa0, pc0);  // the parameter copy is in place behind the same barrier
        if (PT % 2 == 0 && (MODE == SIM_MODE_L2_SQRTW || MODE == SIM_MODE_L2))
            sim_pin_pairs<PT, MT>(acc);
        if (ROW3 && wave_active) {
            // ---- rows (channel, dh) of the chunk in k order; per row: the next row's values and, per tap, the
            //      next tap's parameters are requested before the arithmetic on the current ones ----
            const int nrow = ccn * 3;
            int roff = a.TC, rdh = 1;   // LDS offset and dh of the row to request next (row 1 at first)
            float xa[PT + 2], xb[PT + 2];
#pragma unroll
            for (int j = 0; j < PT + 2; ++j)
                xa[j] = lds[lds_base + j];
            auto tap = [&](const float *xr, const float (&pac)[2 * MT], const float (&pcc)[MT], float (&panx)[2 * MT],
                           float (&pcnx)[MT]) {
                fetch_params(panx, pcnx);  // one k of slack exists behind the arrays
                __builtin_amdgcn_sched_barrier(0);
                float xs[PT];
#pragma unroll
                for (int p = 0; p < PT; ++p)
                    xs[p] = xr[p];
                sim_step<MODE, PT, MT, true>(acc, xs, pac, pcc);
                __builtin_amdgcn_sched_barrier(0);
            };
            auto row = [&](int r, const float (&cur)[PT + 2], float (&nxt)[PT + 2], float (&pA)[2 * MT], float (&cA)[MT],
                           float (&pB)[2 * MT], float (&cB)[MT]) {
                // everything outstanding was issued a whole tap ago
                __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
                __builtin_amdgcn_sched_barrier(0);
                const int off = r + 1 < nrow ? roff : 0;  // behind the chunk's last row: any valid address
#pragma unroll
                for (int j = 0; j < PT + 2; ++j)
                    nxt[j] = lds[lds_base + off + j];
                rdh += 1;
                roff += a.TC;
                if (rdh == 3) {
                    rdh = 0;
                    roff += chan_lds - 3 * a.TC;
                }
                tap(cur, pA, cA, pB, cB);
                __builtin_amdgcn_s_waitcnt(0x0070);
                __builtin_amdgcn_sched_barrier(0);
                tap(cur + 1, pB, cB, pA, cA);
                __builtin_amdgcn_s_waitcnt(0x0070);
                __builtin_amdgcn_sched_barrier(0);
                tap(cur + 2, pA, cA, pB, cB);
            };
            int r = 0;
            for (; r + 2 <= nrow; r += 2) {
                row(r, xa, xb, pa0, pc0, pa1, pc1);
                row(r + 1, xb, xa, pa1, pc1, pa0, pc0);
            }
            if (r < nrow) {
                row(r, xa, xb, pa0, pc0, pa1, pc1);
#pragma unroll
                for (int i = 0; i < 2 * MT; ++i)
                    pa0[i] = pa1[i];
#pragma unroll
                for (int i = 0; i < MT; ++i)
                    pc0[i] = pc1[i];
            }
        }
        if (!ROW3 && wave_active) {
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
        if (MODE == SIM_MODE_L2_SQRTW && ch0 == 0) {
            // Guard of the sqrt-weight form.  The terms all have one sign, so |acc| only grows from here on: a partial sum
            // that already lies beyond the template's threshold proves the final output does; a wave with a partial
            // sum that does not (or is NaN) stops here and leaves its outputs to the recomputing pass.
            bool suspect = false;
            if (wave_active && lane_valid) {
#pragma unroll
                for (int m = 0; m < MT; ++m) {
                    const int mm = mtile * MT + m;
                    if (mm >= a.O)
                        break;
                    const float thr = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, thr_lane), m));
#pragma unroll
                    for (int p = 0; p < PT; ++p)
                        suspect |= gw * PT + p < a.ow && !(acc[m][p] >= thr);  // (this form accumulates +d*d)
                }
            }
            const bool bail = __any(suspect);
            wave_bail = bail ? 1 : 0;
            if (bail)
                wave_active = false;
        }
    }

    if (!wave_active || !lane_valid)
        return;
    // ---- epilogue ----
    int reps = 0;
    if (MODE == SIM_MODE_L2_NORM)
        reps = a.norm_every_iteration ? (a.B - b) : 1;
    const int w0 = gw * PT;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const int mm = mtile * MT + m;
        if (mm >= a.O)
            break;
        float v[PT];
#pragma unroll
        for (int p = 0; p < PT; ++p) {
            // the sqrt-weight form summed +d*d: 0 - acc is its exact negative, with +0 for an empty sum like the
            // reference's 0 + (-0)
            v[p] = MODE == SIM_MODE_L2_SQRTW ? 0.0f - acc[m][p] : acc[m][p];
            for (int r = 0; r < reps; ++r)
                v[p] += a.norm_const;
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
}

// The kernel: one pass of the body; the sqrt-weight form follows it, in the (rare) workgroups with a flagged wave, by
// the recomputing pass - MODE = SIM_MODE_L2 on the second packed copy for the flagged waves, bit-identical to
// SIMNETS_ALGO_DIRECT - as a cold path of the same launch.
// The recomputing pass as a function of its own, not inlined: its registers are allocated apart from the hot pass's,
// which would otherwise spill to make room for it.  It reads the argument block from the kernel's argument segment
// again instead of taking it from the caller (who would have to keep a copy for the call).  A callable function is not
// given the segment's address (that value is only defined inside kernels), but it is given the address of the
// implicit arguments, which follow the explicit ones - here the block, the kernel's only parameter - at the next
// multiple of 8 bytes.
#if defined(__HIP_DEVICE_COMPILE__)
typedef __attribute__((address_space(3))) float lds_float;
template <int PT, int MT, int SWT, bool ROW3>
__device__ __noinline__ void sim_direct_recompute(lds_float *lds, int wave_bail)
{
    constexpr size_t kExplicitArgs = (sizeof(SimKernelArgs) + 7) & ~size_t(7);
    const SimKernelArgs a = *reinterpret_cast<const SimKernelArgs *>(
        reinterpret_cast<const char *>(__builtin_amdgcn_implicitarg_ptr()) - kExplicitArgs);
    sim_direct_body<SIM_MODE_L2, PT, MT, SWT, true, false, ROW3>(a, (float *)lds, wave_bail);
}
#endif

template <int MODE, int PT, int MT, int SWT, bool PLDS = false, bool ROW3 = false>
__global__ __launch_bounds__(kThreads, waves_per_simd(PT, MT)) void sim_direct_kernel(const SimKernelArgs a)
{
    extern __shared__ float lds[];
    int wave_bail = 0;
    sim_direct_body<MODE, PT, MT, SWT, false, PLDS, ROW3>(a, lds, wave_bail);
    if constexpr (MODE == SIM_MODE_L2_SQRTW) {
        if (__syncthreads_or(wave_bail)) {
#if defined(__HIP_DEVICE_COMPILE__)
            sim_direct_recompute<PT, MT, SWT, ROW3>((lds_float *)lds, wave_bail);
#endif
        }
    }
}

// Small maps (an image has fewer pixel groups than a wave has lanes, or the grid of the tiled kernel would leave
// most SIMDs idle - hundreds of templates over 7 x 7 or 14 x 14 images at small batch): a wave covers NI images
// (lane -> (image, pixel group)), a workgroup one tile of MT templates, and its four waves split K: each walks a
// quarter of every staged channel chunk, the partial sums are added through LDS in wave order at the end (so the
// summation order over k is by quarters of a chunk, not strictly ascending).  Same LDS staging rule (out-of-image ->
// out_of_bounds_value), same packed parameters and offset table, same combine step as the tiled kernel.
template <int MODE, bool GATED = false, int WAVES = kSmWaves>
__global__ __launch_bounds__(64 * WAVES) void sim_small_map_kernel(const SimKernelArgs a)
{
    constexpr int kSmThreads = 64 * WAVES;
    constexpr int PT = kSmallPT, MT = kSmallMT;
    constexpr int NP = 4;   // tile elements per thread and channel the fast staging covers (NP * 256 per channel)
    extern __shared__ float lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int flag_at = blockIdx.y * gridDim.x + blockIdx.x;   // sqrt-weight form: one flag per workgroup
    if (GATED) {
        const int SIMNETS_CONST_AS *fl = (const int SIMNETS_CONST_AS *)(a.flags);
        if (fl[flag_at] == 0)
            return;
    }
    const int img_l = lane / a.gpi, g_l = lane - img_l * a.gpi;
    const int b0 = blockIdx.x * a.NI;
    const bool lane_valid = img_l < a.NI && b0 + img_l < a.B;
    const int img = lane_valid ? img_l : 0, g = lane_valid ? g_l : 0;
    const int b = b0 + img;
    const int h = g / a.G, gw = g - h * a.G;
    const int lds_base = img * a.img_lds + h * a.sh * a.TC + gw * PT * a.sw;
    const int mtile = blockIdx.y;
    const int taps = a.bh * a.bw;
    const int chan_lds = a.NI * a.img_lds;
    const size_t plane = (size_t)a.H * a.W;

    float acc[MT][PT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int p = 0; p < PT; ++p)
            acc[m][p] = 0.0f;
    const float *pa_t = (GATED ? a.pa2 : a.pa) + (size_t)mtile * a.K * MT * 2;
    const float *pc_t = a.pc + (size_t)mtile * a.K * MT;
    const int SIMNETS_CONST_AS *koff = (const int SIMNETS_CONST_AS *)(a.koff);

    // where this thread's tile elements come from: its NP elements span a group of channels (every group of a chunk
    // has the same geometry), several groups are in flight at once
    const bool fast = chan_lds <= NP * kSmThreads;
    GroupedTile<NP> gt;
    if (fast)
        gt.template init<kSmThreads>(a.H, a.W, a.img_lds / a.TC, a.TC, -a.ph, a.pw, a.NI, min(a.NI, a.B - b0),
                                     a.C * a.H * a.W, chan_lds, a.CC);

    for (int ch0 = 0; ch0 < a.C; ch0 += a.CC) {
        const int ccn = min(a.CC, a.C - ch0);
        __syncthreads();
        // ---- the chunk's tile ----
        if (fast) {
            gt.template stage<kSmStageGroups>(lds, a.in + ((size_t)b0 * a.C + ch0) * plane, (int)plane, ccn, ccn, chan_lds,
                                              a.oob, nullptr);
        } else {
            const int total = ccn * chan_lds;
            for (int idx = tid; idx < total; idx += kSmThreads) {
                const int cc = (int)fast_div((unsigned)idx, a.d_chan), r1 = idx - cc * chan_lds;
                const int im = (int)fast_div((unsigned)r1, a.d_img), r2 = r1 - im * a.img_lds;
                const int r = (int)fast_div((unsigned)r2, a.d_tc), c = r2 - r * a.TC;
                const int ih = r - a.ph, iw = c - a.pw, bb = b0 + im;
                float v = a.oob;
                if (bb < a.B && ih >= 0 && ih < a.H && iw >= 0 && iw < a.W)
                    v = a.in[((size_t)bb * a.C + ch0 + cc) * plane + (size_t)ih * a.W + iw];
                lds[idx] = v;   // == cc * chan_lds + im * img_lds + r * TC + c
            }
        }
        __syncthreads();
        const int cpw = (ccn + WAVES - 1) / WAVES;
        const int c_lo = min(wave * cpw, ccn), c_hi = min(c_lo + cpw, ccn);
        const int kl0 = c_lo * taps, nk = (c_hi - c_lo) * taps;   // this wave's steps, counted inside the chunk
        // Software pipeline: the pixel values (LDS) and the parameters of the next U steps are requested before the
        // arithmetic of the current U, two register sets.  The parameters come through scalar loads (one
        // s_load_dwordx16 per step) and are moved to VGPRs once per step by the combine (sim_step without VP): on this
        // narrow tile a step has only 64-96 VALU instructions, and four lane-uniform vector or LDS loads per step -
        // 16 / 8 cycles of the compute unit's one texture / LDS pipe each, shared by its four SIMDs - would bound the
        // loop (a coalesced vector load per eight steps with the values taken out of the lanes by v_readlane measured
        // slower as well: 0.53 against 0.44 ms on 512x7x7 at batch 32).  Scalar loads return in any order, so the wait
        // is for all of them: two steps per wait (where the scalar registers allow it: the modes without a
        // per-template constant) double the time a load has to arrive.
        constexpr int U = (MODE == SIM_MODE_L2_NORM || MODE == SIM_MODE_L2_NORM_IGNORE_NAN) ? 1 : 2;
        if (nk > 0) {
            const int kg0 = ch0 * taps + kl0;   // this wave's first step, counted over all K
            const int SIMNETS_CONST_AS *kt = koff + kg0;
            const float SIMNETS_CONST_AS *pw = (const float SIMNETS_CONST_AS *)(pa_t) + (size_t)kg0 * (2 * MT);
            const float SIMNETS_CONST_AS *pq = (const float SIMNETS_CONST_AS *)(pc_t) + (size_t)kg0 * MT;
            float x0[U][PT], x1[U][PT], pa0[U][2 * MT], pa1[U][2 * MT], pc0[U][MT], pc1[U][MT];
            int offn[U];   // LDS offsets of the steps the next fetch reads (steps beyond the wave's last repeat it)
#pragma unroll
            for (int u = 0; u < U; ++u)
                offn[u] = kt[min(u, nk - 1)];
            auto fetch = [&](int j, float (&xs)[U][PT], float (&pas)[U][2 * MT], float (&pcs)[U][MT]) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int jj = min(j + u, nk - 1);
#pragma unroll
                    for (int p = 0; p < PT; ++p)
                        xs[u][p] = lds[lds_base + offn[u] + p * a.sw];
                    load_params<MODE, MT>(pas[u], pcs[u], pw + (size_t)jj * (2 * MT), pq + (size_t)jj * MT);
                }
#pragma unroll
                for (int u = 0; u < U; ++u)
                    offn[u] = kt[min(j + U + u, nk - 1)];
            };
            auto run = [&](int j, const float (&xs)[U][PT], const float (&pas)[U][2 * MT], const float (&pcs)[U][MT]) {
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (j + u < nk)
                        sim_step<MODE, PT, MT, false>(acc, xs[u], pas[u], pcs[u]);
            };
            fetch(0, x0, pa0, pc0);
            for (int j = 0; j < nk; j += 2 * U) {
                __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): issued a whole block of steps ago
                __builtin_amdgcn_sched_barrier(0);
                fetch(j + U, x1, pa1, pc1);
                __builtin_amdgcn_sched_barrier(0);
                run(j, x0, pa0, pc0);
                __builtin_amdgcn_sched_barrier(0);
                if (j + U >= nk)
                    break;
                __builtin_amdgcn_s_waitcnt(0xC07F);
                __builtin_amdgcn_sched_barrier(0);
                fetch(j + 2 * U, x0, pa0, pc0);
                __builtin_amdgcn_sched_barrier(0);
                run(j + U, x1, pa1, pc1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    // ---- partial sums of waves 1..3 -> wave 0, in wave order; the tile's LDS is reused ----
    constexpr int kPart = MT * PT * 64;
    __syncthreads();
    if (wave > 0) {
        float *dst = lds + (size_t)(wave - 1) * kPart + lane;
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int p = 0; p < PT; ++p)
                dst[(m * PT + p) * 64] = acc[m][p];
    }
    __syncthreads();
    if (wave > 0)
        return;
#pragma unroll 1
    for (int w = 1; w < WAVES; ++w) {
        const float *src = lds + (size_t)(w - 1) * kPart + lane;
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int p = 0; p < PT; ++p)
                acc[m][p] += src[(m * PT + p) * 64];
    }
    const int w0 = gw * PT;
    if (MODE == SIM_MODE_L2_SQRTW) {
        // guard of the sqrt-weight form on the finished sums: a workgroup with an output below its template's
        // threshold (or a template with a negative weight: threshold +inf) raises its flag and is recomputed
        const float SIMNETS_CONST_AS *thr = (const float SIMNETS_CONST_AS *)(a.thr);
        bool suspect = false;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const float th = thr[min(mtile * MT + m, a.O - 1)];
#pragma unroll
            for (int p = 0; p < PT; ++p)
                suspect |= lane_valid && mtile * MT + m < a.O && w0 + p < a.ow && !(acc[m][p] >= th);
        }
        const int bail = __any(suspect) ? 1 : 0;
        if (lane == 0)
            a.flags[flag_at] = bail;
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
        float *o = a.out + (((size_t)b * a.O + mm) * a.oh + h) * a.ow + w0;
#pragma unroll
        for (int p = 0; p < PT; ++p) {
            float v = MODE == SIM_MODE_L2_SQRTW ? 0.0f - acc[m][p] : acc[m][p];
            for (int r = 0; r < reps; ++r)
                v += a.norm_const;
            if (w0 + p < a.ow)
                o[p] = v;
        }
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
        float v = MODE == SIM_MODE_L2_SQRTW ? 0.0f - acc[m][0] : acc[m][0];
        for (int r = 0; r < reps; ++r)
            v += a.norm_const;
        a.out[(((size_t)b * a.O + mm) * a.oh + h) * a.ow + w] = v;
    }
}

// The gather kernel for patches of at most kGatherMaxK elements when the caller's parameters have not been packed
// (the self-packing forward call): the workgroup packs the parameters of its template tile into LDS itself (the same
// sim_pack_element, so the same values) and reads them from there, which saves the pack launch, at this size as long
// as the kernel itself.  Same order over k, same combine step: results identical to sim_gather_kernel's.
template <int MODE, int MT>
__global__ __launch_bounds__(256) void sim_gather_selfpack_kernel(const SimKernelArgs a)
{
    constexpr bool HAS_PC = MODE == SIM_MODE_L2_NORM || MODE == SIM_MODE_L2_NORM_IGNORE_NAN;
    __shared__ float spa[kGatherMaxK * 2 * MT];
    __shared__ float spc[kGatherMaxK * MT];
    const int mtile = blockIdx.y;
    for (int i = threadIdx.x; i < a.K * MT; i += 256) {
        const int k = i / MT, m = mtile * MT + (i - k * MT);
        float t = 0.0f, w = 0.0f;
        if (m < a.O) {
            t = a.raw_t[(size_t)m * a.K + k];
            w = a.raw_w[(size_t)m * a.K + k];
        }
        sim_pack_element(MODE, m < a.O, t, w, a.fudge, spa[2 * i], spa[2 * i + 1], spc[i]);
    }
    __syncthreads();
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
    const float *img = a.in + (size_t)b * a.C * a.H * a.W;
    const float *pa = spa, *pc = spc;
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
#pragma unroll
                for (int i = 0; i < 2 * MT; ++i)
                    pav[i] = pa[i];
#pragma unroll
                for (int i = 0; i < MT; ++i)
                    pcv[i] = HAS_PC ? pc[i] : 0.0f;
                sim_step<MODE, 1, MT, true>(acc, x, pav, pcv);
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
// Sqrt-weight form (pa2 != nullptr): pa holds (sqrt(w) t, -sqrt(w)), pa2 the plain (t, -w) pairs of the recomputing
// pass, and the workgroups from `pack_blocks` on write the thresholds, one wave per template:
// thr[m] = sum_k w t^2 / 1024, or +inf for a template with a negative or NaN weight (sqrt undefined).
__global__ __launch_bounds__(256) void sim_pack_params_kernel(const float *__restrict__ templates,
                                                             const float *__restrict__ weights, int O, int K, int MT,
                                                             int n_mtiles, int mode, float fudge, float *__restrict__ pa,
                                                             float *__restrict__ pc, int *__restrict__ koff, int taps,
                                                             int bw, int CC, int chan_pitch, int TC,
                                                             float *__restrict__ pa2, float *__restrict__ thr,
                                                             int pack_blocks)
{
    if ((int)blockIdx.x >= pack_blocks) {
        const int lane = threadIdx.x & 63;
        const int nb = gridDim.x - pack_blocks;
        for (int m = (blockIdx.x - pack_blocks) * 4 + (threadIdx.x >> 6); m < O; m += nb * 4) {
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
        return;
    }
    const int nthreads = pack_blocks * 256;
    // LDS offset of patch element k inside a staged chunk of CC channels; 0 behind the last k
    for (int k = blockIdx.x * 256 + threadIdx.x; k < K + 2; k += nthreads) {
        int off = 0;
        if (k < K) {
            const int c = k / taps, rem = k - c * taps;
            const int dh = rem / bw, dw = rem - dh * bw;
            off = (c % CC) * chan_pitch + dh * TC + dw;
        }
        koff[k] = off;
    }
    const long long total = (long long)n_mtiles * K * MT;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += nthreads) {
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
        if (pa2 != nullptr) {
            float unused;
            sim_pack_element(SIM_MODE_L2, m < O, t, w, fudge, pa2[2 * i], pa2[2 * i + 1], unused);
        }
    }
}

struct Tiling {
    int PT, MT, nws, G, gpi, tiles, TC, TRmax, CC;
    int NI;            // > 0: the small-map kernel with NI images per workgroup (CC, chan_pitch are then that kernel's)
    int sm_waves;      // ... and its waves per workgroup
    int chan_pitch;    // LDS floats of one staged channel
    bool lds_ok;       // the tiled kernels run: the rows of a workgroup's pixel groups fit the LDS tile and the
                       // patches are not too short to be worth staging (else: gather kernel)
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
    t.NI = 0;
    t.chan_pitch = t.TRmax * t.TC;
    return t;
}

constexpr int kSmallMapLdsFloats = 8192;   // 32 KiB of tile per workgroup of the small-map kernel; twice that when the
                                           // grid has at most two workgroups per compute unit (half as many chunk phases)

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
    Tiling t = pick(kSmallPT, kSmallMT);
    // Short patches (the 2x2 first layer of the missing-data network, 1x1 and 3x3 patches of one channel): a pixel's
    // whole patch is a handful of loads, and staging rows through LDS behind a barrier only adds dependent phases -
    // one pixel per lane straight from global memory, four template tiles per pixel group of 256 (1x28x28 -> 32, 2x2
    // s2 p2: 8.3 -> 4.0 us per prepared call at 64 images, 11.6 -> 9.5 at 512, 26.3 -> 24.8 at 2048; 3x3 of one channel
    // 10.2 -> 6.6 / 28.2 -> 25.0; 12 elements 11.8 -> 8.1 / 37.7 -> 33.5; 16 and more: no gain on large grids)
    if (p.K <= kGatherMaxK) {
        t.lds_ok = false;
        return t;
    }
    // Small maps: a whole image is one tile of at most 64 pixel groups, and either several images fit a wave or the
    // tiled grid has at most one wave per SIMD while K is long enough to split over the four waves.
    if (t.lds_ok && t.nws == 1 && t.tiles == 1 && p.C >= kSmWaves) {
        const int NI = (int)std::max(1, std::min(p.B, 64 / t.gpi));
        const long long per_chan = 1LL * NI * t.TRmax * t.TC;
        if ((NI >= 2 || waves(t) <= 1024) && per_chan <= kSmallMapLdsFloats) {
            t.NI = NI;
            t.chan_pitch = (int)per_chan;
            const int n_mtiles = (p.O + t.MT - 1) / t.MT;
            const long long wgs = (long long)((p.B + NI - 1) / NI) * n_mtiles;
            t.sm_waves = (wgs * kSmWaves <= 1024 && p.C >= 2 * kSmWaves) ? 2 * kSmWaves : kSmWaves;
            const int lds_floats = wgs <= 512 ? 2 * kSmallMapLdsFloats : kSmallMapLdsFloats;
            const int cc_max = (int)std::min<long long>(p.C, lds_floats / per_chan);
            const int chunks = (p.C + cc_max - 1) / cc_max;
            t.CC = (p.C + chunks - 1) / chunks;
            // the waves of the workgroup split a chunk's channels: a multiple of their number keeps them even
            if (t.CC >= t.sm_waves && t.CC % t.sm_waves)
                t.CC = t.CC / t.sm_waves * t.sm_waves;
        }
    }
    return t;
}

template <int MODE, int PT, int MT, bool PLDS>
hipError_t launch_direct(const SimKernelArgs &a, dim3 grid, size_t lds_bytes, hipStream_t s)
{
    // (the normalized modes keep the table-driven loop: with their extra operands the row form does not fit the
    // register file)
    constexpr bool kRow3 = PT == kBigPT && !PLDS && (MODE == SIM_MODE_L1 || MODE == SIM_MODE_L2 || MODE == SIM_MODE_L2_SQRTW);
    if (kRow3 && a.sw == 1 && a.bh == 3 && a.bw == 3) {
        hipLaunchKernelGGL((sim_direct_kernel<MODE, PT, MT, 1, false, kRow3>), grid, dim3(kThreads), lds_bytes, s,
                           a);
        return hipGetLastError();
    }
    if (a.sw == 1)
        hipLaunchKernelGGL((sim_direct_kernel<MODE, PT, MT, 1, PLDS>), grid, dim3(kThreads), lds_bytes, s, a);
    else if (a.sw == 2)
        hipLaunchKernelGGL((sim_direct_kernel<MODE, PT, MT, 2, PLDS>), grid, dim3(kThreads), lds_bytes, s, a);
    else
        hipLaunchKernelGGL((sim_direct_kernel<MODE, PT, MT, 0, PLDS>), grid, dim3(kThreads), lds_bytes, s, a);
    return hipGetLastError();
}

// Floats of the workgroup's parameter copy in LDS (PLDS variants): per template wave (K + 1) * MT * 3.
size_t plds_floats(const SimPlan &p, const Tiling &t) { return (size_t)(kWaves / t.nws) * (p.K + 1) * t.MT * 3; }

// Short K on the small lane tile: the parameters go through LDS (one memory latency instead of one per k).
bool use_plds(const SimPlan &p, const Tiling &t)
{
    return t.lds_ok && t.NI == 0 && t.PT == kSmallPT && t.MT == kSmallMT && plds_floats(p, t) * sizeof(float) <= 16384;
}

template <int MODE, bool GATED = false>
hipError_t launch_mode(const SimKernelArgs &a0, const Tiling &t, bool plds, hipStream_t s)
{
    SimKernelArgs a = a0;
    if (!t.lds_ok) {
        const long long npix = (long long)a.B * a.oh * a.ow;
        dim3 grid((unsigned)((npix + 255) / 256), (unsigned)a.n_mtiles);
        if (a.raw_t != nullptr) {
            if constexpr (MODE != SIM_MODE_L2_SQRTW && !GATED)
                hipLaunchKernelGGL((sim_gather_selfpack_kernel<MODE, kSmallMT>), grid, dim3(256), 0, s, a);
        } else if (t.MT == 4)
            hipLaunchKernelGGL((sim_gather_kernel<MODE, 4>), grid, dim3(256), 0, s, a);
        else if (t.MT == 16)
            hipLaunchKernelGGL((sim_gather_kernel<MODE, 16>), grid, dim3(256), 0, s, a);
        else
            hipLaunchKernelGGL((sim_gather_kernel<MODE, 8>), grid, dim3(256), 0, s, a);
        return hipGetLastError();
    }
    if (t.NI > 0) {
        dim3 grid((unsigned)((a.B + t.NI - 1) / t.NI), (unsigned)a.n_mtiles);
        const size_t floats = std::max<size_t>((size_t)t.CC * t.chan_pitch, (size_t)(t.sm_waves - 1) * kSmallMT * kSmallPT * 64);
        if (t.sm_waves == kSmWaves)
            hipLaunchKernelGGL((sim_small_map_kernel<MODE, GATED, kSmWaves>), grid, dim3(64 * kSmWaves),
                               floats * sizeof(float), s, a);
        else
            hipLaunchKernelGGL((sim_small_map_kernel<MODE, GATED, 2 * kSmWaves>), grid, dim3(128 * kSmWaves),
                               floats * sizeof(float), s, a);
        return hipGetLastError();
    }
    const int nwm = kWaves / a.nws;
    dim3 grid((unsigned)(a.B * a.tiles), (unsigned)((a.n_mtiles + nwm - 1) / nwm));
    size_t lds_bytes = (size_t)a.CC * a.TRmax * a.TC * sizeof(float);
    if (GATED)
        return hipSuccess;   // the tiled kernels recompute flagged waves inside the main launch
    a.xcd_group = grid.y > 1 && grid.x % 8 == 0;
    if (t.PT == kBigPT && t.MT == kBigMT)
        return launch_direct<MODE, kBigPT, kBigMT, false>(a, grid, lds_bytes, s);
    if (plds) {
        lds_bytes = ((size_t)a.plds_off + (size_t)nwm * (a.K + 1) * kSmallMT * 3) * sizeof(float);
        return launch_direct<MODE, kSmallPT, kSmallMT, true>(a, grid, lds_bytes, s);
    }
    return launch_direct<MODE, kSmallPT, kSmallMT, false>(a, grid, lds_bytes, s);
}

// The sqrt-weight form runs on the tiled kernels and on the small-map kernel; there only with enough pixels per
// parameter, or packing the second copy of the parameters costs more than the shorter inner loop saves (512
// templates over 512 x 7 x 7 inputs: at 32 images 0.425 -> 0.391 ms per self-packing call and 0.413 -> 0.358 ms
// prepared, at 16 images 0.222 -> 0.223 and 0.212 -> 0.190 ms, at 8 images the same ratios).
bool use_sqrtw(const SimPlan &p, const Tiling &t)
{
    return p.algo == SIMNETS_ALGO_SQRTW && t.lds_ok && (t.NI == 0 || (long long)p.B * p.oh * p.ow >= 512);
}

// flags of the guard that live in the workspace: one per workgroup of the small-map kernel (the tiled kernels keep
// theirs in registers)
long long guard_flags(const SimPlan &p, const Tiling &t)
{
    const int n_mtiles = (p.O + t.MT - 1) / t.MT;
    return t.NI > 0 ? (long long)((p.B + t.NI - 1) / t.NI) * n_mtiles : 0;
}

// Where the pieces of the workspace lie.  The first three are what every mode reads; the sqrt-weight form adds
// the second packed copy and the thresholds (all written by the pack kernel) and, for the small-map kernel, the
// workgroup flags (written by every main launch, read by the recomputing launch behind it).
struct Layout {
    size_t pa, pc, koff, pa2, thr, flags, total;
};

Layout layout(const SimPlan &p, const Tiling &t)
{
    const size_t n_mtiles = (p.O + t.MT - 1) / t.MT;
    // one extra k of slack behind each array: the parameter loads are issued one step ahead
    const size_t pa_bytes = align_up((n_mtiles * p.K + 1) * t.MT * 2 * sizeof(float), 256);
    Layout l;
    l.pa = 0;
    l.pc = l.pa + pa_bytes;
    l.koff = l.pc + align_up((n_mtiles * p.K + 1) * t.MT * sizeof(float), 256);
    l.pa2 = l.koff + align_up(((size_t)p.K + 2) * sizeof(int), 256);
    l.thr = l.pa2;
    l.flags = l.pa2;
    l.total = l.pa2;
    if (use_sqrtw(p, t)) {
        l.thr = l.pa2 + pa_bytes;
        l.flags = l.thr + align_up((size_t)p.O * sizeof(float), 256);
        l.total = l.flags + align_up((size_t)guard_flags(p, t) * sizeof(int), 256);
    }
    return l;
}

}  // namespace

size_t sim_direct_workspace_bytes(const SimPlan &p) { return layout(p, choose_tiling(p)).total; }

// Writes everything of the workspace that depends on the parameters only (one launch).
int sim_direct_prepare(const SimPlan &p, const float *templates, const float *weights, void *workspace,
                       size_t workspace_bytes, hipStream_t s)
{
    const Tiling t = choose_tiling(p);
    const Layout l = layout(p, t);
    if (workspace_bytes < l.total)
        return SIMNETS_ERR_WORKSPACE;
    char *ws = reinterpret_cast<char *>(workspace);
    const int n_mtiles = (p.O + t.MT - 1) / t.MT;
    const long long total = (long long)n_mtiles * p.K * t.MT;
    const int pack_blocks = (int)std::min<long long>((total + 255) / 256, 4096);
    const bool sqrtw = use_sqrtw(p, t);
    const int mode = sqrtw ? (int)SIM_MODE_L2_SQRTW : p.mode;
    const int thr_blocks = sqrtw ? std::min((p.O + 3) / 4, 1024) : 0;
    hipLaunchKernelGGL(sim_pack_params_kernel, dim3(pack_blocks + thr_blocks), dim3(256), 0, s, templates, weights, p.O,
                       p.K, t.MT, n_mtiles, mode, p.fudge, reinterpret_cast<float *>(ws + l.pa),
                       reinterpret_cast<float *>(ws + l.pc), reinterpret_cast<int *>(ws + l.koff), p.bh * p.bw, p.bw, t.CC,
                       t.chan_pitch, t.TC, sqrtw ? reinterpret_cast<float *>(ws + l.pa2) : nullptr,
                       reinterpret_cast<float *>(ws + l.thr), pack_blocks);
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

// The self-packing call of a short-patch geometry on the gather kernel needs no packed parameters.
static bool gather_packs_itself(const SimPlan &p, const Tiling &t)
{
    return !t.lds_ok && p.K <= kGatherMaxK && t.MT == kSmallMT;
}

// raw_templates / raw_weights: non-null for a geometry that packs inside the kernel (gather_packs_itself).
static int sim_direct_run_on(const SimPlan &p, const float *input, float *output, void *workspace,
                             size_t workspace_bytes, hipStream_t s, const float *raw_templates,
                             const float *raw_weights)
{
    const Tiling t = choose_tiling(p);
    const Layout l = layout(p, t);
    if (workspace_bytes < l.total)
        return SIMNETS_ERR_WORKSPACE;
    char *ws = reinterpret_cast<char *>(workspace);
    const int n_mtiles = (p.O + t.MT - 1) / t.MT;
    const bool sqrtw = use_sqrtw(p, t);
    const int mode = sqrtw ? (int)SIM_MODE_L2_SQRTW : p.mode;

    SimKernelArgs a;
    a.in = input; a.out = output;
    a.pa = reinterpret_cast<const float *>(ws + l.pa); a.pc = reinterpret_cast<const float *>(ws + l.pc);
    a.koff = reinterpret_cast<const int *>(ws + l.koff);
    a.B = p.B; a.C = p.C; a.H = p.H; a.W = p.W; a.O = p.O; a.oh = p.oh; a.ow = p.ow;
    a.bh = p.bh; a.bw = p.bw; a.sh = p.sh; a.sw = p.sw; a.ph = p.ph; a.pw = p.pw; a.K = p.K;
    a.G = t.G; a.gpi = t.gpi; a.tiles = t.tiles; a.nws = t.nws; a.n_mtiles = n_mtiles;
    a.nws_log2 = t.nws == 4 ? 2 : (t.nws == 2 ? 1 : 0);
    a.vec_store = (p.ow % 4 == 0) && ((reinterpret_cast<uintptr_t>(output) & 15) == 0);
    a.TC = t.TC; a.TRmax = t.TRmax; a.CC = t.CC; a.fast_stage = t.fast_stage;
    a.plds_off = (int)align_up((size_t)t.CC * t.chan_pitch, 4);
    a.xcd_group = 0;
    a.NI = t.NI; a.img_lds = t.TRmax * t.TC;
    a.d_chan = make_fast_div((unsigned)std::max(1, t.chan_pitch)); a.d_img = make_fast_div((unsigned)std::max(1, a.img_lds));
    a.d_tc = make_fast_div((unsigned)std::max(1, t.TC));
    a.oob = p.oob;
    // Dtype(-0.5) * Dtype(K_) * std::log(2.0 * M_PI), rounded to float by Eigen's constant()
    a.norm_const = (p.mode == SIM_MODE_L2_NORM) ? (float)((double)(-0.5f * (float)p.K) * std::log(2.0 * M_PI)) : 0.0f;
    a.norm_every_iteration = p.norm_const_every_iteration;
    a.pa2 = reinterpret_cast<const float *>(ws + l.pa2);
    a.thr = reinterpret_cast<const float *>(ws + l.thr);
    a.flags = reinterpret_cast<int *>(ws + l.flags);
    a.raw_t = raw_templates; a.raw_w = raw_weights; a.fudge = p.fudge;

    const bool plds = use_plds(p, t);
    hipError_t e;
    switch (mode) {
    case SIM_MODE_L1: e = launch_mode<SIM_MODE_L1>(a, t, plds, s); break;
    case SIM_MODE_L2: e = launch_mode<SIM_MODE_L2>(a, t, plds, s); break;
    case SIM_MODE_L2_NORM: e = launch_mode<SIM_MODE_L2_NORM>(a, t, plds, s); break;
    case SIM_MODE_L2_NORM_IGNORE_NAN: e = launch_mode<SIM_MODE_L2_NORM_IGNORE_NAN>(a, t, plds, s); break;
    default: e = launch_mode<SIM_MODE_L2_SQRTW>(a, t, plds, s); break;
    }
    if (e == hipSuccess && sqrtw)  // small maps: same grid, a workgroup looks at its flag and, almost always, returns
        e = launch_mode<SIM_MODE_L2, true>(a, t, false, s);
    return e == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

// The forward launches on a prepared workspace.
int sim_direct_run(const SimPlan &p, const float *input, float *output, void *workspace, size_t workspace_bytes,
                   hipStream_t s)
{
    return sim_direct_run_on(p, input, output, workspace, workspace_bytes, s, nullptr, nullptr);
}

int sim_direct_launch(const SimPlan &p, const float *input, const float *templates, const float *weights,
                      float *output, void *workspace, size_t workspace_bytes, hipStream_t s)
{
    if (gather_packs_itself(p, choose_tiling(p)))
        return sim_direct_run_on(p, input, output, workspace, workspace_bytes, s, templates, weights);
    const int rc = sim_direct_prepare(p, templates, weights, workspace, workspace_bytes, s);
    return rc ? rc : sim_direct_run(p, input, output, workspace, workspace_bytes, s);
}

}  // namespace simnets
