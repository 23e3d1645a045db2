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
//     include/utils/mex_utils.hpp:69-116).  A workgroup takes 64*PX consecutive slots of ONE region,
//     so the offsets it needs, offsets[r, m, k], do not depend on the pixel; nothing is regrouped in
//     memory, each thread maps its slot straight to the (c, h, w) it belongs to for either region
//     flavour (contiguous "shared" tiles or interleaved "unshared" ones).
//   * K is walked in chunks of KC (32, or 64 / 128 for long K at one pixel per lane): the workgroup gathers the patch elements of its pixels with the
//     im2col_3d index rule (out of image -> blocks_out_of_bounds_value) into LDS, [k][pixel], and
//     copies the matching offsets, pre-packed [k][instance], next to them.
//   * a lane owns PX pixels (slots lane, lane+64, ...) and its wave 16 instances: per k it reads its
//     PX pixel values (lane-distinct) and 16 offsets (one address for the whole wave: an LDS
//     broadcast, so the operand arrives in VGPRs; VALU instructions with SGPR operands issue at half
//     rate on this chip) and updates PX*16 running values held in VGPRs.
//   * the 4 waves of a workgroup split the instances (WM ways) and, when the grid would otherwise
//     leave SIMDs idle, K (KS ways, WM*KS = 4): each K-split wave keeps its own (max, sum) pair and
//     the pairs are merged through LDS at the end: sum = sum_i s_i * exp(eps*(m_i - max_i m_i)).
//   * default for finite eps: the product form on the fp32 matrix cores (below).  Offsets too far apart for it, and
//     infinite eps, take one pass over K with a max-tracked ("online") log-sum-exp at chunk granularity: per staged
//     chunk the maximum of patch + offset first, then the running sums are rescaled to the new maximum and the
//     chunk's exponentials added (the reference sweeps K twice: maximum, then sum of exp relative to it,
//     src/kernels/mex_kernel_cpu.cpp:11-38).  For finite eps the patch values (when staged) and the offsets (when
//     packed) are multiplied by eps*log2(e) once, so a term is add, subtract, v_exp_f32, add; a negative eps turns
//     the reference's minimum into a maximum of the scaled values.
//   * workgroups that own the different regions of the same pixel chunk are numbered a multiple of
//     8 apart, so they run on the same XCD and their interleaved partial cache lines meet in one L2.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>
#include <cmath>

#include "internal.h"
#include "mex_common.h"
#include "sim_step.h"

namespace simnets {

namespace {

constexpr int MX = 16;        // instances per wave
constexpr int kChunkMin = 32;  // k per LDS chunk: 32, or 64 / 128 for long K with one pixel per lane
constexpr int kXcds = 8;
#ifndef SIMNETS_MEX_WAVES
#define SIMNETS_MEX_WAVES 4096  // pixels per lane shrink until the grid has this many waves
#endif

constexpr int cmax(int a, int b) { return a > b ? a : b; }

typedef float floatx4 __attribute__((ext_vector_type(4)));

// EPS: 0 = finite epsilon, +1 / -1 = epsilon +inf / -inf (plain maximum / minimum of patch + offset).
template <int PX, int KS, int KC, int EPS, bool CHECK>
__global__ __launch_bounds__(256, PX == 2 ? 4 : 1) void mex_fwd_kernel(const MexKernelArgs a)
{
    constexpr bool NEG = EPS < 0, INF = EPS != 0;
    constexpr int WM = 4 / KS;            // instance waves per workgroup
    constexpr int TM = WM * MX;           // instances per workgroup
    constexpr int TP = 64 * PX;           // pixels per workgroup
    constexpr int KSTEP = 256 / TP;       // k handled per staging round (4, 2 or 1)
    constexpr int KW = KC / KS;           // k of a chunk each K-split wave walks
    constexpr int kMergeFloats = (KS - 1) * WM * 64 * PX * MX * 2;
    // The k-oriented gather (below) writes xs with lanes along k: its rows get a pitch of TP + 1 floats so
    // that those writes spread over the banks.  Only the K-split variants can take it (LDS room).
    constexpr bool KGATHER = PX == 1 && KS >= 2;
    constexpr int XP = KGATHER ? TP + 1 : TP;   // KC * XP stays a multiple of 4: the offsets tile behind it is 16-byte aligned
    __shared__ __attribute__((aligned(16))) float smem[cmax(KC * XP + KC * TM, kMergeFloats)];
    __shared__ long long pref_off[KGATHER ? 64 : 1];
    __shared__ int pref_c[KGATHER ? 64 * 3 : 1];
    __shared__ float pmx[256];            // product form: partial pixel maxima [k phase][pixel]
    __shared__ float fsh[TP], msh[TP];    // product form: per pixel, the rescale factor of this chunk and the running maximum
    __shared__ long long pout[TP];        // product form: where instance 0 of the pixel goes in the output, -1 for an empty slot
    float *xs = smem;                     // [k][pixel], row pitch XP
    float *os = smem + KC * XP;           // [k][instance]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WM, wk = wave / WM;

    // blockIdx.x -> (pixel chunk, region): the R regions of chunk c get ids that agree mod 8
    int r, chunk;
    {
        const int per_super = kXcds * a.R;
        const int super = (int)fast_div(blockIdx.x, a.dSuper);
        const int within = blockIdx.x - super * per_super;
        r = within / kXcds;
        chunk = super * kXcds + (within - r * kXcds);
    }
    if (chunk >= a.cpr)
        return;  // padding of the last super-group (uniform for the whole workgroup)
    const int mgroup = blockIdx.y;
    const int m0 = mgroup * TM + wm * MX;            // first instance of this wave
    const bool wave_active = m0 < a.M;

    // staging role: this thread gathers pixel `sp` for k = sk, sk + KSTEP, ...
    const int sp = tid % TP, sk = tid / TP;
    const int sk_u = __builtin_amdgcn_readfirstlane(sk);
    const PixelRef gp = locate(a, r, chunk * TP + sp);
    // Product form (finite epsilon): with bounds mp >= patch values of the pixel and mo >= offsets of the instance,
    // sum_k exp2(x_k + o_k - mp - mo) = sum_k exp2(x_k - mp) * exp2(o_k - mo): one exponential per staged patch
    // element (shared by all instances), the offsets' exponentials packed once, and one fused multiply-add per
    // term.  The largest term is at least exp2(-(row range of the offsets)), so the form is used when the ranges
    // of all instances of the workgroup are small enough for that to stay far inside the normal range; otherwise
    // the workgroup runs the two sweeps.
    bool prod = false;
    if constexpr (!INF) {
        const float *rng = a.orng + ((size_t)r * a.n_mgroups + mgroup) * TM;
        const float rg = tid < TM ? rng[tid] : 0.0f;
        prod = !__syncthreads_or(!(rg <= kProductRange));
        if (!prod && !(KGATHER && a.kgather)) {
            // Rows too wide on their own but finite: the product form still holds where every pixel's patch spans at
            // most kProductRange (see there).  One extra sweep over the patches, only in such workgroups: thread
            // (pixel sp, phase sk) takes the elements sk, sk + KSTEP, ... of its pixel.
            const int any_unbounded = __syncthreads_or(!(rg < INFINITY));
            float hi = -INFINITY, lo = INFINITY;
            for (int k = sk_u; k < a.K; k += KSTEP) {
                const int4 ke = a.ktab[k];
                bool ok = true;
                if (CHECK) {
                    const int ci = gp.ci0 + ke.y, hi_ = gp.hi0 + ke.z, wi = gp.wi0 + ke.w;
                    ok = ci >= 0 && ci < a.C && hi_ >= 0 && hi_ < a.H && wi >= 0 && wi < a.W;
                }
                const float raw = *(ok ? gp.base + ke.x : a.in);   // (always a valid address)
                const float v = (ok ? raw : a.oob) * a.scale;
                hi = fmaxf(hi, v);
                lo = fminf(lo, v);
            }
            pmx[sk * TP + sp] = hi;
            __syncthreads();
            float chi = hi;
#pragma unroll
            for (int j = 0; j < KSTEP; ++j)
                chi = fmaxf(chi, pmx[j * TP + sp]);
            __syncthreads();
            pmx[sk * TP + sp] = lo;
            __syncthreads();
            float clo = lo;
#pragma unroll
            for (int j = 0; j < KSTEP; ++j)
                clo = fminf(clo, pmx[j * TP + sp]);
            // (a pixel with an infinite value, or nothing finite, is not narrow; the barrier frees the array again)
            prod = !__syncthreads_or(!(chi - clo <= kProductRange)) && !any_unbounded;
        }
    }
    const float *offp = (prod ? a.offe : a.offp) + ((size_t)r * a.n_mgroups + mgroup) * a.K * TM;
    float m_run = -INFINITY;  // running maximum of this thread's staging pixel (product form)
    if (prod && sk == 0)
        pout[sp] = gp.out_off < 0 ? -1 : (long long)gp.b * a.M * ((long long)a.Co * a.Ho * a.Wo) + gp.out_off;
    if (KGATHER && a.kgather && tid < 64) {
        // pixel table for the k-oriented gather: where each of the 64 pixels' patches starts
        pref_off[tid] = gp.base - a.in;
        pref_c[3 * tid] = gp.ci0; pref_c[3 * tid + 1] = gp.hi0; pref_c[3 * tid + 2] = gp.wi0;
    }

    auto stage = [&](int k0, int kc) {
        constexpr int U = KC / KSTEP;                    // patch elements per thread and chunk
        const bool full = kc == KC;                      // all but the last chunk: no per-element guards
        // offsets: a straight copy of kc * TM floats, after the gather's loads have been issued
        const float4 *src = reinterpret_cast<const float4 *>(offp + (size_t)k0 * TM);
        float4 *dst = reinterpret_cast<float4 *>(os);
        const int on = kc * (TM / 4);
        float v[U];
        if (KGATHER && a.kgather) {
            // Consecutive pixel slots are different images here (one pixel per image and region), a whole image
            // apart in memory, while consecutive patch elements are one channel plane apart: lanes run along k.
            // Thread (kq, pq) gathers elements kq, kq + 64, ... of pixels pq, pq + 4, ...
            const int kq = tid & 63, pq = tid >> 6;   // (the pixel table was written before the barrier in front of this call)
            for (int kk = kq; kk < kc; kk += 64) {
                const int4 ke = a.ktab[k0 + kk];
                const int o = ke.x, dc = ke.y, dh = ke.z, dw = ke.w;
                float g[16];
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int p = pq + 4 * i;
                    bool ok = true;
                    if (CHECK) {
                        const int ci = pref_c[3 * p] + dc, hi = pref_c[3 * p + 1] + dh, wi = pref_c[3 * p + 2] + dw;
                        ok = ci >= 0 && ci < a.C && hi >= 0 && hi < a.H && wi >= 0 && wi < a.W;
                    }
                    g[i] = ok ? a.in[pref_off[p] + o] : a.oob;
                }
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    xs[kk * XP + pq + 4 * i] = g[i] * a.scale;
            }
            if (prod) {
                __syncthreads();
#pragma unroll
                for (int u = 0; u < U; ++u)
                    v[u] = xs[min(sk + u * KSTEP, kc - 1) * XP + sp];
            }
        } else {
            // patch elements: xs[kk][sp] = patch(sp)[k0 + kk], kk = sk, sk + KSTEP, ...: all gathers of the chunk
            // in flight before the first LDS store
#pragma unroll
            for (int u = 0; u < U; ++u) {
                // sk is the same for a whole wave (TP is a multiple of 64): the table entry comes through a scalar load
                const int kk = sk_u + u * KSTEP;
                const int4 ke = a.ktab[k0 + (full ? kk : min(kk, kc - 1))];
                const int o = ke.x;
                if (CHECK) {
                    const int dc = ke.y, dh = ke.z, dw = ke.w;
                    const int ci = gp.ci0 + dc, hi = gp.hi0 + dh, wi = gp.wi0 + dw;
                    const bool ok = ci >= 0 && ci < a.C && hi >= 0 && hi < a.H && wi >= 0 && wi < a.W;
                    v[u] = ok ? gp.base[o] : a.oob;
                } else {
                    v[u] = gp.base[o];
                }
            }
        }
        for (int i = tid; i < on; i += 256)
            dst[i] = src[i];
        if (!(KGATHER && a.kgather)) {
#pragma unroll
            for (int u = 0; u < U; ++u)
                v[u] *= a.scale;
            if (!prod) {
#pragma unroll
                for (int u = 0; u < U; ++u)
                    if (full || sk_u + u * KSTEP < kc)
                        xs[(sk + u * KSTEP) * XP + sp] = v[u];
            }
        }
        if (prod) {
            // pixel maximum over the chunk -> running maximum; the staged values become exp2(x - maximum)
            float pm = -INFINITY;
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (full || sk_u + u * KSTEP < kc)
                    pm = fmaxf(pm, v[u]);
            if (KSTEP > 1) {
                pmx[sk * TP + sp] = pm;
                __syncthreads();
#pragma unroll
                for (int j = 0; j < KSTEP; ++j)
                    pm = fmaxf(pm, pmx[j * TP + sp]);
            }
            const float m_new = fmaxf(m_run, pm);
            const float m_sub = m_new == -INFINITY ? 0.0f : m_new;  // nothing finite yet: the terms are exp2(-inf) = 0
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (full || sk_u + u * KSTEP < kc)
                    xs[(sk + u * KSTEP) * XP + sp] = __builtin_amdgcn_exp2f(v[u] - m_sub);
            if (sk == 0) {
                fsh[sp] = m_run == m_new ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
                msh[sp] = m_new;
            }
            m_run = m_new;
            if (!full) {
                // the matrix instruction takes 4 k at a time: rows kc .. next multiple of 4 are zeros
                const int kc4 = (kc + 3) & ~3;
                for (int i = tid; i < (kc4 - kc) * TP; i += 256)
                    xs[(kc + i / TP) * XP + i % TP] = 0.0f;
                for (int i = tid; i < (kc4 - kc) * TM; i += 256)
                    os[kc * TM + i] = 0.0f;
            }
        }
    };

    float mx[PX][MX];
#pragma unroll
    for (int p = 0; p < PX; ++p)
#pragma unroll
        for (int m = 0; m < MX; ++m)
            mx[p][m] = NEG ? INFINITY : -INFINITY;

    const float *xl = xs + lane;                 // this lane's pixels: xl[kk*TP + p*64]
    const float *ol = os + wm * MX;              // this wave's instances: ol[kk*TM + m]

    float s[PX][MX];
#pragma unroll
    for (int p = 0; p < PX; ++p)
#pragma unroll
        for (int m = 0; m < MX; ++m)
            s[p][m] = 0.0f;

    if (prod) {
        // ---- one sweep on the fp32 matrix cores: S[instance][pixel] = sum_k exp2(o_k - mo) * exp2(x_k - mp), in
        //      tiles of 16 instances x 16 pixels x 4 k (v_mfma_f32_16x16x4_f32: lane (lr, lq) supplies
        //      A[instance lr][k lq] and B[k lq][pixel lr] and holds D[instance 4*lq + v][pixel lr]); the sums are
        //      rescaled when a chunk raises mp ----
        constexpr int NT = 4 * PX;  // 16-pixel tiles across the workgroup's pixels
        const int lr = lane & 15, lq = lane >> 4;
        floatx4 acc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t)
            acc[t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        const float *xa = xs + lq * XP + lr;
        const float *oa = os + lq * TM + wm * MX + lr;
        for (int k0 = 0; k0 < a.K; k0 += KC) {
            const int kc = min(KC, a.K - k0);
            __syncthreads();
            stage(k0, kc);
            __syncthreads();
            if (!wave_active)
                continue;
            if (k0 > 0) {
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    acc[t] *= fsh[t * 16 + lr];
            }
            const int kend = min((kc + 3) & ~3, (wk + 1) * KW);  // rows kc .. kend - 1 hold zeros
            for (int kq = wk * KW; kq < kend; kq += 4) {
                const float av = oa[kq * TM];
                float bv[NT];
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    bv[t] = xa[kq * XP + t * 16];
#pragma unroll
                for (int t = 0; t < NT; ++t)
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv[t], acc[t], 0, 0, 0);
            }
        }
        float mp[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t)
            mp[t] = msh[t * 16 + lr];
        if (KS > 1) {
            // the K-split waves saw the same pixel maxima: their sums add up in wave wk == 0
            __syncthreads();  // everyone is done with xs / os
            if (wk > 0 && wave_active) {
                float *mg = smem + (size_t)((wk - 1) * WM + wm) * (NT * 4 * 64) + lane;
#pragma unroll
                for (int t = 0; t < NT; ++t)
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        mg[(t * 4 + v) * 64] = acc[t][v];
            }
            __syncthreads();
            if (wk > 0)
                return;
            if (wave_active) {
                for (int j = 1; j < KS; ++j) {
                    const float *src = smem + (size_t)((j - 1) * WM + wm) * (NT * 4 * 64) + lane;
#pragma unroll
                    for (int t = 0; t < NT; ++t)
#pragma unroll
                        for (int v = 0; v < 4; ++v)
                            acc[t][v] += src[(t * 4 + v) * 64];
                }
            }
        }
        if (!wave_active)
            return;
        const size_t plane = (size_t)a.Co * a.Ho * a.Wo;
        const float *omax = a.omax + ((size_t)r * a.n_mgroups + mgroup) * TM + wm * MX + 4 * lq;
        float shift[4];
#pragma unroll
        for (int v = 0; v < 4; ++v)
            shift[v] = omax[v] + a.c0;
        const size_t row0 = (size_t)(m0 + 4 * lq) * plane;  // this lane's first instance row
        const bool all_rows = m0 + MX <= a.M;               // same for the whole wave
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const long long po = pout[t * 16 + lr];  // written before the first barrier
            if (po < 0)
                continue;
            float *o = a.out + po + row0;
            // an infinite pixel bound makes the result NaN, as the reference's exp(inf - inf) does
            const float mpt = (mp[t] - mp[t]) + mp[t];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float res = (__builtin_amdgcn_logf(acc[t][v]) + (mpt + shift[v])) * a.ln2_over_eps;
                if (all_rows || m0 + 4 * lq + v < a.M)
                    o[v * plane] = res;
            }
        }
        return;
    }
    // ---- one pass over K, chunk by chunk (wide offsets, infinite epsilon): per chunk first the maximum (minimum for a
    //      negative infinite epsilon) of patch + offset over the chunk's k, then - finite epsilon - the running sums are
    //      rescaled to the new running maximum and the chunk's exponentials added: a max-tracked ("online") log-sum-exp
    //      at chunk granularity, one exponential per term and one per output and chunk; the patch elements and the
    //      offsets are fetched once.  Patch values and offsets are already multiplied by eps*log2(e), so a term is
    //      exp2 of a plain difference.  Infinite epsilon stops after the maximum. ----
    if constexpr (INF) {
        // The extreme value alone: two k per step, a term is an add whose offset operand comes from another lane of
        // the quad and half a three-operand maximum.  Lane q of a quad fetches instances 4q .. 4q + 3 of the wave's
        // 16 (one 16-byte read per lane and k instead of four: the reads of a step are what the LDS return path
        // carries, whether or not the lanes ask for the same address).
        auto quad = [](float v, auto q) {
            return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v),
                                                                         decltype(q)::value * 0x55, 0xF, 0xF, true));
        };
        auto best3 = [](float m, float p, float q) {
            return NEG ? __builtin_fminf(__builtin_fminf(m, p), q) : __builtin_fmaxf(__builtin_fmaxf(m, p), q);
        };
        const float *oq = ol + 4 * (lane & 3);
        for (int k0 = 0; k0 < a.K; k0 += KC) {
            const int kc = min(KC, a.K - k0);
            __syncthreads();
            stage(k0, kc);
            __syncthreads();
            if (!wave_active)
                continue;
            const int kend = min(kc, (wk + 1) * KW);
            for (int kk = wk * KW; kk < kend; kk += 2) {
                const int k1 = min(kk + 1, kend - 1);   // (an odd count takes its last k twice)
                float x0[PX], x1[PX];
#pragma unroll
                for (int p = 0; p < PX; ++p) {
                    x0[p] = xl[kk * XP + p * 64];
                    x1[p] = xl[k1 * XP + p * 64];
                }
                const float4 f0 = *reinterpret_cast<const float4 *>(oq + kk * TM);
                const float4 f1 = *reinterpret_cast<const float4 *>(oq + k1 * TM);
                const float o0[4] = {f0.x, f0.y, f0.z, f0.w}, o1[4] = {f1.x, f1.y, f1.z, f1.w};
#pragma unroll
                for (int p = 0; p < PX; ++p)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        using std::integral_constant;
                        mx[p][j] = best3(mx[p][j], x0[p] + quad(o0[j], integral_constant<int, 0>{}),
                                         x1[p] + quad(o1[j], integral_constant<int, 0>{}));
                        mx[p][4 + j] = best3(mx[p][4 + j], x0[p] + quad(o0[j], integral_constant<int, 1>{}),
                                             x1[p] + quad(o1[j], integral_constant<int, 1>{}));
                        mx[p][8 + j] = best3(mx[p][8 + j], x0[p] + quad(o0[j], integral_constant<int, 2>{}),
                                             x1[p] + quad(o1[j], integral_constant<int, 2>{}));
                        mx[p][12 + j] = best3(mx[p][12 + j], x0[p] + quad(o0[j], integral_constant<int, 3>{}),
                                              x1[p] + quad(o1[j], integral_constant<int, 3>{}));
                    }
            }
        }
    } else {
    for (int k0 = 0; k0 < a.K; k0 += KC) {
        const int kc = min(KC, a.K - k0);
        __syncthreads();
        stage(k0, kc);
        __syncthreads();
        if (!wave_active)
            continue;
        const int kend = min(kc, (wk + 1) * KW);
        // (one pixel of the lane and eight of the wave's instances at a time: the chunk maxima of those eight outputs
        // are all that is held beside the running pairs, which keeps this path inside the register budget of the
        // product form above)
        constexpr int HM = 8;
#pragma unroll
        for (int ph = 0; ph < PX * (MX / HM); ++ph) {
            const int p = ph / (MX / HM), h0 = (ph % (MX / HM)) * HM;
            const float *xp = xl + p * 64;
            const float *op = ol + h0;
            float cm[HM];
#pragma unroll
            for (int m = 0; m < HM; ++m)
                cm[m] = -INFINITY;
#pragma nounroll
            for (int kk = wk * KW; kk < kend; ++kk) {
                const float x = xp[kk * XP];
                float v[HM];
                // stage by stage across the instances: a dependent VALU instruction issued right behind its producer
                // stalls, so producers and consumers are kept apart
#pragma unroll
                for (int m = 0; m < HM; ++m)
                    v[m] = x + op[kk * TM + m];
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int m = 0; m < HM; ++m)
                    cm[m] = __builtin_fmaxf(cm[m], v[m]);
                __builtin_amdgcn_sched_barrier(0);
            }
            // new running maximum; sums so far rescaled to it (a maximum that did not move: factor 1, which also keeps
            // -inf - -inf out of the exponent while nothing finite has been seen)
#pragma unroll
            for (int m = 0; m < HM; ++m) {
                const float mo = mx[p][h0 + m];
                const float mn = __builtin_fmaxf(mo, cm[m]);
                s[p][h0 + m] *= mn == mo ? 1.0f : __builtin_amdgcn_exp2f(mo - mn);
                mx[p][h0 + m] = mn;
                cm[m] = mn == -INFINITY ? 0.0f : mn;   // what the chunk's terms subtract
            }
#pragma nounroll
            for (int kk = wk * KW; kk < kend; ++kk) {
                const float x = xp[kk * XP];
                float v[HM];
#pragma unroll
                for (int m = 0; m < HM; ++m)
                    v[m] = x + op[kk * TM + m];
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int m = 0; m < HM; ++m)
                    v[m] = v[m] - cm[m];
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int m = 0; m < HM; ++m)
                    v[m] = __builtin_amdgcn_exp2f(v[m]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int m = 0; m < HM; ++m)
                    s[p][h0 + m] += v[m];
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    }
    }

    if (KS > 1) {
        // ---- merge the (max, sum) pairs of the K-split waves into wave wk == 0 ----
        __syncthreads();  // everyone is done with xs / os
        // layout [split wave][value][lane]: consecutive lanes hit consecutive banks
        float *mg = smem + (size_t)((wk > 0 ? wk - 1 : 0) * WM + wm) * (PX * MX * 2 * 64) + lane;
        if (wk > 0 && wave_active) {
#pragma unroll
            for (int p = 0; p < PX; ++p)
#pragma unroll
                for (int m = 0; m < MX; ++m) {
                    mg[((p * MX + m) * 2) * 64] = mx[p][m];
                    if constexpr (!INF)
                        mg[((p * MX + m) * 2 + 1) * 64] = s[p][m];
                }
        }
        __syncthreads();
        if (wk > 0)
            return;
        if (wave_active) {
            for (int j = 1; j < KS; ++j) {
                const float *src = smem + (size_t)((j - 1) * WM + wm) * (PX * MX * 2 * 64) + lane;
#pragma unroll
                for (int p = 0; p < PX; ++p)
#pragma unroll
                    for (int m = 0; m < MX; ++m) {
                        const float m2 = src[((p * MX + m) * 2) * 64];
                        const float m1 = mx[p][m];
                        const float mm = NEG ? __builtin_fminf(m1, m2) : __builtin_fmaxf(m1, m2);
                        mx[p][m] = mm;
                        if constexpr (INF)
                            continue;
                        const float s2 = src[((p * MX + m) * 2 + 1) * 64];
                        // a side that saw no finite term keeps sum 0; skip the rescale when its
                        // max equals the merged one (also avoids inf - inf)
                        const float f1 = (m1 == mm) ? 1.0f : __builtin_amdgcn_exp2f(m1 - mm);
                        const float f2 = (m2 == mm) ? 1.0f : __builtin_amdgcn_exp2f(m2 - mm);
                        s[p][m] = s[p][m] * f1 + s2 * f2;
                    }
            }
        }
    }
    if (!wave_active)
        return;

    // output channel = instance * channels_out + c  (src/kernels/mex_kernel_cpu.cpp:113-115)
    const size_t plane = (size_t)a.Co * a.Ho * a.Wo;
#pragma unroll
    for (int p = 0; p < PX; ++p) {
        const PixelRef cp = locate(a, r, chunk * TP + p * 64 + lane);
        if (cp.out_off < 0)
            continue;
        float *o = a.out + (size_t)cp.b * a.M * plane + cp.out_off;
#pragma unroll
        for (int m = 0; m < MX; ++m) {
            // (max + ey*log2(e) + log2(sum)) * log(2)/eps in the scaled domain; the plain max for infinite eps
            // (an infinite extreme value makes the finite-epsilon result NaN, as the reference's exp(inf - inf) does)
            const float b = mx[p][m];
            const float res = INF ? b : (__builtin_amdgcn_logf(s[p][m]) + ((b - b) + b + a.c0)) * a.ln2_over_eps;
            if (m0 + m < a.M)
                o[(size_t)(m0 + m) * plane] = res;
        }
    }
}

// One wave per (region, instance) row of the offsets: optional logsumexp normalisation
// (python/simnets/keras.py:155-160) and the scaling, then the row is scattered into the k-major packed layout
// [r][mgroup][k][tm]; for finite epsilon also its exponentials relative to the row maximum, the maximum and the
// row's range (what the product form of the forward kernel reads).  KL > 0: the row (K <= 64 * KL) is read once and
// kept in registers for the three reductions and the scatter; KL = 0: every pass reads it again.
template <int KL>
__global__ __launch_bounds__(256) void mex_pack_offsets_kernel(const float *__restrict__ offsets, int R, int M, int K,
                                                              int n_mgroups, int tm, int normalize, float scale,
                                                              int finite_eps, float *__restrict__ offp,
                                                              float *__restrict__ offe, float *__restrict__ omax,
                                                              float *__restrict__ orng, int4 *__restrict__ ktab, int H,
                                                              int W, int bh, int bw, int row_blocks, SimPackJob job,
                                                              float *__restrict__ normalized_out, MexPackTwin tw,
                                                              int for_gradients)
{
    if ((int)blockIdx.x >= row_blocks) {
        // extra workgroups: the parameters of a Similarity layer evaluated inside the MEX staging
        // layout: channels in chunks of 32, inside a chunk by staging phase (k % 4) and then k / 4, so that the 8
        // channels one staging thread evaluates for a tap are 16 (pa) / 8 (pc) consecutive floats
        const int Opad = (job.O + 31) & ~31;
        const long long total = (long long)Opad * job.K;
        for (long long i = (long long)(blockIdx.x - row_blocks) * 256 + threadIdx.x; i < total;
             i += (long long)(gridDim.x - row_blocks) * 256) {
            const int k = (int)(i / job.K), j = (int)(i - (long long)k * job.K);
            const size_t src = (size_t)min(k, job.O - 1) * job.K + j;   // past the last channel: a copy (never used)
            const int r32 = k & 31;
            const size_t pos = ((((size_t)(k >> 5) * 4 + (r32 & 3)) * job.K + j) * 8) + (r32 >> 2);
            sim_pack_element(job.mode, true, job.templates[src], job.weights[src], job.fudge, job.pa[2 * pos],
                             job.pa[2 * pos + 1], job.pc[pos]);
        }
        return;
    }
    if (blockIdx.x == 0) {
        // patch element k = (dc*bh + dh)*bw + dw -> where it lies relative to the patch origin
        for (int k = threadIdx.x; k < K; k += 256) {
            const int dc = k / (bh * bw);
            const int rem = k - dc * bh * bw;
            const int dh = rem / bw, dw = rem - dh * bw;
            ktab[k] = make_int4((dc * H + dh) * W + dw, dc, dh, dw);
            if (tw.offp != nullptr)
                tw.ktab[k] = ktab[k];
        }
    }
    // a wave per (region, instance) with the instances padded to the groups of the layout (of the wider of the two
    // layouts when the launch writes a second one)
    const int lane = threadIdx.x & 63;
    // Workgroups go to the chip's eight dies in turn, each with an L2 of its own, and the 64 rows of a packed group
    // interleave in 4-byte pieces of the same cache lines: the 16 workgroups of such a group are numbered 8 apart, so
    // that one die's L2 collects their pieces into whole lines (pieces of a line written from several dies each reach
    // memory as a partial line).
    unsigned wg = blockIdx.x;
    if (wg < ((unsigned)row_blocks & ~127u))
        wg = (((wg >> 7) * 8 + (wg & 7)) << 4) + ((wg >> 3) & 15);
    const long long wave = (long long)wg * 4 + (threadIdx.x >> 6);
    const int Mp = n_mgroups * tm, Mp2 = tw.offp != nullptr ? tw.n_mgroups * tw.tm : 0;
    const int Mw = max(Mp, Mp2);
    if (wave >= (long long)R * Mw)
        return;
    const int m = (int)(wave % Mw), r = (int)(wave / Mw);
    const long long row = (long long)r * Mp + m;
    float *dst = offp + ((size_t)r * n_mgroups + m / tm) * K * tm + m % tm;
    float *dste = offe + (dst - offp);
    // the second layout (finite epsilon only; its readers, the gradient kernels, take the exponentials, the row maxima
    // and the ranges, not the scaled values): same values, its own group size
    const int tm2 = tw.tm;
    const long long row2 = (long long)r * Mp2 + m;
    float *dste2 = nullptr;
    if (m < Mp2)
        dste2 = tw.offe + ((size_t)r * tw.n_mgroups + m / tm2) * K * tm2 + m % tm2;
    if (m >= M) {
        for (int k = lane; k < K; k += 64) {
            if (m < Mp) {
                dst[(size_t)k * tm] = 0.0f;
                if (finite_eps)
                    dste[(size_t)k * tm] = 0.0f;
            }
            if (dste2 != nullptr)
                dste2[(size_t)k * tm2] = 0.0f;
        }
        if (finite_eps && lane == 0) {
            if (m < Mp) {
                omax[row] = 0.0f;
                orng[row] = 0.0f;
            }
            if (dste2 != nullptr) {
                tw.omax[row2] = 0.0f;
                tw.orng[row2] = 0.0f;
            }
        }
        return;
    }
    const float *src = offsets + ((size_t)r * M + m) * K;
    float rv[KL > 0 ? KL : 1];
    if (KL > 0) {
#pragma unroll
        for (int j = 0; j < KL; ++j)
            rv[j] = src[min(lane + 64 * j, K - 1)];
    }
    auto each = [&](auto &&f) __attribute__((always_inline)) {
        if constexpr (KL > 0) {
#pragma unroll
            for (int j = 0; j < KL; ++j)
                if (lane + 64 * j < K)
                    f(lane + 64 * j, rv[j]);
        } else {
            for (int k = lane; k < K; k += 64)
                f(k, src[k]);
        }
    };
    float lse = 0.0f;
    if (normalize) {
        float mxv = -INFINITY;
        each([&](int, float x) { mxv = fmaxf(mxv, x); });
        for (int d = 32; d > 0; d >>= 1)
            mxv = fmaxf(mxv, __shfl_xor(mxv, d, 64));
        if (!(fabsf(mxv) < INFINITY))
            mxv = 0.0f;
        float sum = 0.0f;
        each([&](int, float x) { sum += mex_exp_term(x - mxv); });
        for (int d = 32; d > 0; d >>= 1)
            sum += __shfl_xor(sum, d, 64);
        lse = mex_lse_of(sum, mxv);
    }
    if (normalized_out != nullptr) {   // the same values as mex_normalize_rows_kernel writes
        float *nd = normalized_out + ((size_t)r * M + m) * K;
        each([&](int k, float x) { nd[k] = x - lse; });
    }
    if (!finite_eps) {
        each([&](int k, float x) { dst[(size_t)k * tm] = mex_scaled_offset(x, lse, scale); });
        return;
    }
    // the row's extreme elements (scaling is monotone: they give the largest and the smallest scaled value)
    float xmx = -INFINITY, xmn = INFINITY;
    each([&](int, float x) {
        xmx = fmaxf(xmx, x);
        xmn = fminf(xmn, x);
    });
    for (int d = 32; d > 0; d >>= 1) {
        xmx = fmaxf(xmx, __shfl_xor(xmx, d, 64));
        xmn = fminf(xmn, __shfl_xor(xmn, d, 64));
    }
    const float xh = scale >= 0.0f ? xmx : xmn;
    const float hi = mex_scaled_offset(xh, lse, scale), lo = mex_scaled_offset(scale >= 0.0f ? xmn : xmx, lse, scale);
    each([&](int k, float x) {
        const float v = mex_scaled_offset(x, lse, scale);
        const float e = __builtin_amdgcn_exp2f(mex_offset_exponent(x, xh, lse, scale));
        dst[(size_t)k * tm] = v;
        dste[(size_t)k * tm] = e;
        if (dste2 != nullptr)
            dste2[(size_t)k * tm2] = e;
    });
    if (lane == 0) {
        // the gradient kernels' copy: a row far from zero counts as too wide for their product form (kGradOffsetsSize)
        const float grng = fabsf(hi) > kGradOffsetsSize || fabsf(lo) > kGradOffsetsSize ? INFINITY : hi - lo;
        omax[row] = hi;
        orng[row] = for_gradients ? grng : hi - lo;  // NaN or inf (infinite entries) sends the workgroup to the two sweeps
        if (dste2 != nullptr) {
            tw.omax[row2] = hi;
            tw.orng[row2] = grng;
        }
    }
}

template <int PX, int KS, int KC>
hipError_t launch_variant(const MexKernelArgs &a, dim3 grid, int eps, bool inside, hipStream_t s)
{
    if (eps < 0 && inside)
        hipLaunchKernelGGL((mex_fwd_kernel<PX, KS, KC, -1, false>), grid, dim3(256), 0, s, a);
    else if (eps < 0)
        hipLaunchKernelGGL((mex_fwd_kernel<PX, KS, KC, -1, true>), grid, dim3(256), 0, s, a);
    else if (eps > 0 && inside)
        hipLaunchKernelGGL((mex_fwd_kernel<PX, KS, KC, 1, false>), grid, dim3(256), 0, s, a);
    else if (eps > 0)
        hipLaunchKernelGGL((mex_fwd_kernel<PX, KS, KC, 1, true>), grid, dim3(256), 0, s, a);
    else if (inside)
        hipLaunchKernelGGL((mex_fwd_kernel<PX, KS, KC, 0, false>), grid, dim3(256), 0, s, a);
    else
        hipLaunchKernelGGL((mex_fwd_kernel<PX, KS, KC, 0, true>), grid, dim3(256), 0, s, a);
    return hipGetLastError();
}

// one pixel per lane: the LDS chunk grows with K (fewer gather/barrier phases; K <= chunk needs one gather only)
template <int KS>
hipError_t launch_px1(const MexKernelArgs &a, dim3 grid, int eps, bool inside, int kc, hipStream_t s)
{
    if (kc == 128)
        return launch_variant<1, KS, 128>(a, grid, eps, inside, s);
    if (kc == 64)
        return launch_variant<1, KS, 64>(a, grid, eps, inside, s);
    return launch_variant<1, KS, kChunkMin>(a, grid, eps, inside, s);
}

// Few pixels, long K (the classifier head of a network: a handful of instances over hundreds of channels at 1x1
// spatial size): the tiling above would launch a few workgroups with long serial instruction streams.  Here one
// wave owns one output pixel and the lanes split K: KL patch elements per lane stay in registers.  Finite epsilon:
// the product form of the tiled kernel, per wave - the pixel's maximum mp (one shuffle reduction), exp2(x_k - mp)
// once per element, then per instance a dot product with the packed exp2(o_k - mo) row and one shuffle reduction.
// Instances whose offsets range is too wide for that, and infinite epsilon, take patch + offset term by term
// (maximum, then the sum of exponentials relative to it).  The offsets come packed with one instance per group:
// rows [r][m][k].
constexpr int kSmallMChunk = 16;  // instances per wave

template <int KL, bool NEG>
__global__ __launch_bounds__(256) void mex_small_kernel(const MexKernelArgs a)
{
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const long long gid = (long long)blockIdx.x * 4 + wave;
    if (gid >= (long long)a.R * a.slots)
        return;
    const int r = (int)(gid / a.slots);
    const int slot = (int)(gid - (long long)r * a.slots);
    const PixelRef px = locate(a, r, slot);
    if (px.out_off < 0)
        return;  // ragged region edge (same for the whole wave)

    const int m_first = blockIdx.y * kSmallMChunk;
    const int m_end = min(a.M, m_first + kSmallMChunk);
    const size_t row0 = (size_t)r * a.M;
    constexpr int MG = 4;   // instances at a time: their shuffle reductions are independent, so the latencies overlap
    bool kv[KL];
#pragma unroll
    for (int j = 0; j < KL; ++j)
        kv[j] = lane + 64 * j < a.K;
    // The packed rows of the next four instances are requested while the current four are reduced, the first four
    // before anything else: exp2(o - row maximum) for finite epsilon (the product form; an instance whose range
    // turns out too wide loads its plain row again), the plain rows otherwise.
    const float *rows = (a.finite_eps ? a.offe : a.offp) + row0 * a.K;
    float on[MG][KL];
    auto fetch_rows = [&](int m0) __attribute__((always_inline)) {
#pragma unroll
        for (int g = 0; g < MG; ++g) {
            const float *row = rows + (size_t)min(m0 + g, a.M - 1) * a.K;
#pragma unroll
            for (int j = 0; j < KL; ++j)
                on[g][j] = row[kv[j] ? lane + 64 * j : 0];
        }
    };
    fetch_rows(m_first);

    const int bhw = a.bh * a.bw;
    float x[KL];
#pragma unroll
    for (int j = 0; j < KL; ++j) {
        const int k = lane + 64 * j;
        const int kk = kv[j] ? k : 0;
        const int dc = kk / bhw;
        const int rem = kk - dc * bhw;
        const int dh = rem / a.bw, dw = rem - dh * a.bw;
        const int ci = px.ci0 + dc, hi = px.hi0 + dh, wi = px.wi0 + dw;
        const bool ok = ci >= 0 && ci < a.C && hi >= 0 && hi < a.H && wi >= 0 && wi < a.W;
        x[j] = ok ? px.base[((ptrdiff_t)dc * a.H + dh) * a.W + dw] : a.oob;
    }
    // Wave reductions through the data-parallel-primitive lane patterns (neighbour, pair, half-row mirror, row mirror:
    // after the four steps every lane holds its 16-lane row's result) and four lane reads for the rows: VALU latencies
    // instead of a round trip through the LDS crossbar per step.  All 64 lanes are active here.
    auto dpp = [](float v, auto ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), decltype(ctrl)::value,
                                                                      0xF, 0xF, false));
    };
    auto lane_of = [](float v, int l) {
        return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
    };
    using std::integral_constant;
    auto wave_sum = [&](float (&v)[MG]) {
#pragma unroll
        for (int g = 0; g < MG; ++g) v[g] += dpp(v[g], integral_constant<int, 0xB1>{});
#pragma unroll
        for (int g = 0; g < MG; ++g) v[g] += dpp(v[g], integral_constant<int, 0x4E>{});
#pragma unroll
        for (int g = 0; g < MG; ++g) v[g] += dpp(v[g], integral_constant<int, 0x141>{});
#pragma unroll
        for (int g = 0; g < MG; ++g) v[g] += dpp(v[g], integral_constant<int, 0x140>{});
#pragma unroll
        for (int g = 0; g < MG; ++g)
            v[g] = (lane_of(v[g], 0) + lane_of(v[g], 16)) + (lane_of(v[g], 32) + lane_of(v[g], 48));
    };
    auto best2 = [](float p, float q, bool neg) { return neg ? __builtin_fminf(p, q) : __builtin_fmaxf(p, q); };
    auto wave_best = [&](float (&v)[MG], bool neg) {
#pragma unroll
        for (int g = 0; g < MG; ++g) v[g] = best2(v[g], dpp(v[g], integral_constant<int, 0xB1>{}), neg);
#pragma unroll
        for (int g = 0; g < MG; ++g) v[g] = best2(v[g], dpp(v[g], integral_constant<int, 0x4E>{}), neg);
#pragma unroll
        for (int g = 0; g < MG; ++g) v[g] = best2(v[g], dpp(v[g], integral_constant<int, 0x141>{}), neg);
#pragma unroll
        for (int g = 0; g < MG; ++g) v[g] = best2(v[g], dpp(v[g], integral_constant<int, 0x140>{}), neg);
#pragma unroll
        for (int g = 0; g < MG; ++g)
            v[g] = best2(best2(lane_of(v[g], 0), lane_of(v[g], 16), neg), best2(lane_of(v[g], 32), lane_of(v[g], 48), neg), neg);
    };
    const size_t plane = (size_t)a.Co * a.Ho * a.Wo;
    float *out = a.out + (size_t)px.b * a.M * plane + px.out_off;
    // which form each instance of this wave takes (wave-uniform): bit g of `wide` set -> term by term
    // (wide_finite: range beyond the product form's on its own, but finite - decided below, once the pixel is known)
    unsigned wide = a.finite_eps ? 0u : 0xffffu, wide_finite = 0u;
    if (a.finite_eps) {
        for (int m = m_first; m < m_end; ++m) {
            const float rg = a.orng[row0 + m];
            if (!(rg <= kProductRange))
                (rg < INFINITY ? wide_finite : wide) |= 1u << (m - m_first);
        }
    }
    // scaled patch values, their maximum and exponentials (finite epsilon)
    float ex[KL];
    float mp = -INFINITY;
#pragma unroll
    for (int j = 0; j < KL; ++j) {
        x[j] *= a.scale;
        if (kv[j])
            mp = fmaxf(mp, x[j]);
    }
    if (a.finite_eps) {
        float mpv[MG] = {mp, mp, mp, mp};
        wave_best(mpv, false);
        mp = mpv[0];
        if (wide_finite != 0u) {
            // the largest term of sum_k exp2(x_k - max x) exp2(o_k - max o) is at least exp2(-range) of either factor:
            // a pixel whose patch spans at most kProductRange keeps the product form whatever the offsets' range
            float mn = INFINITY;
#pragma unroll
            for (int j = 0; j < KL; ++j)
                if (kv[j])
                    mn = fminf(mn, x[j]);
            float mnv[MG] = {mn, mn, mn, mn};
            wave_best(mnv, true);
            if (!(mp - mnv[0] <= kProductRange))
                wide |= wide_finite;
        }
        const float m_sub = mp == -INFINITY ? 0.0f : mp;
#pragma unroll
        for (int j = 0; j < KL; ++j)
            ex[j] = kv[j] ? __builtin_amdgcn_exp2f(x[j] - m_sub) : 0.0f;
    }
    const float mpt = (mp - mp) + mp;  // an infinite pixel bound makes the result NaN, as the reference's exp(inf - inf) does
    for (int m0 = m_first; m0 < m_end; m0 += MG) {
        float o[MG][KL];
#pragma unroll
        for (int g = 0; g < MG; ++g)
#pragma unroll
            for (int j = 0; j < KL; ++j)
                o[g][j] = on[g][j];
        if (m0 + MG < m_end)
            fetch_rows(m0 + MG);
        const unsigned wide4 = (wide >> (m0 - m_first)) & 0xfu;
        float res[MG];
        if (wide4 != 0xfu) {
            float sum[MG];
#pragma unroll
            for (int g = 0; g < MG; ++g) {
                sum[g] = 0.0f;
#pragma unroll
                for (int j = 0; j < KL; ++j)
                    sum[g] = __builtin_fmaf(ex[j], kv[j] ? o[g][j] : 0.0f, sum[g]);
            }
            wave_sum(sum);
#pragma unroll
            for (int g = 0; g < MG; ++g)
                res[g] = (__builtin_amdgcn_logf(sum[g]) + (mpt + (a.omax[row0 + min(m0 + g, a.M - 1)] + a.c0))) *
                         a.ln2_over_eps;
        }
        if (wide4 != 0) {
            float best[MG], v[MG][KL];
#pragma unroll
            for (int g = 0; g < MG; ++g) {
                best[g] = NEG ? INFINITY : -INFINITY;
                const float *prow = a.offp + (row0 + min(m0 + g, a.M - 1)) * a.K;   // the plain (scaled) row
#pragma unroll
                for (int j = 0; j < KL; ++j) {
                    v[g][j] = x[j] + (a.finite_eps ? prow[kv[j] ? lane + 64 * j : 0] : o[g][j]);   // patch + offset
                    if (kv[j])
                        best[g] = NEG ? __builtin_fminf(best[g], v[g][j]) : __builtin_fmaxf(best[g], v[g][j]);
                }
            }
            wave_best(best, NEG);
            float sum[MG];
            if (a.finite_eps) {
#pragma unroll
                for (int g = 0; g < MG; ++g) {
                    sum[g] = 0.0f;
#pragma unroll
                    for (int j = 0; j < KL; ++j)
                        if (kv[j])
                            sum[g] += __builtin_amdgcn_exp2f(v[g][j] - best[g]);
                }
                wave_sum(sum);
            }
#pragma unroll
            for (int g = 0; g < MG; ++g)
                if ((wide4 >> g) & 1u)
                    // (an infinite extreme value makes the finite-epsilon result NaN, as the reference's exp(inf - inf) does)
                    res[g] = a.finite_eps ? (__builtin_amdgcn_logf(sum[g]) + ((best[g] - best[g]) + best[g] + a.c0)) * a.ln2_over_eps
                                          : best[g];
        }
        if (lane == 0) {
#pragma unroll
            for (int g = 0; g < MG; ++g)
                if (m0 + g < m_end)
                    out[(size_t)(m0 + g) * plane] = res[g];
        }
    }
}

template <int KL>
hipError_t launch_small(const MexKernelArgs &a, dim3 grid, bool neg, hipStream_t s)
{
    if (neg)
        hipLaunchKernelGGL((mex_small_kernel<KL, true>), grid, dim3(256), 0, s, a);
    else
        hipLaunchKernelGGL((mex_small_kernel<KL, false>), grid, dim3(256), 0, s, a);
    return hipGetLastError();
}

// the wave-per-pixel kernel pays when the tiled one would not even give every CU a workgroup
bool mex_use_small(const MexPlan &p)
{
    const long long slots = (long long)p.B * p.d.region_size;
    const long long tiled_waves = p.d.num_regions * ((slots + 63) / 64) * ((p.d.M + MX - 1) / MX);
    return p.d.K >= 64 && p.d.K <= 64 * 16 && tiled_waves < 256 && (long long)p.d.num_regions * slots < (1LL << 31);
}

struct MexTiling {
    int px, ks, kc, tm, n_mgroups;
};

// Pixels per lane and K-split: the largest register tile that still gives every SIMD about four
// waves (a wave issues at most one VALU instruction per 4 cycles, a SIMD retires one per 2, so it
// takes several resident waves to keep it busy across LDS waits); when even one pixel per lane
// leaves SIMDs idle and K is long, the waves split K instead.
MexTiling mex_tiling(const MexPlan &p)
{
    const long long slots = (long long)p.B * p.d.region_size;
    const long long mtiles = (p.d.M + MX - 1) / MX;
    auto waves = [&](int px) { return p.d.num_regions * ((slots + 64 * px - 1) / (64 * px)) * mtiles; };
    MexTiling t;
    if (mex_panel_geometry(p)) {
        // the panel kernel's packing: 64 instances per group; its fallback for unaligned inputs is the plain tiling
        t.px = 1; t.ks = 1;
        t.kc = p.d.K >= 128 ? 128 : (p.d.K >= 64 ? 64 : kChunkMin);
        t.tm = 4 * MX;
        t.n_mgroups = (p.d.M + t.tm - 1) / t.tm;
        return t;
    }
    // two pixels per lane at most: with four the kernel holds 220 VGPRs, one workgroup per compute unit, and every
    // dependent phase (gather, barrier, matrix loop, stores) shows (32x16x16 -> 64 at batch 4096: 0.229 ms with four,
    // 0.150 ms with two)
    t.px = 2;
    while (t.px > 1 && waves(t.px) < SIMNETS_MEX_WAVES)
        t.px >>= 1;
    t.ks = 1;
    if (t.px == 1) {
        if (waves(1) < 1024 && p.d.K >= 4 * 16)
            t.ks = 4;
        else if (waves(1) < 2048 && p.d.K >= 2 * 16)
            t.ks = 2;
    }
    t.kc = kChunkMin;
    if (t.px == 1)
        t.kc = p.d.K >= 128 ? 128 : (p.d.K >= 64 ? 64 : kChunkMin);
    t.tm = (4 / t.ks) * MX;
    t.n_mgroups = (p.d.M + t.tm - 1) / t.tm;
    return t;
}

}  // namespace

size_t mex_packed_bytes(const MexPlan &p, int tm, int n_mgroups)
{
    const size_t packed = align_up((size_t)p.d.num_regions * n_mgroups * p.d.K * tm * sizeof(float), 256);
    const size_t rows = align_up((size_t)p.d.num_regions * n_mgroups * tm * sizeof(float), 256);
    // scaled offsets, their exponentials; row maxima, row ranges; patch element table
    return 2 * packed + 2 * rows + align_up((size_t)p.d.K * sizeof(int4), 256);
}

size_t mex_grad_pack_bytes(const MexPlan &p)
{
    if (!std::isfinite(p.epsilon))
        return 0;   // those gradient kernels read the offsets as they are
    const size_t rmk = (size_t)p.d.num_regions * p.d.M * p.d.K * sizeof(float);
    return (mex_grads_read_packed(p) ? mex_packed_bytes(p, kGradPackTm, (p.d.M + kGradPackTm - 1) / kGradPackTm) : 0) +
           (p.normalize_offsets ? align_up(rmk, 256) : 0);
}

void mex_grad_pack_layout(const MexPlan &p, void *buffer, MexPackTwin *tw, float **normalized)
{
    const simnets_mex_dims &d = p.d;
    char *ws = reinterpret_cast<char *>(buffer);
    if (!mex_grads_read_packed(p)) {
        // only the normalised copy
        *tw = MexPackTwin{nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0};
        *normalized = p.normalize_offsets ? reinterpret_cast<float *>(ws) : nullptr;
        return;
    }
    tw->tm = kGradPackTm;
    tw->n_mgroups = (d.M + kGradPackTm - 1) / kGradPackTm;
    const long long rows = (long long)d.num_regions * tw->n_mgroups * tw->tm;
    const size_t packed = align_up((size_t)rows * d.K * sizeof(float), 256);
    const size_t row_bytes = align_up((size_t)rows * sizeof(float), 256);
    tw->offp = reinterpret_cast<float *>(ws);
    tw->offe = reinterpret_cast<float *>(ws + packed);
    tw->omax = reinterpret_cast<float *>(ws + 2 * packed);
    tw->orng = reinterpret_cast<float *>(ws + 2 * packed + row_bytes);
    tw->ktab = reinterpret_cast<int4 *>(ws + 2 * packed + 2 * row_bytes);
    *normalized = p.normalize_offsets
                      ? reinterpret_cast<float *>(ws + mex_packed_bytes(p, tw->tm, tw->n_mgroups)) : nullptr;
}

int mex_pack_offsets(const MexPlan &p, const float *offsets, int tm, int n_mgroups, void *workspace, MexKernelArgs *a,
                     void *stream, const SimPackJob *job, bool launch, float *normalized_out, bool for_gradients)
{
    const simnets_mex_dims &d = p.d;
    const long long rows = (long long)d.num_regions * n_mgroups * tm;
    const size_t packed = align_up((size_t)rows * d.K * sizeof(float), 256);
    const size_t row_bytes = align_up((size_t)rows * sizeof(float), 256);
    char *ws = reinterpret_cast<char *>(workspace);
    float *offp = reinterpret_cast<float *>(ws);
    float *offe = reinterpret_cast<float *>(ws + packed);
    float *omax = reinterpret_cast<float *>(ws + 2 * packed);
    float *orng = reinterpret_cast<float *>(ws + 2 * packed + row_bytes);
    int4 *ktab = reinterpret_cast<int4 *>(ws + 2 * packed + 2 * row_bytes);
    if ((long long)d.block_c * p.H * p.W > 0x7fffffffLL)
        return SIMNETS_ERR_TOO_LARGE;  // the table holds 32-bit offsets
    a->offp = offp; a->offe = offe; a->omax = omax; a->orng = orng; a->ktab = ktab;
    a->n_mgroups = n_mgroups;
    if (!launch)
        return SIMNETS_OK;  // the arrays are in place already: only the pointers were wanted
    // a forward call that keeps the gradient kernels' layout as well: the same launch writes it
    MexPackTwin tw = {nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0};
    long long waves = rows;
    if (p.grad_pack != nullptr && normalized_out == nullptr && mex_grad_pack_bytes(p) > 0) {
        mex_grad_pack_layout(p, p.grad_pack->buffer, &tw, &normalized_out);
        waves = (long long)d.num_regions * std::max(n_mgroups * tm, tw.n_mgroups * tw.tm);
        p.grad_pack->written = true;
    }
    const int row_blocks = (int)((waves + 3) / 4);
    SimPackJob pj = {nullptr, nullptr, nullptr, nullptr, 0, 0, 0, 0.0f};
    int extra = 0;
    if (job) {
        pj = *job;
        extra = (int)std::min<long long>(((long long)((pj.O + 31) & ~31) * pj.K + 255) / 256, 64);
    }
    const dim3 grid((unsigned)(row_blocks + extra));
    hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
#define SIMNETS_PACK_LAUNCH(KL)                                                                                        \
    hipLaunchKernelGGL(mex_pack_offsets_kernel<KL>, grid, dim3(256), 0, hs, offsets, d.num_regions, d.M, d.K, n_mgroups, \
                       tm, p.normalize_offsets, a->scale, a->finite_eps, offp, offe, omax, orng, ktab, p.H, p.W,         \
                       d.block_h, d.block_w, row_blocks, pj, normalized_out, tw, for_gradients ? 1 : 0)
    if (d.K <= 64)
        SIMNETS_PACK_LAUNCH(1);
    else if (d.K <= 256)
        SIMNETS_PACK_LAUNCH(4);
    else if (d.K <= 1024)
        SIMNETS_PACK_LAUNCH(16);
    else
        SIMNETS_PACK_LAUNCH(0);
#undef SIMNETS_PACK_LAUNCH
    if (launch && hipGetLastError() != hipSuccess)
        return SIMNETS_ERR_HIP;
    return SIMNETS_OK;
}

size_t mex_workspace_bytes(const MexPlan &p)
{
    if (mex_use_small(p))
        return mex_packed_bytes(p, 1, p.d.M);
    const MexTiling t = mex_tiling(p);
    return mex_packed_bytes(p, t.tm, t.n_mgroups);
}

// phase: kMexPrepare = only the launch that depends on the offsets alone (packing), kMexRun = only the launches
// that read the packed workspace, both = the whole call.
int mex_launch(const MexPlan &p, const float *input, const float *offsets, float *output, void *workspace,
               size_t workspace_bytes, void *stream, int phase)
{
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const simnets_mex_dims &d = p.d;
    if (workspace_bytes < mex_workspace_bytes(p))
        return SIMNETS_ERR_WORKSPACE;
    const bool pack = (phase & kMexPrepare) != 0;
    if (mex_use_small(p)) {
        MexKernelArgs a = mex_kernel_args(p);
        const int rc = mex_pack_offsets(p, offsets, 1, d.M, workspace, &a, stream, nullptr, pack);
        if (rc || !(phase & kMexRun))
            return rc;
        a.in = input; a.out = output;
        const long long waves = (long long)d.num_regions * a.slots;
        dim3 grid((unsigned)((waves + 3) / 4), (unsigned)((d.M + kSmallMChunk - 1) / kSmallMChunk));
        if (grid.y > 65535)
            return SIMNETS_ERR_TOO_LARGE;
        const bool neg = !a.finite_eps && p.epsilon < 0;
        const int kl = (d.K + 63) / 64;
        hipError_t e;
        if (kl <= 2)
            e = launch_small<2>(a, grid, neg, s);
        else if (kl <= 4)
            e = launch_small<4>(a, grid, neg, s);
        else if (kl <= 8)
            e = launch_small<8>(a, grid, neg, s);
        else
            e = launch_small<16>(a, grid, neg, s);
        return e == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
    }
    const MexTiling t = mex_tiling(p);
    MexKernelArgs a = mex_kernel_args(p);
    if (pack && (phase & kMexRun) && mex_panel_geometry(p)) {
        // a whole self-packing call of a small single-chunk layer: one launch that packs inside its workgroups
        a.n_mgroups = t.n_mgroups;
        const int src = mex_panel_launch_selfpack(p, a, input, offsets, output, stream);
        if (src != SIMNETS_PANEL_NOT_TAKEN)
            return src;
    }
    const int rc = mex_pack_offsets(p, offsets, t.tm, t.n_mgroups, workspace, &a, stream, nullptr, pack);
    if (rc || !(phase & kMexRun))
        return rc;
    if (mex_panel_geometry(p)) {
        const int prc = mex_panel_launch(p, a, input, output, stream);
        if (prc != SIMNETS_PANEL_NOT_TAKEN)
            return prc;
    }
    a.in = input; a.out = output;
    a.kgather = t.px == 1 && t.ks >= 2 && d.region_size == 1;

    // bounds checks are needed unless every patch lies inside the image
    const bool inside = d.pad_c == 0 && d.pad_h == 0 && d.pad_w == 0 &&
                        (d.channels_out - 1) * d.stride_c + d.block_c <= p.C &&
                        (d.height_out - 1) * d.stride_h + d.block_h <= p.H &&
                        (d.width_out - 1) * d.stride_w + d.block_w <= p.W;
    a.cpr = (a.slots + 64 * t.px - 1) / (64 * t.px);
    const long long supers = (a.cpr + kXcds - 1) / kXcds;
    const long long gx = supers * kXcds * d.num_regions;
    if (gx > 0x7fffffffLL || t.n_mgroups > 65535)
        return SIMNETS_ERR_TOO_LARGE;
    dim3 grid((unsigned)gx, (unsigned)t.n_mgroups);
    // finite eps: values are pre-multiplied by eps*log2(e), so the shift is always the maximum
    const int eps = a.finite_eps ? 0 : p.epsilon < 0 ? -1 : 1;
    hipError_t e;
    if (t.px == 2)
        e = launch_variant<2, 1, kChunkMin>(a, grid, eps, inside, s);
    else if (t.ks == 1)
        e = launch_px1<1>(a, grid, eps, inside, t.kc, s);
    else if (t.ks == 2)
        e = launch_px1<2>(a, grid, eps, inside, t.kc, s);
    else
        e = launch_px1<4>(a, grid, eps, inside, t.kc, s);
    return e == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

namespace {
// I: index type (int while the element count fits: 64-bit divisions cost several times the rest of the kernel)
template <typename I>
__global__ void sum_pool_kernel(const float *__restrict__ in, float *__restrict__ out, I total, int H, int W, int Ho,
                                int Wo, int ph, int pw)
{
    for (I idx = (I)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (I)gridDim.x * blockDim.x) {
        const I wo = idx % Wo;
        const I t = idx / Wo;
        const I ho = t % Ho;
        const I bc = t / Ho;
        const float *src = in + ((size_t)bc * H + (size_t)ho * ph) * W + (size_t)wo * pw;
        float acc = 0.0f;
        for (int i = 0; i < ph; ++i)
            for (int j = 0; j < pw; ++j)
                acc += src[(size_t)i * W + j];
        out[idx] = acc;
    }
}

// 2x2 windows on maps whose width is a multiple of 4 (16-byte aligned tensors, fewer than 2^31 elements): a thread
// takes two neighbouring windows - one 16-byte load per input row, one 8-byte store - and the row index comes from
// a multiply-high instead of divisions.  Same order of additions as the kernel above.
__global__ __launch_bounds__(256) void sum_pool_2x2_kernel(const float4 *__restrict__ in, float2 *__restrict__ out,
                                                          unsigned pairs, unsigned W4, FastDiv dW4)
{
    const unsigned idx = blockIdx.x * 256u + threadIdx.x;   // (image-channel-output row, pair of windows)
    if (idx >= pairs)
        return;
    const unsigned row = fast_div(idx, dW4);                // output row over all images and channels
    const unsigned c = idx - row * W4;
    const float4 a = in[(size_t)(2 * row) * W4 + c], b = in[(size_t)(2 * row + 1) * W4 + c];
    float2 r;
    r.x = (((0.0f + a.x) + a.y) + b.x) + b.y;
    r.y = (((0.0f + a.z) + a.w) + b.z) + b.w;
    out[idx] = r;
}

// gradient of the sum pooling: every input element of a window receives the window's gradient, the elements
// of a dropped trailing row or column receive 0
template <typename I>
__global__ void sum_pool_grad_kernel(const float *__restrict__ gout, float *__restrict__ gin, I total, int H, int W,
                                     int Ho, int Wo, int ph, int pw)
{
    for (I idx = (I)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (I)gridDim.x * blockDim.x) {
        const I w = idx % W;
        const I t = idx / W;
        const I h = t % H;
        const I bc = t / H;
        const I ho = h / ph, wo = w / pw;
        gin[idx] = (ho < Ho && wo < Wo) ? gout[((size_t)bc * Ho + ho) * Wo + wo] : 0.0f;
    }
}

// ... and of the 2x2 case above: a thread reads the gradients of two neighbouring windows and writes their four input
// elements of both rows
__global__ __launch_bounds__(256) void sum_pool_grad_2x2_kernel(const float2 *__restrict__ gout, float4 *__restrict__ gin,
                                                               unsigned pairs, unsigned W4, FastDiv dW4)
{
    const unsigned idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= pairs)
        return;
    const unsigned row = fast_div(idx, dW4);
    const unsigned c = idx - row * W4;
    const float2 g = gout[idx];
    const float4 v = make_float4(g.x, g.x, g.y, g.y);
    gin[(size_t)(2 * row) * W4 + c] = v;
    gin[(size_t)(2 * row + 1) * W4 + c] = v;
}

// the 2x2 kernels' case: even height, width a multiple of 4, 16-byte aligned tensors, 32-bit element counts
bool pool_2x2_fast(long long planes, int H, int W, int ph, int pw, const void *full, const void *pooled)
{
    return ph == 2 && pw == 2 && H % 2 == 0 && W % 4 == 0 && planes * H * W < 0x7fffffffLL &&
           reinterpret_cast<uintptr_t>(full) % 16 == 0 && reinterpret_cast<uintptr_t>(pooled) % 8 == 0;
}
}  // namespace

int sum_pool_grad_launch(int B, int C, int H, int W, int ph, int pw, const float *output_grad, float *input_grad,
                         void *stream)
{
    const long long total = (long long)B * C * H * W;
    if (total == 0)
        return SIMNETS_OK;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (pool_2x2_fast((long long)B * C, H, W, ph, pw, input_grad, output_grad)) {
        const unsigned pairs = (unsigned)(total / 8), W4 = (unsigned)(W / 4);
        hipLaunchKernelGGL(sum_pool_grad_2x2_kernel, dim3((pairs + 255) / 256), dim3(256), 0, s,
                           reinterpret_cast<const float2 *>(output_grad), reinterpret_cast<float4 *>(input_grad), pairs, W4,
                           make_fast_div(W4));
        return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
    }
    const int blocks = (int)std::min<long long>((total + 255) / 256, 1 << 20);
    if (total + 256LL * blocks < 0x7fffffffLL)
        hipLaunchKernelGGL(sum_pool_grad_kernel<int>, dim3(blocks), dim3(256), 0, s, output_grad, input_grad, (int)total,
                           H, W, H / ph, W / pw, ph, pw);
    else
        hipLaunchKernelGGL(sum_pool_grad_kernel<long long>, dim3(blocks), dim3(256), 0, s, output_grad, input_grad,
                           total, H, W, H / ph, W / pw, ph, pw);
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

int sum_pool_launch(int B, int C, int H, int W, int ph, int pw, const float *input, float *output, void *stream)
{
    const int Ho = H / ph, Wo = W / pw;
    const long long total = (long long)B * C * Ho * Wo;
    if (total == 0)
        return SIMNETS_OK;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (pool_2x2_fast((long long)B * C, H, W, ph, pw, input, output)) {
        const unsigned pairs = (unsigned)(total / 2), W4 = (unsigned)(W / 4);
        hipLaunchKernelGGL(sum_pool_2x2_kernel, dim3((pairs + 255) / 256), dim3(256), 0, s,
                           reinterpret_cast<const float4 *>(input), reinterpret_cast<float2 *>(output), pairs, W4,
                           make_fast_div(W4));
        return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
    }
    const int blocks = (int)std::min<long long>((total + 255) / 256, 1 << 20);
    if (total + 256LL * blocks < 0x7fffffffLL)
        hipLaunchKernelGGL(sum_pool_kernel<int>, dim3(blocks), dim3(256), 0, s, input, output, (int)total, H, W, Ho, Wo,
                           ph, pw);
    else
        hipLaunchKernelGGL(sum_pool_kernel<long long>, dim3(blocks), dim3(256), 0, s, input, output, total, H, W, Ho,
                           Wo, ph, pw);
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

}  // namespace simnets
