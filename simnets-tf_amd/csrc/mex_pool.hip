// MEX forward fused with the non-overlapping sum pooling that follows it in the reference's networks
// (README.md:108-129, examples/mnist_ght_model_missing_data.py:60-66: MEX with unshared offset regions of the
// pooling window's size, then AveragePooling2D * window area).
//
// With unshared regions [1, ph, pw] the pixels of one pooling window are one pixel of each of the ph*pw regions,
// and they carry the same slot number inside their regions (include/utils/mex_utils.hpp:69-116).  A workgroup
// therefore takes 16 (or 32) slots of ALL regions and 64 instances: the MEX values of a window end up in one
// lane and are added there, in the window's row-major order (the order sum pooling uses), and only the pooled
// tensor is written: a quarter of the MEX output, and no pooling launch.
//
// Arithmetic as in the tiled forward kernel (finite epsilon): product form on the fp32 matrix cores,
//   S[instance][pixel] = sum_k exp2(o_k - max o) * exp2(x_k - max x)   (v_mfma_f32_16x16x4_f32),
// per 16-pixel tile with the offsets tile of that tile's region; workgroups whose offsets span too wide a range
// for the product form evaluate a max-tracked log-sum-exp on the VALU from the same LDS tiles instead (lse_chunk).
#include <hip/hip_runtime.h>

#include <cmath>

#include "internal.h"
#include "mex_common.h"
#include "sim_step.h"

namespace simnets {

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int KC = 32;             // k per LDS chunk
constexpr int TM = 64, MX = 16;    // instances per workgroup / per wave
constexpr int KSTEP = 4, U = KC / KSTEP;

constexpr int kSimTaps = 16;       // longest Similarity patch the kernel evaluates inside its staging

struct PoolArgs {
    float *pooled;
    float *full;  // not null: the MEX values before pooling are stored there as well, [B][M * Co][Ho][Wo]
    int full_pairs, out_pairs;  // `full` / the unpooled output of the panel form may be stored 8 bytes at a time
                                // (aligned, even row length: the two regions of a window row are one float2)
    int Hp, Wp;   // pooled height and width
    int spw;      // slots per workgroup: NH * 64 / R
    // SIMF: the MEX input is the output of a Similarity layer that is evaluated on the fly
    const float *sx;        // its input [B][sC][sH][sW]
    const float *spa, *spc; // packed parameters [O][sK] (pairs) and [O][sK] (sim_pack_element)
    int sC, sH, sW, sbh, sbw, ssh, ssw, sph, spw_, sK, smode;
    float soob, snorm;      // out-of-bounds value; -0.5 K log(2 pi) of the normalized mode
    int snorm_every, sB;    // reproduce the reference's per-iteration addition of that constant
};

// Offsets too far apart for the product form: max-tracked ("online") log-sum-exp at chunk granularity on the VALU, on
// the same LDS tiles and the same lane layout as the matrix form - lane (lr, lq) owns column lr of each of the four
// 16-column tiles of its column half and instances 4*lq + v of its wave.  xs holds the scaled patch values of the
// chunk ([k][column]), os the scaled offsets ([region][k][instance], not their exponentials); tile t belongs to
// region t % R.  Per chunk: the maximum of patch + offset over the chunk's k, then the running sums are rescaled to the
// new running maximum and the chunk's exponentials added - one exponential per term and one per output and chunk,
// the tiles read twice from LDS and nothing again from memory.  SWZ: the panel kernel's swizzled tiles.
template <int R, int XP, bool SWZ>
__device__ __forceinline__ void lse_chunk(float (&best)[4][4], float (&sum)[4][4], const float *xs, const float *os,
                                          int colbase, int wm, int lr, int lq, int kc)
{
    // (one tile at a time: four running pairs' worth of temporaries, so that this path stays inside the register
    // budget of the matrix form, whose occupancy the whole kernel's allocation decides)
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        auto fetch = [&](int kk, float &x, float4 &o) {
            const int sx = SWZ ? (((kk & 3) << 4) | (((kk >> 2) & 3) << 2)) : 0;
            const int so = SWZ ? ((kk & 3) << 4) : 0;
            x = xs[kk * XP + ((colbase + t * 16 + lr) ^ sx)];
            o = *reinterpret_cast<const float4 *>(os + (t % R) * KC * TM + kk * TM + ((wm * MX + 4 * lq) ^ so));
        };
        float cb[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll 2
        for (int kk = 0; kk < kc; ++kk) {
            float x;
            float4 o;
            fetch(kk, x, o);
            cb[0] = fmaxf(cb[0], x + o.x); cb[1] = fmaxf(cb[1], x + o.y);
            cb[2] = fmaxf(cb[2], x + o.z); cb[3] = fmaxf(cb[3], x + o.w);
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float bo = best[t][v];
            const float nb = fmaxf(bo, cb[v]);
            // (a maximum that did not move: factor 1, which also keeps -inf - -inf out of the exponent)
            sum[t][v] *= bo == nb ? 1.0f : __builtin_amdgcn_exp2f(bo - nb);
            best[t][v] = nb;
            cb[v] = nb == -INFINITY ? 0.0f : nb;   // what the chunk's terms subtract
        }
#pragma unroll 2
        for (int kk = 0; kk < kc; ++kk) {
            float x;
            float4 o;
            fetch(kk, x, o);
            sum[t][0] += __builtin_amdgcn_exp2f(x + o.x - cb[0]);
            sum[t][1] += __builtin_amdgcn_exp2f(x + o.y - cb[1]);
            sum[t][2] += __builtin_amdgcn_exp2f(x + o.z - cb[2]);
            sum[t][3] += __builtin_amdgcn_exp2f(x + o.w - cb[3]);
        }
    }
}

// Infinite epsilon on the panel kernel's tiles: the maximum of patch + offset alone (the caller stages negated values
// for the minimum).  Same lane layout as above.  The 16 offsets the 16 lanes of a row need per k - instances
// 4*lq + v of the four regions - are fetched one per lane (lane lr: region lr / 4, v = lr % 4) and reach the others
// through the add's row broadcast, so a k costs five 4-byte LDS reads per lane; two k per step, a term is an add and
// half a three-operand maximum.  os: [region][k][position], position = ((instance ^ (k & 3) << 4) + 16 * region) % 64
// (the rotation by the region keeps the four regions' reads of one instruction in different banks).
template <int XP>
__device__ __forceinline__ void max_chunk(float (&best)[4][4], const float *xs, const float *os, int colbase, int wm,
                                          int lr, int lq)
{
    auto bcast = [](float v, auto n) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v),
                                                                     0x150 + decltype(n)::value, 0xF, 0xF, true));
    };
    const int ot = lr >> 2;
    const float *op = os + ot * KC * TM;
    const int oi = wm * MX + 4 * lq + (lr & 3);
    // the operands of two k: x[h][tile], o[h]
    auto fetch = [&](int kk, float (&x)[2][4], float (&o)[2]) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = kk + h;
            const int sx = ((k & 3) << 4) | (((k >> 2) & 3) << 2);
            o[h] = op[k * TM + (((oi ^ ((k & 3) << 4)) + 16 * ot) & 63)];
#pragma unroll
            for (int t = 0; t < 4; ++t)
                x[h][t] = xs[k * XP + ((colbase + t * 16 + lr) ^ sx)];
        }
    };
#define SIMNETS_MAX_TERM(x, o, t, v)                                                                            \
    best[t][v] = __builtin_fmaxf(                                                                               \
        __builtin_fmaxf(best[t][v], x[0][t] + bcast(o[0], std::integral_constant<int, 4 * (t) + (v)>{})),      \
        x[1][t] + bcast(o[1], std::integral_constant<int, 4 * (t) + (v)>{}));
#define SIMNETS_MAX_TILE(x, o, t) \
    SIMNETS_MAX_TERM(x, o, t, 0) SIMNETS_MAX_TERM(x, o, t, 1) SIMNETS_MAX_TERM(x, o, t, 2) SIMNETS_MAX_TERM(x, o, t, 3)
#define SIMNETS_MAX_STEP(x, o) \
    SIMNETS_MAX_TILE(x, o, 0) SIMNETS_MAX_TILE(x, o, 1) SIMNETS_MAX_TILE(x, o, 2) SIMNETS_MAX_TILE(x, o, 3)
    // two register sets: the reads of the next step are on their way while a step's 48 instructions issue
    float xa[2][4], oa[2], xb[2][4], ob[2];
    fetch(0, xa, oa);
#pragma nounroll
    for (int kk = 0; kk < KC; kk += 4) {
        fetch(kk + 2, xb, ob);
        __builtin_amdgcn_sched_barrier(0);
        SIMNETS_MAX_STEP(xa, oa)
        __builtin_amdgcn_sched_barrier(0);
        fetch(kk + 4 < KC ? kk + 4 : 0, xa, oa);   // (the last round reads the first step again, unused)
        __builtin_amdgcn_sched_barrier(0);
        SIMNETS_MAX_STEP(xb, ob)
        __builtin_amdgcn_sched_barrier(0);
    }
#undef SIMNETS_MAX_STEP
#undef SIMNETS_MAX_TILE
#undef SIMNETS_MAX_TERM
}

// NH = column halves of a workgroup (64 pixel columns = 4 tiles of 16 each), 4 instance waves per half: two halves
// share the offsets tiles and double the waves per SIMD the LDS budget allows, which is what hides the latencies of
// the short dependent phases; one half only when there are no slots for a second one.
// SIMF: the input of the MEX layer is a Similarity layer's output whose channels are exactly the MEX patch (blocks
// [O, 1, 1], no padding): the staging evaluates Similarity channel k of its pixel from the layer's input (the patch
// taps of the pixel sit in LDS, the packed parameters of channel k come through scalar loads) with the Similarity
// kernel's own combine step in the same order, so the value is the one that kernel would have stored, and neither
// that tensor nor its launches exist.
template <int R, int NH, bool CHECK, bool SIMF>
__global__ __launch_bounds__(256 * NH) void mex_pool_kernel(const MexKernelArgs a, const PoolArgs q)
{
    constexpr int XP = 64 * NH;         // pixel columns of a workgroup
    constexpr int kThreads = 256 * NH;
    constexpr int G = 4 / R;       // slot groups of 16 per column half
    __shared__ __attribute__((aligned(16))) float xs[KC * XP];       // [k][column]
    __shared__ __attribute__((aligned(16))) float os[R * KC * TM];   // [region][k][instance]
    __shared__ float pmx[KSTEP * XP];   // partial column maxima
    __shared__ float fsh[XP], msh[XP];  // per column: rescale factor of this chunk, running maximum
    __shared__ long long ppos[16 * G * NH];  // per slot: where instance 0 goes in the pooled tensor, -1 = no window
    __shared__ float xt[SIMF ? kSimTaps * XP : 1];  // SIMF: Similarity patch taps of the columns, [tap][column]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 3, wh = wave >> 2;      // computing: instance group and column half of this wave
    const int sk = wave / NH, sh = wave % NH;     // staging: k phase and column half of this wave
    const int chunk = blockIdx.x, mgroup = blockIdx.y;
    const int m0 = mgroup * TM + wm * MX;
    const bool wave_active = m0 < a.M;

    // staging role: column of tile (slot group, region), consecutive threads = neighbouring pixels of a window row
    const int sreg = lane % R, ssl = lane / R;
    const int col = sh * 64 + ((ssl >> 4) * R + sreg) * 16 + (ssl & 15);
    const PixelRef gp = locate(a, sreg, (chunk * NH + sh) * (16 * G) + ssl);

    if (tid < 16 * G * NH) {
        const int slot = chunk * (16 * G * NH) + tid;
        long long pos = -1;
        if (slot < a.slots) {
            const int b = (int)fast_div((unsigned)slot, a.dRS);
            const int sq = slot - b * a.RS;
            const int qw = (int)fast_div((unsigned)sq, a.dWs);
            const int i = sq - qw * a.Ws;
            const int l = (int)fast_div((unsigned)sq, a.dWsHs);
            const int j = qw - l * a.Hs;
            if (l < a.Co && j < q.Hp && i < q.Wp)
                pos = ((long long)b * a.M * a.Co + l) * ((long long)q.Hp * q.Wp) + (long long)j * q.Wp + i;
        }
        ppos[tid] = pos;
    }

    bool prod = true;
    float m_run = -INFINITY;  // running maximum of this thread's staging column

    // patch elements k0 + sk + 4u of this thread's column (Similarity channels when SIMF): loads issued, not awaited
    auto gather = [&](int k0, int kc, float (&v)[U]) {
        const bool full = kc == KC;
        if (SIMF) {
            if (k0 == 0) {
                // taps of this column's Similarity patch (im2col_3d rule of that layer), once per workgroup
                const int sbhw = q.sbh * q.sbw;
                for (int j = sk; j < q.sK; j += KSTEP) {
                    const int c = j / sbhw, rem = j - c * sbhw;
                    const int hi = gp.hi0 * q.ssh - q.sph + rem / q.sbw, wi = gp.wi0 * q.ssw - q.spw_ + rem % q.sbw;
                    const bool ok = hi >= 0 && hi < q.sH && wi >= 0 && wi < q.sW;
                    xt[j * XP + col] = ok ? q.sx[(((size_t)gp.b * q.sC + c) * q.sH + hi) * q.sW + wi] : q.soob;
                }
                __syncthreads();
            }
            int reps = 0;
            if (q.smode == SIM_MODE_L2_NORM)
                reps = q.snorm_every ? q.sB - gp.b : 1;
            // this thread's 8 channels of the chunk (k0 + sk + 4u) are 8 "templates" of one pixel for the combine
            // step; their parameters for a tap are consecutive (one scalar load each for pa and pc)
            static_assert(U == 8 && KC == 32 && KSTEP == 4, "parameter layout of the Similarity evaluation");
            float acc[U][1];
#pragma unroll
            for (int u = 0; u < U; ++u)
                acc[u][0] = 0.0f;
            const float *pa = q.spa + ((size_t)(k0 / KC) * KSTEP + sk) * q.sK * (2 * U);
            const float *pc = q.spc + ((size_t)(k0 / KC) * KSTEP + sk) * q.sK * U;
            for (int j = 0; j < q.sK; ++j) {
                const float x1[1] = {xt[j * XP + col]};
                float p2[2 * U], c1[U];
#pragma unroll
                for (int i = 0; i < 2 * U; ++i)
                    p2[i] = pa[j * 2 * U + i];
#pragma unroll
                for (int i = 0; i < U; ++i)
                    c1[i] = pc[j * U + i];
                switch (q.smode) {
                case SIM_MODE_L1: sim_step<SIM_MODE_L1, 1, U, true>(acc, x1, p2, c1); break;
                case SIM_MODE_L2: sim_step<SIM_MODE_L2, 1, U, true>(acc, x1, p2, c1); break;
                case SIM_MODE_L2_NORM: sim_step<SIM_MODE_L2_NORM, 1, U, true>(acc, x1, p2, c1); break;
                default: sim_step<SIM_MODE_L2_NORM_IGNORE_NAN, 1, U, true>(acc, x1, p2, c1); break;
                }
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                float val = acc[u][0];
                for (int rr = 0; rr < reps; ++rr)
                    val += q.snorm;
                v[u] = val;
            }
        } else
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int kk = sk + u * KSTEP;
            const int4 ke = a.ktab[k0 + (full ? kk : min(kk, kc - 1))];  // same for the whole wave: scalar load
            if (CHECK) {
                const int ci = gp.ci0 + ke.y, hi = gp.hi0 + ke.z, wi = gp.wi0 + ke.w;
                const bool ok = ci >= 0 && ci < a.C && hi >= 0 && hi < a.H && wi >= 0 && wi < a.W;
                v[u] = ok ? gp.base[ke.x] : a.oob;
            } else {
                v[u] = gp.base[ke.x];
            }
        }
    };

    auto stage = [&](int k0, int kc) {
        const bool full = kc == KC;
        float v[U];
        gather(k0, kc, v);
        // offsets tiles of the R regions: straight copies of kc * TM floats each
        const int on = kc * (TM / 4);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float4 *src = reinterpret_cast<const float4 *>(
                (prod ? a.offe : a.offp) + (((size_t)r * a.n_mgroups + mgroup) * a.K + k0) * TM);
            float4 *dst = reinterpret_cast<float4 *>(os + r * KC * TM);
            for (int i = tid; i < on; i += kThreads)
                dst[i] = src[i];
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            v[u] *= a.scale;
        if (!prod) {
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (full || sk + u * KSTEP < kc)
                    xs[(sk + u * KSTEP) * XP + col] = v[u];
            return;
        }
        // column maximum over the chunk -> running maximum; the staged values become exp2(x - maximum)
        float pm = -INFINITY;
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (full || sk + u * KSTEP < kc)
                pm = fmaxf(pm, v[u]);
        pmx[sk * XP + col] = pm;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < KSTEP; ++j)
            pm = fmaxf(pm, pmx[j * XP + col]);
        const float m_new = fmaxf(m_run, pm);
        const float m_sub = m_new == -INFINITY ? 0.0f : m_new;  // nothing finite yet: the terms are exp2(-inf) = 0
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (full || sk + u * KSTEP < kc)
                xs[(sk + u * KSTEP) * XP + col] = __builtin_amdgcn_exp2f(v[u] - m_sub);
        if (sk == 0) {
            fsh[col] = m_run == m_new ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
            msh[col] = m_new;
        }
        m_run = m_new;
        if (!full) {
            // the matrix instruction takes 4 k at a time: rows kc .. next multiple of 4 are zeros
            const int kc4 = (kc + 3) & ~3;
            for (int i = tid; i < (kc4 - kc) * XP; i += kThreads)
                xs[kc * XP + i] = 0.0f;
            for (int i = tid; i < (kc4 - kc) * TM * R; i += kThreads)
                os[(i / ((kc4 - kc) * TM)) * KC * TM + kc * TM + i % ((kc4 - kc) * TM)] = 0.0f;
        }
    };

    const int lr = lane & 15, lq = lane >> 4;
    const size_t plane_p = (size_t)a.Co * q.Hp * q.Wp;
    const size_t row0 = (size_t)(m0 + 4 * lq) * plane_p;  // this lane's first instance row
    const bool all_rows = m0 + MX <= a.M;                 // same for the whole wave
    float res[4][4];  // [tile][v]: MEX value of (pixel lr of the tile, instance m0 + 4*lq + v)

    // ---- product form, software pipelined: the global loads of chunk i + 1 (patch elements and offsets tiles, into
    //      registers) are issued before the matrix loop of chunk i and written to LDS after it ----
    constexpr int TILE4 = KC * TM / 4;                       // float4 of one region's offsets tile
    constexpr int NO = (TILE4 + kThreads - 1) / kThreads;    // ... per thread
    float vn[U];
    float4 on[R * NO];
    auto issue = [&](int k0, int kc) {
        const int cnt = kc * (TM / 4);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float4 *src = reinterpret_cast<const float4 *>(
                a.offe + (((size_t)r * a.n_mgroups + mgroup) * a.K + k0) * TM);
#pragma unroll
            for (int j = 0; j < NO; ++j) {
                const int i = tid + j * kThreads;
                on[r * NO + j] = i < cnt ? src[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);  // rows past kc: zeros
            }
        }
        gather(k0, kc, vn);
    };
    // Product form or term by term: decided from the packed row ranges, after the first chunk's loads have been
    // issued (those assume the product form; a workgroup that turns out wide loads again).  Rows whose range is too
    // wide on its own but finite keep the product form when the patch of every pixel column spans at most
    // kProductRange (see there): the first chunk is in the registers, the others take a sweep of their own.
    auto decide = [&]() {
        int wide = 0, unbounded = 0;
        if (tid < TM) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const float rg = a.orng[((size_t)r * a.n_mgroups + mgroup) * TM + tid];
                wide |= !(rg <= kProductRange);
                unbounded |= !(rg < INFINITY);
            }
        }
        if (!__syncthreads_or(wide))
            return true;
        const int any_unbounded = __syncthreads_or(unbounded);
        float hi = -INFINITY, lo = INFINITY;
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (sk + u * KSTEP < a.K) {
                const float v = vn[u] * a.scale;
                hi = fmaxf(hi, v);
                lo = fminf(lo, v);
            }
        // (longer patches: one extra sweep over the remaining chunks, only in workgroups with such a row)
        for (int k0 = KC; k0 < a.K; k0 += KC) {
            const int kc = min(KC, a.K - k0);
            float v[U];
            gather(k0, kc, v);
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (sk + u * KSTEP < kc) {
                    hi = fmaxf(hi, v[u] * a.scale);
                    lo = fminf(lo, v[u] * a.scale);
                }
        }
        pmx[sk * XP + col] = hi;
        xs[sk * XP + col] = lo;   // (the tile is filled later)
        __syncthreads();
#pragma unroll
        for (int j = 0; j < KSTEP; ++j) {
            hi = fmaxf(hi, pmx[j * XP + col]);
            lo = fminf(lo, xs[j * XP + col]);
        }
        // (a column with an infinite value, or with nothing finite, is not narrow; the barrier frees the arrays again)
        return !__syncthreads_or(!(hi - lo <= kProductRange)) && !any_unbounded;
    };
    issue(0, min(KC, a.K));
    prod = decide();
    if (prod) {
        floatx4 acc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t)
            acc[t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        const float *xa = xs + lq * XP + wh * 64 + lr;
        const float *oa = os + lq * TM + wm * MX + lr;
        for (int k0 = 0; k0 < a.K; k0 += KC) {
            const int kc = min(KC, a.K - k0);
            // ---- registers -> LDS (the previous chunk's readers are behind the barrier that ended its loop) ----
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
                for (int j = 0; j < NO; ++j)
                    if (TILE4 % kThreads == 0 || tid + j * kThreads < TILE4)
                        reinterpret_cast<float4 *>(os + r * KC * TM)[tid + j * kThreads] = on[r * NO + j];
            float pm = -INFINITY;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                vn[u] *= a.scale;
                if (sk + u * KSTEP < kc)
                    pm = fmaxf(pm, vn[u]);
            }
            pmx[sk * XP + col] = pm;
            __syncthreads();
#pragma unroll
            for (int j = 0; j < KSTEP; ++j)
                pm = fmaxf(pm, pmx[j * XP + col]);
            const float m_new = fmaxf(m_run, pm);
            const float m_sub = m_new == -INFINITY ? 0.0f : m_new;  // nothing finite yet: the terms are exp2(-inf) = 0
#pragma unroll
            for (int u = 0; u < U; ++u)   // rows past kc hold zeros (the matrix instruction takes 4 k at a time)
                xs[(sk + u * KSTEP) * XP + col] = sk + u * KSTEP < kc ? __builtin_amdgcn_exp2f(vn[u] - m_sub) : 0.0f;
            if (sk == 0) {
                fsh[col] = m_run == m_new ? 1.0f : __builtin_amdgcn_exp2f(m_run - m_new);
                msh[col] = m_new;
            }
            m_run = m_new;
            __syncthreads();
            if (k0 + KC < a.K)
                issue(k0 + KC, min(KC, a.K - k0 - KC));
            if (wave_active) {
                if (k0 > 0) {
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        acc[t] *= fsh[wh * 64 + t * 16 + lr];
                }
                const int kend = (kc + 3) & ~3;
                for (int kq = 0; kq < kend; kq += 4) {
                    float av[R], bv[4];
#pragma unroll
                    for (int r = 0; r < R; ++r)
                        av[r] = oa[r * KC * TM + kq * TM];
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        bv[t] = xa[kq * XP + t * 16];
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[t % R], bv[t], acc[t], 0, 0, 0);
                }
            }
            if (k0 + KC < a.K)
                __syncthreads();  // everyone is done with this chunk's tiles
        }
        if (!wave_active)
            return;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float *omax = a.omax + ((size_t)(t % R) * a.n_mgroups + mgroup) * TM + wm * MX + 4 * lq;
            const float mp = msh[wh * 64 + t * 16 + lr];
            // an infinite column bound makes the result NaN, as the reference's exp(inf - inf) does
            const float mpt = (mp - mp) + mp + a.c0;
#pragma unroll
            for (int v = 0; v < 4; ++v)
                res[t][v] = (__builtin_amdgcn_logf(acc[t][v]) + (mpt + omax[v])) * a.ln2_over_eps;
        }
    } else {
        // wide offsets: running (maximum, sum) per output on the VALU, chunk by chunk from the staged tiles
        float best[4][4], sum[4][4];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                best[t][v] = -INFINITY;
                sum[t][v] = 0.0f;
            }
        for (int k0 = 0; k0 < a.K; k0 += KC) {
            const int kc = min(KC, a.K - k0);
            __syncthreads();
            stage(k0, kc);
            __syncthreads();
            if (wave_active)
                lse_chunk<R, XP, false>(best, sum, xs, os, wh * 64, wm, lr, lq, kc);
        }
        if (!wave_active)
            return;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float b = best[t][v];
                res[t][v] = (__builtin_amdgcn_logf(sum[t][v]) + ((b - b) + b + a.c0)) * a.ln2_over_eps;
            }
    }

    if (q.full != nullptr) {
        // the MEX output itself, for the gradient operators: tile t = (slot group t / R, region t % R)
        const size_t plane = (size_t)a.Co * a.Ho * a.Wo;
        if (R == 4 && q.full_pairs) {
            // regions 2 ry and 2 ry + 1 of a window are neighbours in a row: one 8-byte store
#pragma unroll
            for (int ry = 0; ry < 2; ++ry) {
                const PixelRef cp = locate(a, 2 * ry, (chunk * NH + wh) * 16 + lr);
                if (cp.out_off < 0)
                    continue;
                float *o = q.full + (size_t)cp.b * a.M * plane + cp.out_off + (size_t)(m0 + 4 * lq) * plane;
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (all_rows || m0 + 4 * lq + v < a.M)
                        *reinterpret_cast<float2 *>(o + v * plane) = make_float2(res[2 * ry][v], res[(2 * ry + 1) % 4][v]);
            }
        } else {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const PixelRef cp = locate(a, t % R, (chunk * NH + wh) * (16 * G) + (t / R) * 16 + lr);
                if (cp.out_off < 0)
                    continue;
                float *o = q.full + (size_t)cp.b * a.M * plane + cp.out_off + (size_t)(m0 + 4 * lq) * plane;
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (all_rows || m0 + 4 * lq + v < a.M)
                        o[v * plane] = res[t][v];
            }
        }
    }
    // ---- sum over the window (one pixel per region, row-major) and store the pooled pixel ----
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const long long pos = ppos[(wh * G + g) * 16 + lr];  // written before the first barrier
        if (pos < 0)
            continue;
        float *o = q.pooled + pos + row0;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            float w = res[g * R][v];
#pragma unroll
            for (int r = 1; r < R; ++r)
                w += res[g * R + r][v];
            if (all_rows || m0 + 4 * lq + v < a.M)
                o[v * plane_p] = w;
        }
    }
}

// Panel form of the kernel above for the deep layers of such a stack: 2x2 windows, patches that are exactly the C
// channels of a pixel (blocks [C, 1, 1], stride 1, no padding), C = 32 * NCH = 32 (plain call on a small grid only), 64, 128 or 256.  The pixels of a workgroup's
// windows are then whole rows of a few images, i.e. per channel one contiguous run of floats, and the K values of all
// its 64 * NH columns ("the panel") fit its registers (K / 16 float4 per thread).  The workgroup loads the panel once
// with coalesced 16-byte loads (lanes along the run, then along k), takes each column's maximum over all of K once
// (through LDS), and the chunk loop is left with two barriers: exponentials of 32 panel rows and the offsets tiles go
// to LDS, the next offsets tiles are requested, the matrix loop runs.  Against the kernel above (per chunk: a gather
// of dwords an image apart, a running maximum with its own barrier, rescaling of the accumulators) the chunk takes
// about half the time where one workgroup per compute unit is all a layer offers.
// LDS tiles are stored with column ^ swizzle(k): bits 4-5 of the column take k & 3, so that the four k rows a matrix
// instruction's operand fetch touches (lane >> 4) fall into different banks; for the panel tile bits 2-3 take
// (k >> 2) & 3 as well, which spreads the lanes of the staging writes that hold one column at 16 different k.
// The four MEX values of a 2x2 window (region t = pixel (t / 2, t % 2)) for instances v < live, planes `plane`
// floats apart: the two pixels of a window row as one 8-byte store where the tensor allows it.
__device__ __forceinline__ void store_window(float *o, size_t plane, int lgW, int pairs, const float (&res)[4][4], int live)
{
    if (pairs) {
#pragma unroll
        for (int ry = 0; ry < 2; ++ry)
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (v < live)
                    *reinterpret_cast<float2 *>(o + v * plane + ((size_t)ry << lgW)) =
                        make_float2(res[2 * ry][v], res[2 * ry + 1][v]);
    } else {
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (v < live)
                    o[v * plane + ((size_t)(t >> 1) << lgW) + (t & 1)] = res[t][v];
    }
}

constexpr int kPanelWorkgroups = 256;   // below this many two-half workgroups (one per compute unit) the panel form runs one-half ones

struct PanelArgs {
    int lgF;          // log2 of the float4 per (part, k): run / 4
    int lgTPP;        // log2 of the threads per part
    int lgW, Ws, RS;  // log2(width); windows per row; windows per image
    int run;          // pixels of a part: whole rows of one image, contiguous per channel
    int nparts;       // parts per workgroup
    int ppi;          // parts per image
    int total_parts;  // B * ppi
    int HW;
    const float *raw_offsets;  // SELFPACK: the offsets as the caller holds them, [region][M][K]
    int normalize;             // SELFPACK: subtract every row's logsumexp first (normalize_offsets)
};

// One offsets row of 32 elements packed by one thread, with the arithmetic of mex_pack_offsets_kernel<1> in its order:
// the lanes of that kernel hold one element each and add their exponentials in a butterfly (partner lane ^ 32, 16, 8,
// 4, 2, 1; the upper half of the wave holds zeros for a row of 32), which is the tree below.
__device__ __forceinline__ void pack_row32(const float (&x)[32], int normalize, float scale, float &lse, float &hi,
                                           float &lo, float &xh)
{
    lse = 0.0f;
    if (normalize) {
        float mxv = -INFINITY;
#pragma unroll
        for (int k = 0; k < 32; ++k)
            mxv = fmaxf(mxv, x[k]);
        if (!(fabsf(mxv) < INFINITY))
            mxv = 0.0f;
        float e[32];
#pragma unroll
        for (int k = 0; k < 32; ++k)
            e[k] = mex_exp_term(x[k] - mxv);
#pragma unroll
        for (int d = 16; d > 0; d >>= 1)
#pragma unroll
            for (int k = 0; k < d; ++k)
                e[k] = e[k] + e[k + d];
        lse = mex_lse_of(e[0], mxv);
    }
    float xmx = -INFINITY, xmn = INFINITY;
#pragma unroll
    for (int k = 0; k < 32; ++k) {
        xmx = fmaxf(xmx, x[k]);
        xmn = fminf(xmn, x[k]);
    }
    xh = scale >= 0.0f ? xmx : xmn;
    hi = mex_scaled_offset(xh, lse, scale);
    lo = mex_scaled_offset(scale >= 0.0f ? xmn : xmx, lse, scale);
}

// POOL = false: the same tiling without the pooling, every MEX value stored (the plain MEX call on such a layer).
// SELFPACK (one column half, one chunk, no pooling): no packed offsets exist; thread (region tid / 64, instance
// tid % 64) packs its row of the caller's offsets into the LDS tile itself (pack_row32), so that a self-packing call of
// a small layer is this one launch.
// INF (plain call only): infinite epsilon - the extreme value of patch + offset through max_chunk, from the panel and
// the scaled offsets; nothing of the product form (column maxima, packed exponentials, row ranges) is touched.
template <int NH, int NCH, bool POOL, bool SELFPACK = false, bool INF = false>
__global__ __launch_bounds__(256 * NH) void mex_pool_panel_kernel(const MexKernelArgs a, const PoolArgs q,
                                                                  const PanelArgs g)
{
    static_assert(!SELFPACK || (NH == 1 && NCH == 1 && !POOL), "in-kernel packing: one row per thread, one chunk");
    static_assert(!INF || (!SELFPACK && !POOL), "infinite epsilon: the plain call on packed offsets");
    constexpr int R = 4;
    constexpr int XP = 64 * NH;
    constexpr int kThreads = 256 * NH;
    constexpr int NV = 2 * NCH;   // float4 of the panel per thread: rows kslot + 16 u
    __shared__ __attribute__((aligned(16))) float xs[KC * XP];       // [k][column ^ swizzle]
    __shared__ __attribute__((aligned(16))) float os[R * KC * TM];   // [region][k][instance ^ swizzle]
    __shared__ __attribute__((aligned(16))) float pmx[16 * XP];      // [kslot][column]: partial column maxima
    __shared__ float msh[XP];                                        // column maxima
    __shared__ float omax_sh[SELFPACK ? R * TM : 1];                 // SELFPACK: row maxima of the scaled offsets
    // per slot: where instance 0 goes in the pooled tensor (POOL = false: where the window's first pixel goes in the
    // MEX output), -1 = no window
    __shared__ long long ppos[16 * NH];
    __shared__ long long fpos[16 * NH];   // POOL with q.full: where the window's first pixel goes in the unpooled output

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 3, wh = wave >> 2;
    const int chunk = blockIdx.x, mgroup = blockIdx.y;
    const int m0 = mgroup * TM + wm * MX;
    const bool wave_active = m0 < a.M;

    // ---- offsets tiles of a chunk: kThreads float4 per region and round ----
    constexpr int TILE4 = KC * TM / 4;
    constexpr int NO = TILE4 / kThreads;
    static_assert(TILE4 % kThreads == 0, "offsets tile copy");
    static_assert((NO == 1 || NO == 2) && R == 4, "offsets tile registers");
    float4 on0, on1, on2, on3, on4, on5, on6, on7;   // float4 i: region i / NO, round i % NO
    const float4 *osrc = reinterpret_cast<const float4 *>(a.offe + (size_t)mgroup * a.K * TM) + tid;
    const size_t ostep = (size_t)a.n_mgroups * a.K * (TM / 4);   // float4 between the regions' tiles
#define SIMNETS_PANEL_LOAD(i, k0) \
    on##i = osrc[(size_t)((i) / NO) * ostep + ((i) % NO) * kThreads + (size_t)(k0) * (TM / 4)];
#define SIMNETS_PANEL_ISSUE(k0)                                                                              \
    {                                                                                                        \
        SIMNETS_PANEL_LOAD(0, k0) SIMNETS_PANEL_LOAD(1, k0) SIMNETS_PANEL_LOAD(2, k0) SIMNETS_PANEL_LOAD(3, k0) \
        if constexpr (NO == 2) {                                                                             \
            SIMNETS_PANEL_LOAD(4, k0) SIMNETS_PANEL_LOAD(5, k0) SIMNETS_PANEL_LOAD(6, k0) SIMNETS_PANEL_LOAD(7, k0) \
        }                                                                                                    \
    }

    // ---- the panel: this thread's float4 (4 neighbouring pixels of one channel) of rows kslot + 16 u ----
    const int part = tid >> g.lgTPP;
    const int jj = tid & ((1 << g.lgTPP) - 1);
    const int pg = jj & ((1 << g.lgF) - 1);
    const int kslot = jj >> g.lgF;   // 0 .. 15
    const int gpart = chunk * g.nparts + part;
    const bool pvalid = gpart < g.total_parts;
    const int pb = pvalid ? gpart / g.ppi : 0;
    const int po = pvalid ? (gpart - pb * g.ppi) * g.run : 0;   // first pixel of the part inside its image
    float4 pv[NV];
    {
        const float *src = a.in + (size_t)pb * a.K * g.HW + po + 4 * pg + (size_t)kslot * g.HW;
#pragma unroll
        for (int u = 0; u < NV; ++u)
            pv[u] = *reinterpret_cast<const float4 *>(src + (size_t)(16 * u) * g.HW);
    }
    float4 rw[SELFPACK ? KC / 4 : 1];   // SELFPACK: this thread's row of the caller's offsets
    const bool row_valid = SELFPACK && mgroup * TM + (tid & 63) < a.M;
    if constexpr (SELFPACK) {
        const float4 *src = reinterpret_cast<const float4 *>(
            g.raw_offsets + ((size_t)(tid >> 6) * a.M + (row_valid ? mgroup * TM + (tid & 63) : 0)) * KC);
#pragma unroll
        for (int i = 0; i < KC / 4; ++i)
            rw[i] = src[i];
    } else if constexpr (!INF) {
        SIMNETS_PANEL_ISSUE(0)
    }

    // wide: an offsets row whose range is beyond the product form's on its own; unbounded: ... and not even finite
    int wide = 0, unbounded = 0;
    if (!SELFPACK && !INF && tid < TM) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float rg = a.orng[((size_t)r * a.n_mgroups + mgroup) * TM + tid];
            wide |= !(rg <= kProductRange);
            unbounded |= !(rg < INFINITY);
        }
    }

    if (tid < 16 * NH) {
        const int slot = chunk * (16 * NH) + tid;
        long long pos = -1, fp = -1;
        if (slot < a.slots) {
            const int b = (int)fast_div((unsigned)slot, a.dRS);
            const int sq = slot - b * a.RS;
            const int qw = (int)fast_div((unsigned)sq, a.dWs);
            const int i = sq - qw * a.Ws;
            fp = (long long)b * a.M * g.HW + ((long long)(2 * qw) << g.lgW) + 2 * i;
            pos = POOL ? (long long)b * a.M * ((long long)q.Hp * q.Wp) + (long long)qw * q.Wp + i : fp;
        }
        ppos[tid] = pos;
        fpos[tid] = fp;
    }

    // columns of the four pixels: tile (column half, region) x slot inside the half
    int colx[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int pix = po + 4 * pg + e;
        const int h = pix >> g.lgW, w = pix & ((1 << g.lgW) - 1);
        const int sl = pb * g.RS + (h >> 1) * g.Ws + (w >> 1) - chunk * (16 * NH);
        colx[e] = pvalid ? (sl >> 4) * 64 + ((h & 1) * 2 + (w & 1)) * 16 + (sl & 15) : 0;
    }

    if constexpr (INF) {
        // ---- infinite epsilon: chunk by chunk, values times the sign of epsilon (the minimum is a negated maximum) ----
        const int lr = lane & 15, lq = lane >> 4;
        const float sg = a.inf_sign;
        float best[4][4];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v)
                best[t][v] = -INFINITY;
        const int sw = ((kslot & 3) << 4) | (((kslot >> 2) & 3) << 2);
        const float4 *psrc = reinterpret_cast<const float4 *>(a.offp + (size_t)mgroup * a.K * TM) + tid;
        const int dst_row = tid & ~15, dst_col = (tid & 15) ^ (((tid >> 4) & 3) << 2);
        float4 ov[R * NO];   // the scaled offsets of the next chunk: float4 i of region i / NO, round i % NO
#pragma unroll
        for (int i = 0; i < R * NO; ++i)
            ov[i] = psrc[(size_t)(i / NO) * ostep + (i % NO) * kThreads];
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            if (c > 0)
                __syncthreads();  // everyone is done with the previous chunk's tiles
#pragma unroll
            for (int i = 0; i < R * NO; ++i) {
                float4 *dst = reinterpret_cast<float4 *>(os) + (dst_row | ((dst_col + 4 * (i / NO)) & 15));
                dst[(i / NO) * TILE4 + (i % NO) * kThreads] =
                    make_float4(ov[i].x * sg, ov[i].y * sg, ov[i].z * sg, ov[i].w * sg);
            }
            if (pvalid) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const float4 v = pv[2 * c + h];
                    float *row = xs + (kslot + 16 * h) * XP;
                    row[colx[0] ^ sw] = v.x * sg;
                    row[colx[1] ^ sw] = v.y * sg;
                    row[colx[2] ^ sw] = v.z * sg;
                    row[colx[3] ^ sw] = v.w * sg;
                }
            }
            __syncthreads();
            if (c + 1 < NCH) {
#pragma unroll
                for (int i = 0; i < R * NO; ++i)
                    ov[i] = psrc[(size_t)(i / NO) * ostep + (i % NO) * kThreads + (size_t)((c + 1) * KC) * (TM / 4)];
            }
            max_chunk<XP>(best, xs, os, wh * 64, wm, lr, lq);
        }
        if (!wave_active)
            return;
        const long long pos = ppos[wh * 16 + lr];  // written before the first barrier
        if (pos < 0)
            return;
        float res[4][4];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v)
                res[t][v] = best[t][v] * sg;
        store_window(q.pooled + pos + (size_t)(m0 + 4 * lq) * g.HW, g.HW, g.lgW, q.out_pairs, res,
                     m0 + MX <= a.M ? 4 : a.M - (m0 + 4 * lq));
        return;
    }

    // ---- column maxima over all of K ----
    {
        float4 pm = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            pv[u].x *= a.scale; pv[u].y *= a.scale; pv[u].z *= a.scale; pv[u].w *= a.scale;
            pm.x = fmaxf(pm.x, pv[u].x); pm.y = fmaxf(pm.y, pv[u].y);
            pm.z = fmaxf(pm.z, pv[u].z); pm.w = fmaxf(pm.w, pv[u].w);
        }
        const int cg = (part << g.lgF) | pg;   // 0 .. XP / 4 - 1
        reinterpret_cast<float4 *>(pmx)[kslot * (XP / 4) + cg] = pm;
    }
    float rx[SELFPACK ? KC : 1];   // SELFPACK: the row, its logsumexp (0 without normalisation) and its scaled maximum
    float row_lse = 0.0f, row_hi = 0.0f, row_xh = 0.0f;
    if constexpr (SELFPACK) {
#pragma unroll
        for (int i = 0; i < KC / 4; ++i) {
            rx[4 * i] = rw[i].x; rx[4 * i + 1] = rw[i].y; rx[4 * i + 2] = rw[i].z; rx[4 * i + 3] = rw[i].w;
        }
        float lo;
        pack_row32(rx, g.normalize, a.scale, row_lse, row_hi, lo, row_xh);
        if (row_valid) {
            wide = !(row_hi - lo <= kProductRange);
            unbounded = !(row_hi - lo < INFINITY);    // NaN or inf (infinite entries) sends the workgroup to the VALU form
        } else {
            row_hi = 0.0f;   // rows past the last instance: zeros, like the pack kernel's padding
        }
        omax_sh[tid] = row_hi;
    }
    bool prod = !__syncthreads_or(wide);
    float msub[4];
    {
        const int cg = (part << g.lgF) | pg;
        float4 m = reinterpret_cast<const float4 *>(pmx)[cg];
#pragma unroll
        for (int s = 1; s < 16; ++s) {
            const float4 o = reinterpret_cast<const float4 *>(pmx)[s * (XP / 4) + cg];
            m.x = fmaxf(m.x, o.x); m.y = fmaxf(m.y, o.y); m.z = fmaxf(m.z, o.z); m.w = fmaxf(m.w, o.w);
        }
        if (!prod) {
            // Rows with a wide but finite range: the largest term of sum_k exp2(x_k - max x) exp2(o_k - max o) is at
            // least exp2(-range) of the OTHER factor too (take k where the offsets peak), and terms that underflow are
            // then below the sum's last bit.  So the product form still holds if every pixel column of the workgroup
            // spans at most kProductRange: the column minima, through the tile that the chunk loop fills later.
            const int any_unbounded = __syncthreads_or(unbounded);
            float4 pn = make_float4(INFINITY, INFINITY, INFINITY, INFINITY);
#pragma unroll
            for (int u = 0; u < NV; ++u) {
                pn.x = fminf(pn.x, pv[u].x); pn.y = fminf(pn.y, pv[u].y);
                pn.z = fminf(pn.z, pv[u].z); pn.w = fminf(pn.w, pv[u].w);
            }
            reinterpret_cast<float4 *>(xs)[kslot * (XP / 4) + cg] = pn;
            __syncthreads();
            float4 n = reinterpret_cast<const float4 *>(xs)[cg];
#pragma unroll
            for (int s = 1; s < 16; ++s) {
                const float4 o = reinterpret_cast<const float4 *>(xs)[s * (XP / 4) + cg];
                n.x = fminf(n.x, o.x); n.y = fminf(n.y, o.y); n.z = fminf(n.z, o.z); n.w = fminf(n.w, o.w);
            }
            // (a column with a NaN or an infinite value, or nothing finite at all, is not narrow)
            const bool narrow = !pvalid || (m.x - n.x <= kProductRange && m.y - n.y <= kProductRange &&
                                            m.z - n.z <= kProductRange && m.w - n.w <= kProductRange);
            prod = !__syncthreads_or(!narrow) && !any_unbounded;   // (the barrier also frees the tile again)
        }
        if (kslot == 0 && pvalid) {
            msh[colx[0]] = m.x; msh[colx[1]] = m.y; msh[colx[2]] = m.z; msh[colx[3]] = m.w;
        }
        // nothing finite in the column: the terms are exp2(-inf) = 0
        msub[0] = m.x == -INFINITY ? 0.0f : m.x; msub[1] = m.y == -INFINITY ? 0.0f : m.y;
        msub[2] = m.z == -INFINITY ? 0.0f : m.z; msub[3] = m.w == -INFINITY ? 0.0f : m.w;
    }

    const int lr = lane & 15, lq = lane >> 4;
    const size_t plane_p = POOL ? (size_t)q.Hp * q.Wp : (size_t)g.HW;   // floats per instance of the stored tensor
    const size_t row0 = (size_t)(m0 + 4 * lq) * plane_p;
    const bool all_rows = m0 + MX <= a.M;
    float res[4][4];  // [region][v]: MEX value of (slot lr of this half, instance m0 + 4*lq + v)

    if (prod) {
        floatx4 acc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t)
            acc[t] = floatx4{0.0f, 0.0f, 0.0f, 0.0f};
        const int sw = ((kslot & 3) << 4) | (((kslot >> 2) & 3) << 2);
        const float *oa = os + lq * TM + ((wm ^ lq) << 4) + lr;
        int xo[4];   // column of tile t in row lq (+ 4 j): ((t ^ lq) << 4 | lr) ^ (j & 3) << 2
#pragma unroll
        for (int t = 0; t < 4; ++t)
            xo[t] = lq * XP + wh * 64 + ((t ^ lq) << 4) + lr;
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            // ---- registers -> LDS (the previous chunk's readers are behind the barrier that ended its loop) ----
            if constexpr (SELFPACK) {
                // this thread's row: exp2(scaled offset - row maximum) into the region's tile, [k][instance ^ swizzle]
                float *orow = os + (tid >> 6) * KC * TM;
                const int mi = tid & 63;
#pragma unroll
                for (int k = 0; k < KC; ++k)
                    orow[k * TM + (mi ^ ((k & 3) << 4))] =
                        row_valid ? __builtin_amdgcn_exp2f(mex_offset_exponent(rx[k], row_xh, row_lse, a.scale)) : 0.0f;
            } else {
                float4 *dst = reinterpret_cast<float4 *>(os) + ((tid & ~15) | ((tid & 15) ^ (((tid >> 4) & 3) << 2)));
#define SIMNETS_PANEL_PUT(i) dst[((i) / NO) * TILE4 + ((i) % NO) * kThreads] = on##i;
                SIMNETS_PANEL_PUT(0) SIMNETS_PANEL_PUT(1) SIMNETS_PANEL_PUT(2) SIMNETS_PANEL_PUT(3)
                if constexpr (NO == 2) {
                    SIMNETS_PANEL_PUT(4) SIMNETS_PANEL_PUT(5) SIMNETS_PANEL_PUT(6) SIMNETS_PANEL_PUT(7)
                }
#undef SIMNETS_PANEL_PUT
            }
            // (columns of parts past the batch stay unwritten: a column only reaches its own, unstored, outputs)
            if (pvalid) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const float4 v = pv[2 * c + h];
                    float *row = xs + (kslot + 16 * h) * XP;
                    row[colx[0] ^ sw] = __builtin_amdgcn_exp2f(v.x - msub[0]);
                    row[colx[1] ^ sw] = __builtin_amdgcn_exp2f(v.y - msub[1]);
                    row[colx[2] ^ sw] = __builtin_amdgcn_exp2f(v.z - msub[2]);
                    row[colx[3] ^ sw] = __builtin_amdgcn_exp2f(v.w - msub[3]);
                }
            }
            __syncthreads();
            // the matrix loop, with the requests for the next chunk's offsets tiles spread between its steps (a
            // compute unit's vector memory path takes 64 bytes a cycle: issued in one go they hold the waves up)
            const bool more = c + 1 < NCH;
            const int kn = (c + 1) * KC;
#define SIMNETS_PANEL_RD(set, it, t)            \
    av##set[t] = oa[(t) * KC * TM + 4 * (it) * TM]; \
    bv##set[t] = xs[4 * (it) * XP + (xo[t] ^ (((it) & 3) << 2))];
#define SIMNETS_PANEL_READ(set, it) \
    SIMNETS_PANEL_RD(set, it, 0) SIMNETS_PANEL_RD(set, it, 1) SIMNETS_PANEL_RD(set, it, 2) SIMNETS_PANEL_RD(set, it, 3)
#define SIMNETS_PANEL_MM(set, t) \
    acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(av##set[t], bv##set[t], acc[t], 0, 0, 0);
#define SIMNETS_PANEL_FENCE __builtin_amdgcn_sched_barrier(0);
// the four matrix instructions of a step, each followed by the LDS reads of one tile of the step two ahead
#define SIMNETS_PANEL_STEP(cur, nxt, itn)                                        \
    SIMNETS_PANEL_MM(cur, 0) SIMNETS_PANEL_RD(nxt, itn, 0) SIMNETS_PANEL_FENCE   \
    SIMNETS_PANEL_MM(cur, 1) SIMNETS_PANEL_RD(nxt, itn, 1) SIMNETS_PANEL_FENCE   \
    SIMNETS_PANEL_MM(cur, 2) SIMNETS_PANEL_RD(nxt, itn, 2) SIMNETS_PANEL_FENCE   \
    SIMNETS_PANEL_MM(cur, 3) SIMNETS_PANEL_RD(nxt, itn, 3)
#define SIMNETS_PANEL_LAST(cur) \
    SIMNETS_PANEL_MM(cur, 0) SIMNETS_PANEL_MM(cur, 1) SIMNETS_PANEL_MM(cur, 2) SIMNETS_PANEL_MM(cur, 3)
#define SIMNETS_PANEL_NEXT(i2, i1)                    \
    if (more) {                                       \
        if constexpr (NO == 2) {                      \
            SIMNETS_PANEL_LOAD(i2, kn)                \
        } else if constexpr ((i2) % 2 == 0) {         \
            SIMNETS_PANEL_LOAD(i1, kn)                \
        }                                             \
    }                                                 \
    __builtin_amdgcn_sched_barrier(0);
            {
                // (waves past the last instance compute on the padding rows of the packed offsets: no branch whose
                // other side would leave loads pending in the registers used here)
                // operands of step i + 2 are read from LDS between the matrix instructions of step i: a wave issues
                // in order, so reads bunched in front of a step's four matrix instructions would idle the matrix unit
                float avA[R], bvA[4], avB[R], bvB[4], avC[R], bvC[4];
                SIMNETS_PANEL_READ(A, 0) SIMNETS_PANEL_READ(B, 1) SIMNETS_PANEL_FENCE
                SIMNETS_PANEL_STEP(A, C, 2) SIMNETS_PANEL_NEXT(0, 0)
                SIMNETS_PANEL_STEP(B, A, 3) SIMNETS_PANEL_NEXT(1, 0)
                SIMNETS_PANEL_STEP(C, B, 4) SIMNETS_PANEL_NEXT(2, 1)
                SIMNETS_PANEL_STEP(A, C, 5) SIMNETS_PANEL_NEXT(3, 1)
                SIMNETS_PANEL_STEP(B, A, 6) SIMNETS_PANEL_NEXT(4, 2)
                SIMNETS_PANEL_STEP(C, B, 7) SIMNETS_PANEL_NEXT(5, 2)
                SIMNETS_PANEL_LAST(A) SIMNETS_PANEL_NEXT(6, 3)
                SIMNETS_PANEL_LAST(B) SIMNETS_PANEL_NEXT(7, 3)
            }
#undef SIMNETS_PANEL_RD
#undef SIMNETS_PANEL_READ
#undef SIMNETS_PANEL_MM
#undef SIMNETS_PANEL_FENCE
#undef SIMNETS_PANEL_STEP
#undef SIMNETS_PANEL_LAST
#undef SIMNETS_PANEL_NEXT
            if (c + 1 < NCH)
                __syncthreads();  // everyone is done with this chunk's tiles
        }
        if (!wave_active)
            return;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const float *omax = SELFPACK ? omax_sh + t * TM + wm * MX + 4 * lq
                                         : a.omax + ((size_t)t * a.n_mgroups + mgroup) * TM + wm * MX + 4 * lq;
            const float mp = msh[wh * 64 + t * 16 + lr];
            // an infinite column bound makes the result NaN, as the reference's exp(inf - inf) does
            const float mpt = (mp - mp) + mp + a.c0;
#pragma unroll
            for (int v = 0; v < 4; ++v)
                res[t][v] = (__builtin_amdgcn_logf(acc[t][v]) + (mpt + omax[v])) * a.ln2_over_eps;
        }
    } else {
        // offsets too far apart for the product form: the same chunks through the same (swizzled) LDS tiles - the
        // panel's scaled values as they are and the scaled offsets instead of their exponentials - and a max-tracked
        // log-sum-exp on the VALU (lse_chunk); the tiles requested for the product form are dropped
        float best[4][4], sum[4][4];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                best[t][v] = -INFINITY;
                sum[t][v] = 0.0f;
            }
        const int sw = ((kslot & 3) << 4) | (((kslot >> 2) & 3) << 2);
        const float4 *psrc = reinterpret_cast<const float4 *>(a.offp + (size_t)mgroup * a.K * TM) + tid;
        float4 *dst = reinterpret_cast<float4 *>(os) + ((tid & ~15) | ((tid & 15) ^ (((tid >> 4) & 3) << 2)));
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            if (c > 0)
                __syncthreads();  // everyone is done with the previous chunk's tiles
            if constexpr (SELFPACK) {
                float *orow = os + (tid >> 6) * KC * TM;
                const int mi = tid & 63;
#pragma unroll
                for (int k = 0; k < KC; ++k)
                    orow[k * TM + (mi ^ ((k & 3) << 4))] = row_valid ? mex_scaled_offset(rx[k], row_lse, a.scale) : 0.0f;
            } else {
#pragma unroll
                for (int i = 0; i < R * NO; ++i)
                    dst[(i / NO) * TILE4 + (i % NO) * kThreads] =
                        psrc[(size_t)(i / NO) * ostep + (i % NO) * kThreads + (size_t)(c * KC) * (TM / 4)];
            }
            if (pvalid) {
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const float4 v = pv[2 * c + h];
                    float *row = xs + (kslot + 16 * h) * XP;
                    row[colx[0] ^ sw] = v.x;
                    row[colx[1] ^ sw] = v.y;
                    row[colx[2] ^ sw] = v.z;
                    row[colx[3] ^ sw] = v.w;
                }
            }
            __syncthreads();
            lse_chunk<R, XP, true>(best, sum, xs, os, wh * 64, wm, lr, lq, KC);
        }
        if (!wave_active)
            return;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float b = best[t][v];
                res[t][v] = (__builtin_amdgcn_logf(sum[t][v]) + ((b - b) + b + a.c0)) * a.ln2_over_eps;
            }
    }

    // ---- sum over the window (one pixel per region, row-major) and store the pooled pixel ----
    const long long pos = ppos[wh * 16 + lr];  // written before the first barrier
    if (pos < 0)
        return;
    float *o = q.pooled + pos + row0;
    if (POOL) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float w = ((res[0][v] + res[1][v]) + res[2][v]) + res[3][v];
            if (all_rows || m0 + 4 * lq + v < a.M)
                o[v * plane_p] = w;
        }
        if (q.full != nullptr) {
            // ... and the MEX values themselves, for the gradient operators (region t = pixel (t / 2, t % 2))
            float *f = q.full + fpos[wh * 16 + lr] + (size_t)(m0 + 4 * lq) * g.HW;
            store_window(f, g.HW, g.lgW, q.full_pairs, res, all_rows ? 4 : a.M - (m0 + 4 * lq));
        }
    } else {
        store_window(o, plane_p, g.lgW, q.out_pairs, res, all_rows ? 4 : a.M - (m0 + 4 * lq));
    }
}

// Geometry of the panel form for workgroups of nh column halves; false when the layer does not have it.
bool panel_geometry(const MexPlan &p, int ph, int pw, const float *input, int nh, PanelArgs *g)
{
    const simnets_mex_dims &d = p.d;
    if (ph != 2 || pw != 2 || d.block_c != p.C || d.block_h != 1 || d.block_w != 1 || d.stride_h != 1 ||
        d.stride_w != 1 || d.pad_c != 0 || d.pad_h != 0 || d.pad_w != 0 || d.channels_out != 1 || (p.H & 1) ||
        (p.W & 1) || (p.W & (p.W - 1)) != 0)
        return false;
    if (d.K != 32 && d.K != 64 && d.K != 128 && d.K != 256)
        return false;
    if (reinterpret_cast<uintptr_t>(input) % 16 != 0)
        return false;
    const int spw = 16 * nh, Ws = p.W / 2, RS = (p.H / 2) * Ws, HW = p.H * p.W;
    if (d.region_size != RS)
        return false;
    int run;
    if (spw % RS == 0)
        run = HW;        // whole images
    else if (RS % spw == 0 && spw % Ws == 0)
        run = 4 * spw;   // whole window rows of one image
    else
        return false;
    auto lg = [](int v) { int l = 0; while ((1 << l) < v) ++l; return l; };
    g->run = run;
    g->nparts = 4 * spw / run;
    g->ppi = HW / run;
    g->total_parts = p.B * g->ppi;
    g->HW = HW;
    g->lgF = lg(run / 4);
    g->lgTPP = lg(256 * nh / g->nparts);
    g->lgW = lg(p.W);
    g->Ws = Ws;
    g->RS = RS;
    g->raw_offsets = nullptr;
    g->normalize = 0;
    return true;
}

template <int NH, bool POOL>
hipError_t launch_panel(const MexKernelArgs &a, const PoolArgs &q, const PanelArgs &g, dim3 grid, hipStream_t s)
{
    switch (a.K / KC) {
    case 1: hipLaunchKernelGGL((mex_pool_panel_kernel<NH, 1, POOL>), grid, dim3(256 * NH), 0, s, a, q, g); break;
    case 2: hipLaunchKernelGGL((mex_pool_panel_kernel<NH, 2, POOL>), grid, dim3(256 * NH), 0, s, a, q, g); break;
    case 4: hipLaunchKernelGGL((mex_pool_panel_kernel<NH, 4, POOL>), grid, dim3(256 * NH), 0, s, a, q, g); break;
    default: hipLaunchKernelGGL((mex_pool_panel_kernel<NH, 8, POOL>), grid, dim3(256 * NH), 0, s, a, q, g); break;
    }
    return hipGetLastError();
}

template <int NH>
hipError_t launch_panel_inf(const MexKernelArgs &a, const PoolArgs &q, const PanelArgs &g, dim3 grid, hipStream_t s)
{
    switch (a.K / KC) {
    case 1: hipLaunchKernelGGL((mex_pool_panel_kernel<NH, 1, false, false, true>), grid, dim3(256 * NH), 0, s, a, q, g); break;
    case 2: hipLaunchKernelGGL((mex_pool_panel_kernel<NH, 2, false, false, true>), grid, dim3(256 * NH), 0, s, a, q, g); break;
    case 4: hipLaunchKernelGGL((mex_pool_panel_kernel<NH, 4, false, false, true>), grid, dim3(256 * NH), 0, s, a, q, g); break;
    default: hipLaunchKernelGGL((mex_pool_panel_kernel<NH, 8, false, false, true>), grid, dim3(256 * NH), 0, s, a, q, g); break;
    }
    return hipGetLastError();
}

// Workgroup shape of the panel form for this layer (column halves), 0 when the layer does not have its geometry.
int panel_halves(const MexPlan &p, int ph, int pw, const float *input, int slots, int n_mgroups, PanelArgs *g,
                 bool pool)
{
    if (slots <= 16)
        return 0;
    // one column half per workgroup while two would leave compute units without a workgroup
    const int pnh = ((long long)slots + 31) / 32 * n_mgroups < kPanelWorkgroups ? 1 : 2;
    // a single chunk (32 channels): the plain call gains (64 x 32x16x16 -> 64: 7.2 -> 6.0 us per call; 512 images, with
    // the window rows stored 8 bytes at a time: 20.7 -> 19.2 us); with pooling the kernel above stays, and with it the
    // first layer's results stay those of its form with the Similarity inside, bit for bit
    if (p.d.K == 32 && pool)
        return 0;
    if (panel_geometry(p, ph, pw, input, pnh, g))
        return pnh;
    return pnh == 1 && panel_geometry(p, ph, pw, input, 2, g) ? 2 : 0;
}

#undef SIMNETS_PANEL_ISSUE
#undef SIMNETS_PANEL_LOAD

template <int R, int NH>
hipError_t launch_pool(const MexKernelArgs &a, const PoolArgs &q, dim3 grid, bool inside, hipStream_t s)
{
    if (q.sx)
        hipLaunchKernelGGL((mex_pool_kernel<R, NH, false, true>), grid, dim3(256 * NH), 0, s, a, q);
    else if (inside)
        hipLaunchKernelGGL((mex_pool_kernel<R, NH, false, false>), grid, dim3(256 * NH), 0, s, a, q);
    else
        hipLaunchKernelGGL((mex_pool_kernel<R, NH, true, false>), grid, dim3(256 * NH), 0, s, a, q);
    return hipGetLastError();
}

// The fused kernel applies when a pooling window is exactly one pixel of every offsets region.
bool fusable(const MexPlan &p, int ph, int pw, bool any_epsilon = false)
{
    const simnets_mex_dims &d = p.d;
    const int r = ph * pw;
    return p.use_unshared && (any_epsilon || std::isfinite(p.epsilon)) && d.offsets_c == 1 && d.offsets_h == ph &&
           d.offsets_w == pw && (r == 2 || r == 4) && d.num_regions == r;
}

// ... and the Similarity layer in front can be evaluated inside the staging when its channels are exactly the MEX
// patch of a pixel and its own patches are short
bool sim_fusable(const SimPlan &sp, const MexPlan &p, int ph, int pw)
{
    const simnets_mex_dims &d = p.d;
    return fusable(p, ph, pw) && sp.K <= kSimTaps && sp.algo != SIMNETS_ALGO_MFMA && d.block_c == sp.O &&
           d.block_h == 1 && d.block_w == 1 && d.stride_h == 1 && d.stride_w == 1 && d.pad_c == 0 && d.pad_h == 0 &&
           d.pad_w == 0 && d.channels_out == 1;
}

size_t sim_packed_bytes(const SimPlan &sp) { return align_up((size_t)((sp.O + 31) & ~31) * sp.K * 3 * sizeof(float), 256); }

int pool_launch(const MexPlan &p, int ph, int pw, const float *input, const float *offsets, float *pooled,
                void *workspace, const SimPlan *sp, const float *templates, const float *weights, void *stream,
                int phase, float *full = nullptr)
{
    const simnets_mex_dims &d = p.d;
    const int n_mgroups = (d.M + TM - 1) / TM;
    MexKernelArgs a = mex_kernel_args(p);
    PoolArgs q;
    q.sx = nullptr;
    q.full = full;
    q.full_pairs = full != nullptr && reinterpret_cast<uintptr_t>(full) % 8 == 0 && d.width_out % 2 == 0;
    q.out_pairs = 0;
    SimPackJob job;
    if (sp) {
        float *pa = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + mex_packed_bytes(p, TM, n_mgroups));
        job.templates = templates; job.weights = weights; job.pa = pa; job.pc = pa + (size_t)((sp->O + 31) & ~31) * sp->K * 2;
        job.O = sp->O; job.K = sp->K; job.mode = sp->mode; job.fudge = sp->fudge;
        q.sx = input; q.spa = job.pa; q.spc = job.pc;
        q.sC = sp->C; q.sH = sp->H; q.sW = sp->W; q.sbh = sp->bh; q.sbw = sp->bw; q.ssh = sp->sh; q.ssw = sp->sw;
        q.sph = sp->ph; q.spw_ = sp->pw; q.sK = sp->K; q.smode = sp->mode; q.soob = sp->oob;
        q.snorm = (sp->mode == SIM_MODE_L2_NORM) ? (float)((double)(-0.5f * (float)sp->K) * std::log(2.0 * M_PI)) : 0.0f;
        q.snorm_every = sp->norm_const_every_iteration; q.sB = sp->B;
    }
    const int rc = mex_pack_offsets(p, offsets, TM, n_mgroups, workspace, &a, stream, sp ? &job : nullptr,
                                    (phase & kMexPrepare) != 0);
    if (rc || !(phase & kMexRun))
        return rc;
    a.in = sp ? nullptr : input;
    q.pooled = pooled;
    q.Hp = d.height_out / ph;
    q.Wp = d.width_out / pw;
    // two column halves per workgroup whenever there are slots for both: the extra waves per compute unit pay even
    // when the launch then has fewer workgroups than compute units (measured on 512 images of 2x2 pixels)
    // ... and four halves (16 waves) when there are many slots and the patches are short: the offsets tiles are
    // then copied once per 256 pixel columns
    int nh = a.slots > 64 / (ph * pw) ? 2 : 1;
    // ... only with the Similarity inside (its patch taps and parameters are then fetched once per 256 columns:
    // 512 images of the first layer 24.2 -> 18.3 us); without it two halves are as fast or faster (15.6 against
    // 16.0 us, 104.7 against 111.0 us at 4096 images)
    if (sp && ph * pw == 4 && d.K <= 2 * KC && a.slots >= 64 * 128)
        nh = 4;
    // a single chunk on a grid that two halves would leave below one workgroup per compute unit: one half (64 images
    // of 32 x 16 x 16: 6.7 -> 6.1 us)
    const int spw2 = 2 * 64 / (ph * pw);   // slots of a workgroup of two halves
    if (nh == 2 && d.K <= KC && ((long long)a.slots + spw2 - 1) / spw2 * n_mgroups < kPanelWorkgroups)
        nh = 1;
    PanelArgs pg;
    const int panel = sp ? 0 : panel_halves(p, ph, pw, input, a.slots, n_mgroups, &pg, true);
    if (panel)
        nh = panel;
    q.spw = nh * 64 / (ph * pw);
    const long long gx = ((long long)a.slots + q.spw - 1) / q.spw;
    if (gx > 0x7fffffffLL || n_mgroups > 65535)
        return SIMNETS_ERR_TOO_LARGE;
    const bool inside = d.pad_c == 0 && d.pad_h == 0 && d.pad_w == 0 &&
                        (d.channels_out - 1) * d.stride_c + d.block_c <= p.C &&
                        (d.height_out - 1) * d.stride_h + d.block_h <= p.H &&
                        (d.width_out - 1) * d.stride_w + d.block_w <= p.W;
    dim3 grid((unsigned)gx, (unsigned)n_mgroups);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    hipError_t e;
    if (panel)
        e = nh == 1 ? launch_panel<1, true>(a, q, pg, grid, s) : launch_panel<2, true>(a, q, pg, grid, s);
    else if (ph * pw == 4)
        e = nh == 4 ? launch_pool<4, 4>(a, q, grid, inside, s)
                    : (nh == 2 ? launch_pool<4, 2>(a, q, grid, inside, s) : launch_pool<4, 1>(a, q, grid, inside, s));
    else
        e = nh == 2 ? launch_pool<2, 2>(a, q, grid, inside, s) : launch_pool<2, 1>(a, q, grid, inside, s);
    return e == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

}  // namespace

bool mex_panel_geometry(const MexPlan &p)
{
    PanelArgs g;
    const long long slots = (long long)p.B * p.d.region_size;
    // (the plain call's panel kernel also takes an infinite epsilon)
    if (!fusable(p, 2, 2, true) || slots > 0x7fffffffLL)
        return false;
    // (the pointer is checked by the launch; any 16-byte aligned one stands in here)
    return panel_halves(p, 2, 2, reinterpret_cast<const float *>(uintptr_t(16)), (int)slots, (p.d.M + TM - 1) / TM,
                        &g, false) != 0;
}

int mex_panel_launch(const MexPlan &p, const MexKernelArgs &a, const float *input, float *output, void *stream)
{
    PanelArgs g;
    const int nh = panel_halves(p, 2, 2, input, a.slots, a.n_mgroups, &g, false);
    if (!nh)
        return SIMNETS_PANEL_NOT_TAKEN;
    PoolArgs q;
    q.sx = nullptr;
    q.full = nullptr;
    q.full_pairs = 0;
    q.out_pairs = reinterpret_cast<uintptr_t>(output) % 8 == 0;
    q.pooled = output;
    q.Hp = p.d.height_out / 2;
    q.Wp = p.d.width_out / 2;
    q.spw = 16 * nh;
    const long long gx = ((long long)a.slots + q.spw - 1) / q.spw;
    if (gx > 0x7fffffffLL || a.n_mgroups > 65535)
        return SIMNETS_ERR_TOO_LARGE;
    MexKernelArgs b = a;
    b.in = input;
    dim3 grid((unsigned)gx, (unsigned)a.n_mgroups);
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    hipError_t e;
    if (!b.finite_eps)
        e = nh == 1 ? launch_panel_inf<1>(b, q, g, grid, s) : launch_panel_inf<2>(b, q, g, grid, s);
    else
        e = nh == 1 ? launch_panel<1, false>(b, q, g, grid, s) : launch_panel<2, false>(b, q, g, grid, s);
    return e == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

int mex_panel_launch_selfpack(const MexPlan &p, const MexKernelArgs &a, const float *input, const float *offsets,
                              float *output, void *stream)
{
    PanelArgs g;
    if (p.d.K != KC || reinterpret_cast<uintptr_t>(offsets) % 16 != 0 || !std::isfinite(p.epsilon))
        return SIMNETS_PANEL_NOT_TAKEN;
    if (panel_halves(p, 2, 2, input, a.slots, a.n_mgroups, &g, false) != 1)
        return SIMNETS_PANEL_NOT_TAKEN;
    g.raw_offsets = offsets;
    g.normalize = p.normalize_offsets;
    PoolArgs q;
    q.sx = nullptr;
    q.full = nullptr;
    q.full_pairs = 0;
    q.out_pairs = reinterpret_cast<uintptr_t>(output) % 8 == 0;
    q.pooled = output;
    q.Hp = p.d.height_out / 2;
    q.Wp = p.d.width_out / 2;
    q.spw = 16;
    const long long gx = ((long long)a.slots + q.spw - 1) / q.spw;
    if (gx > 0x7fffffffLL || a.n_mgroups > 65535)
        return SIMNETS_ERR_TOO_LARGE;
    MexKernelArgs b = a;
    b.in = input;
    dim3 grid((unsigned)gx, (unsigned)a.n_mgroups);
    hipLaunchKernelGGL((mex_pool_panel_kernel<1, 1, false, true>), grid, dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                       b, q, g);
    return hipGetLastError() == hipSuccess ? SIMNETS_OK : SIMNETS_ERR_HIP;
}

size_t mex_pool_workspace_bytes(const MexPlan &p, int ph, int pw)
{
    if (fusable(p, ph, pw))
        return mex_packed_bytes(p, TM, (p.d.M + TM - 1) / TM);
    // otherwise: MEX into a scratch tensor, then the pooling kernel
    const size_t out = (size_t)p.B * p.d.M * p.d.channels_out * p.d.height_out * p.d.width_out * sizeof(float);
    return mex_workspace_bytes(p) + align_up(out, 256);
}

int mex_pool_launch(const MexPlan &p, int ph, int pw, const float *input, const float *offsets, float *pooled,
                    void *workspace, size_t workspace_bytes, void *stream, int phase, float *full_out)
{
    const simnets_mex_dims &d = p.d;
    if (workspace_bytes < mex_pool_workspace_bytes(p, ph, pw))
        return SIMNETS_ERR_WORKSPACE;
    if (!fusable(p, ph, pw)) {
        // the caller's tensor for the MEX output if it wants one, else scratch
        float *full = full_out ? full_out
                               : reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + mex_workspace_bytes(p));
        const int rc = mex_launch(p, input, offsets, full, workspace, mex_workspace_bytes(p), stream, phase);
        if (rc || !(phase & kMexRun))
            return rc;
        return sum_pool_launch(p.B, d.M * d.channels_out, d.height_out, d.width_out, ph, pw, full, pooled, stream);
    }
    return pool_launch(p, ph, pw, input, offsets, pooled, workspace, nullptr, nullptr, nullptr, stream, phase, full_out);
}

// Similarity -> MEX -> sum pooling.  `mp` is the MEX plan over the Similarity output's shape.
size_t sim_mex_pool_workspace_bytes(const SimPlan &sp, const MexPlan &mp, int ph, int pw)
{
    if (sim_fusable(sp, mp, ph, pw))
        return mex_packed_bytes(mp, TM, (mp.d.M + TM - 1) / TM) + sim_packed_bytes(sp);
    // otherwise: the Similarity output in scratch memory, then the two (or three) kernels
    const size_t mid = align_up((size_t)sp.B * sp.O * sp.oh * sp.ow * sizeof(float), 256);
    return mid + align_up(sim_workspace_bytes(sp), 256) + mex_pool_workspace_bytes(mp, ph, pw);
}

int sim_mex_pool_launch(const SimPlan &sp, const MexPlan &mp, int ph, int pw, const float *input,
                        const float *templates, const float *weights, const float *offsets, float *pooled,
                        void *workspace, size_t workspace_bytes, void *stream, int phase)
{
    if (workspace_bytes < sim_mex_pool_workspace_bytes(sp, mp, ph, pw))
        return SIMNETS_ERR_WORKSPACE;
    if (sim_fusable(sp, mp, ph, pw))
        return pool_launch(mp, ph, pw, input, offsets, pooled, workspace, &sp, templates, weights, stream, phase);
    // separate kernels: [Similarity output | Similarity workspace | MEX + pooling workspace] (the two workspaces side
    // by side, so that both can stay prepared)
    const size_t mid_bytes = align_up((size_t)sp.B * sp.O * sp.oh * sp.ow * sizeof(float), 256);
    const size_t sim_bytes = align_up(sim_workspace_bytes(sp), 256);
    float *mid = reinterpret_cast<float *>(workspace);
    char *sim_ws = reinterpret_cast<char *>(workspace) + mid_bytes;
    char *rest = sim_ws + sim_bytes;
    int rc = SIMNETS_OK;
    if (phase & kMexPrepare)
        rc = sim_prepare(sp, templates, weights, sim_ws, sim_bytes, stream);
    if (!rc && (phase & kMexRun))
        rc = sim_run(sp, input, mid, sim_ws, sim_bytes, stream);
    if (rc)
        return rc;
    return mex_pool_launch(mp, ph, pw, mid, offsets, pooled, rest, workspace_bytes - mid_bytes - sim_bytes, stream, phase);
}

}  // namespace simnets
