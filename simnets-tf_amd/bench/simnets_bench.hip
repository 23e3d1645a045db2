// Standalone C++ bench harness for libsimnets_hip.so.
//
//   simnets_bench --peaks                      machine micro-benchmarks (unpacked FP32 FMA issue rate,
//                                              fp32 MFMA rate, v_exp_f32 rate, HBM copy bandwidth)
//   simnets_bench --config N [--algo A] [--steps K] [--warmup W]     (N = 1..4 forward, 5 backward)
//                                              N in 1..4: times that benchmark configuration through the
//                                              C ABI with hipEvents on its own stream
//   ... --dump DIR                             also writes the synthetic inputs of the configuration to DIR as
//                                              raw float32 files (<tag>_x.bin, <tag>_t.bin, ...)
// Prints one JSON object per line: the measurements, and for every configuration a checksum of the
// output tensors its calls produced ({"checksum": name, "value": "<hex>", "elements": n}; the value is
// sum_i (bits(out[i]) + 1) * (2 i + 1) mod 2^64 over the fp32 bit patterns), so that a caller of the same
// library on the dumped inputs can be compared bit for bit.  Inputs are synthetic (fixed-seed
// counter-based generator), resident in HBM before timing starts.  Parity with the CPU oracle is not
// checked here (tests/ does that through the same ABI); this binary links only the product library.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "simnets_hip.h"

#define HIP_OK(x)                                                                                  \
    do {                                                                                           \
        hipError_t e_ = (x);                                                                       \
        if (e_ != hipSuccess) {                                                                    \
            fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            exit(1);                                                                               \
        }                                                                                          \
    } while (0)
#define SN_OK(x)                                                                                 \
    do {                                                                                         \
        int r_ = (x);                                                                            \
        if (r_ != 0) {                                                                           \
            fprintf(stderr, "simnets error %d (%s) at %s:%d\n", r_, simnets_hip_strerror(r_), __FILE__, __LINE__); \
            exit(1);                                                                             \
        }                                                                                        \
    } while (0)

typedef float floatx16 __attribute__((ext_vector_type(16)));

// ---------------------------------------------------------------- micro-benchmarks
__global__ __launch_bounds__(256) void fma_peak_kernel(float *out, float a, float b, int iters)
{
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
        acc[i] = (float)(threadIdx.x + i);
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int i = 0; i < 16; ++i)
                acc[i] = __builtin_fmaf(acc[i], a, b);
    }
    float s = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i)
        s += acc[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

__global__ __launch_bounds__(256) void mfma_peak_kernel(float *out, float a, float b, int iters)
{
    floatx16 acc[4];
    for (int i = 0; i < 4; ++i)
        for (int v = 0; v < 16; ++v)
            acc[i][v] = (float)v;
    float av = a + threadIdx.x, bv = b;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[i], 0, 0, 0);
    }
    float s = 0;
    for (int i = 0; i < 4; ++i)
        for (int v = 0; v < 16; ++v)
            s += acc[i][v];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

__global__ __launch_bounds__(256) void exp_peak_kernel(float *out, float a, int iters)
{
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
        acc[i] = -(float)(threadIdx.x + i) * a;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i)
            acc[i] = __builtin_amdgcn_exp2f(acc[i]);
    }
    float s = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i)
        s += acc[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

__global__ __launch_bounds__(256) void copy_kernel(const float4 *__restrict__ src, float4 *__restrict__ dst, size_t n)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        dst[i] = src[i];
}

static float time_ms(hipStream_t s, int reps, const std::function<void()> &fn);

#include <functional>
static float time_ms(hipStream_t s, int reps, const std::function<void()> &fn)
{
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    fn();
    HIP_OK(hipStreamSynchronize(s));
    HIP_OK(hipEventRecord(e0, s));
    for (int i = 0; i < reps; ++i)
        fn();
    HIP_OK(hipEventRecord(e1, s));
    HIP_OK(hipEventSynchronize(e1));
    float ms = 0;
    HIP_OK(hipEventElapsedTime(&ms, e0, e1));
    HIP_OK(hipEventDestroy(e0));
    HIP_OK(hipEventDestroy(e1));
    return ms / reps;
}


// ---------------------------------------------------------------- co-issue probes
// Streams of unpacked FP32 VALU instructions on fixed registers, two waves per SIMD (the occupancy of the wide
// Similarity tile): how the parity of the source registers and the number of sources change the issue rate.
//   0: v_fma acc, a, x, acc with a, x, acc all in even registers      1: a in odd registers
//   2: acc += d*d with d and acc of one parity                         3: d and acc of opposite parity
//   4: (d = a*x + b ; acc += d*d), the sqrt-weight pair                5: (d = b - x ; acc = a*|d| + acc), the L1 pair
//   6: (d = b - x ; q = a*d ; acc += q*d), the three-instruction L2 form
template <int V>
__global__ __launch_bounds__(256) void coissue_kernel(float *out, int iters)
{
    extern __shared__ float coissue_lds[];   // only to limit the workgroups per CU
    float r;
    asm volatile(
        "v_cvt_f32_u32 v20, %2\n\t"
        ".irp n,21,22,23,24,25,26,27,28,29,30,31,32,33,34,35,36,40,41,42,43,44,45,46,47,48,49,50,51,52,53,54,55,56,60,61,62,63,64,65,66,67,68,69,70,71,72,73,74,75,80,81,82\n\t"
        "v_mul_f32 v\\n, 0x3a83126f, v20\n\t"
        ".endr\n\t"
        ".irp n,100,104,108,112,116,120,124,128\n\t"
        "v_mov_b32 v\\n, 0\n\t"
        ".endr\n\t"
        "1:\n\t"
        ".rept 16\n\t"
        ".irp i,0,1,2,3,4,5,6,7\n\t"
        ".if %3 == 0\n\t v_fma_f32 v[100+4*\\i], v80, v[20+2*\\i], v[100+4*\\i]\n\t .endif\n\t"
        ".if %3 == 1\n\t v_fma_f32 v[100+4*\\i], v81, v[20+2*\\i], v[100+4*\\i]\n\t .endif\n\t"
        ".if %3 == 2\n\t v_fmac_f32 v[100+4*\\i], v[40+2*\\i], v[40+2*\\i]\n\t .endif\n\t"
        ".if %3 == 3\n\t v_fmac_f32 v[100+4*\\i], v[41+2*\\i], v[41+2*\\i]\n\t .endif\n\t"
        ".if %3 == 4\n\t v_fma_f32 v[41+2*\\i], v81, v[20+2*\\i], v82\n\t .endif\n\t"
        ".if %3 >= 5\n\t v_sub_f32 v[41+2*\\i], v82, v[20+2*\\i]\n\t .endif\n\t"
        ".endr\n\t"
        ".if %3 == 6\n\t .irp i,0,1,2,3,4,5,6,7\n\t v_mul_f32 v[60+2*\\i], v81, v[41+2*\\i]\n\t .endr\n\t .endif\n\t"
        ".if %3 >= 4\n\t .irp i,0,1,2,3,4,5,6,7\n\t"
        ".if %3 == 4\n\t v_fmac_f32 v[100+4*\\i], v[41+2*\\i], v[41+2*\\i]\n\t .endif\n\t"
        ".if %3 == 5\n\t v_fma_f32 v[100+4*\\i], v81, |v[41+2*\\i]|, v[100+4*\\i]\n\t .endif\n\t"
        ".if %3 == 6\n\t v_fmac_f32 v[100+4*\\i], v[60+2*\\i], v[41+2*\\i]\n\t .endif\n\t"
        ".endr\n\t .endif\n\t"
        ".endr\n\t"
        "s_sub_u32 %1, %1, 1\n\t"
        "s_cmp_lg_u32 %1, 0\n\t"
        "s_cbranch_scc1 1b\n\t"
        "v_add_f32 %0, v100, v128"
        : "=v"(r), "+s"(iters)
        : "v"(threadIdx.x), "n"(V)
        : "memory", "scc", "v20", "v21", "v22", "v23", "v24", "v25", "v26", "v27", "v28", "v29", "v30", "v31", "v32", "v33", "v34",
          "v35", "v36", "v40", "v41", "v42", "v43", "v44", "v45", "v46", "v47", "v48", "v49", "v50", "v51", "v52", "v53", "v54",
          "v55", "v56", "v60", "v61", "v62", "v63", "v64", "v65", "v66", "v67", "v68", "v69", "v70", "v71", "v72", "v73", "v74",
          "v75", "v80", "v81", "v82", "v100", "v104", "v108", "v112", "v116", "v120", "v124", "v128");
    out[blockIdx.x * 256 + threadIdx.x] = r;
}

template <int V>
static void run_coissue(const char *name, int valu_per_round, float *out, int cus, hipStream_t s)
{
    const int iters = 2000, blocks = cus * 2;   // 60 KB of LDS each: two workgroups per CU = two waves per SIMD
    HIP_OK(hipFuncSetAttribute((const void *)coissue_kernel<V>, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024));
    float ms = time_ms(s, 5, [&] { hipLaunchKernelGGL(coissue_kernel<V>, dim3(blocks), dim3(256), 60 * 1024, s, out, iters); });
    const double ops = (double)blocks * 256 * iters * 16.0 * valu_per_round;
    printf("{\"probe\": \"%s\", \"waves_per_simd\": 2, \"lane_instr_per_s_T\": %.2f, \"ms\": %.4f}\n", name,
           ops / (ms * 1e-3) / 1e12, ms);
}

static void run_peaks(hipStream_t s)
{
    hipDeviceProp_t prop;
    HIP_OK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    const int blocks = cus * 8;  // 8 workgroups of 4 waves per CU: 8 waves per SIMD
    float *out;
    HIP_OK(hipMalloc(&out, (size_t)blocks * 256 * sizeof(float)));
    {
        const int iters = 4096;
        float ms = time_ms(s, 5, [&] { hipLaunchKernelGGL(fma_peak_kernel, dim3(blocks), dim3(256), 0, s, out, 1.0001f, 0.5f, iters); });
        const double fma = (double)blocks * 256 * iters * 64.0;
        printf("{\"peak\": \"valu_fma_f32_unpacked\", \"lane_fma_per_s_T\": %.3f, \"tflops\": %.2f, \"implied_clock_ghz\": %.3f, "
               "\"cus\": %d, \"ms\": %.4f}\n",
               fma / (ms * 1e-3) / 1e12, 2 * fma / (ms * 1e-3) / 1e12, fma / (ms * 1e-3) / (cus * 64.0) / 1e9, cus, ms);
    }
    {
        const int iters = 2048;
        float ms = time_ms(s, 5, [&] { hipLaunchKernelGGL(mfma_peak_kernel, dim3(cus * 2), dim3(256), 0, s, out, 1.0f, 0.5f, iters); });
        const double mfma = (double)cus * 2 * 4 * iters * 16.0;  // wave-level MFMA instructions
        const double flop = mfma * 4096.0;
        printf("{\"peak\": \"mfma_f32_32x32x2\", \"tflops\": %.2f, \"implied_clock_ghz\": %.3f, \"ms\": %.4f}\n",
               flop / (ms * 1e-3) / 1e12, mfma * 64.0 / (ms * 1e-3) / (cus * 4.0) / 1e9, ms);
    }
    {
        const int iters = 4096;
        float ms = time_ms(s, 5, [&] { hipLaunchKernelGGL(exp_peak_kernel, dim3(blocks), dim3(256), 0, s, out, 1e-3f, iters); });
        const double n = (double)blocks * 256 * iters * 16.0;
        printf("{\"peak\": \"v_exp_f32\", \"exp_per_s_T\": %.3f, \"ms\": %.4f}\n", n / (ms * 1e-3) / 1e12, ms);
    }
    {
        const size_t bytes = (size_t)1 << 30;
        float4 *a, *b;
        HIP_OK(hipMalloc(&a, bytes));
        HIP_OK(hipMalloc(&b, bytes));
        HIP_OK(hipMemsetAsync(a, 1, bytes, s));
        float ms = time_ms(s, 5, [&] { hipLaunchKernelGGL(copy_kernel, dim3(cus * 16), dim3(256), 0, s, a, b, bytes / 16); });
        printf("{\"peak\": \"hbm_copy\", \"GBps_read_plus_write\": %.1f, \"ms\": %.4f}\n", 2.0 * bytes / (ms * 1e-3) / 1e9, ms);
        HIP_OK(hipFree(a));
        HIP_OK(hipFree(b));
    }
    run_coissue<0>("fma, three sources in even registers", 8, out, cus, s);
    run_coissue<1>("fma, sources of mixed parity", 8, out, cus, s);
    run_coissue<2>("acc += d*d, d and acc of one parity", 8, out, cus, s);
    run_coissue<3>("acc += d*d, d and acc of opposite parity", 8, out, cus, s);
    run_coissue<4>("d = a*x + b ; acc += d*d (sqrt-weight pair)", 16, out, cus, s);
    run_coissue<5>("d = b - x ; acc = a*|d| + acc (L1 pair)", 16, out, cus, s);
    run_coissue<6>("d = b - x ; q = a*d ; acc += q*d (three-instruction L2)", 24, out, cus, s);
    HIP_OK(hipFree(out));
}

// ---------------------------------------------------------------- synthetic inputs
static inline uint64_t mix64(uint64_t z)
{
    z += 0x9e3779b97f4a7c15ULL;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
}
static inline float uniform01(uint64_t seed, uint64_t i) { return (float)((mix64(seed * 0x100000001b3ULL + i) >> 40) * (1.0 / 16777216.0)); }
static void fill_uniform(std::vector<float> &v, uint64_t seed, float lo, float hi)
{
    for (size_t i = 0; i < v.size(); ++i)
        v[i] = lo + (hi - lo) * uniform01(seed, i);
}
static void fill_normal(std::vector<float> &v, uint64_t seed, float sigma)
{
    for (size_t i = 0; i < v.size(); ++i) {
        const float u1 = std::max(uniform01(seed, 2 * i), 1e-7f), u2 = uniform01(seed, 2 * i + 1);
        v[i] = sigma * std::sqrt(-2.0f * std::log(u1)) * std::cos(6.2831853f * u2);
    }
}
static std::string g_dump_dir;
static void dump(const std::string &name, const std::vector<float> &v)
{
    if (g_dump_dir.empty())
        return;
    const std::string path = g_dump_dir + "/" + name + ".bin";
    FILE *f = fopen(path.c_str(), "wb");
    if (!f || fwrite(v.data(), sizeof(float), v.size(), f) != v.size()) {
        fprintf(stderr, "cannot write %s\n", path.c_str());
        exit(1);
    }
    fclose(f);
}
// checksum of a device tensor's bit patterns, printed as one JSON line
static void checksum(const char *name, const float *dev, size_t n, hipStream_t s)
{
    std::vector<uint32_t> h(n);
    HIP_OK(hipStreamSynchronize(s));
    HIP_OK(hipMemcpy(h.data(), dev, n * sizeof(float), hipMemcpyDeviceToHost));
    uint64_t acc = 0;
    for (size_t i = 0; i < n; ++i)
        acc += ((uint64_t)h[i] + 1) * (2 * (uint64_t)i + 1);
    printf("{\"checksum\": \"%s\", \"value\": \"%016llx\", \"elements\": %zu}\n", name, (unsigned long long)acc, n);
}
static size_t count4(const int *d) { return (size_t)d[0] * d[1] * d[2] * d[3]; }
static float *upload(const std::vector<float> &v)
{
    float *d;
    HIP_OK(hipMalloc(&d, std::max<size_t>(v.size(), 1) * sizeof(float)));
    HIP_OK(hipMemcpy(d, v.data(), v.size() * sizeof(float), hipMemcpyHostToDevice));
    return d;
}

struct SimCase {
    simnets_similarity_attrs a;
    int in[4], tp[4], out[4];
    float *x, *t, *w, *y;
    void *ws;
    size_t ws_bytes;
};

static SimCase make_similarity(const std::string &tag, int B, int C, int H, int W, int O, int bh, int bw, int s, int p,
                               bool missing, int algo, int l1)
{
    SimCase c;
    simnets_similarity_attrs_default(&c.a);
    c.a.blocks[0] = bh; c.a.blocks[1] = bw;
    c.a.strides[0] = c.a.strides[1] = s;
    c.a.padding[0] = c.a.padding[1] = p;
    c.a.algo = algo;
    c.a.similarity_function = l1 ? SIMNETS_SIM_L1 : SIMNETS_SIM_L2;
    if (missing) {
        c.a.normalization_term = 1;
        c.a.ignore_nan_input = 1;
        c.a.out_of_bounds_value = NAN;
    }
    const int in[4] = {B, C, H, W}, tp[4] = {O, C, bh, bw};
    memcpy(c.in, in, sizeof(in));
    memcpy(c.tp, tp, sizeof(tp));
    SN_OK(simnets_similarity_out_shape(&c.a, c.in, c.tp, c.tp, c.out));
    std::vector<float> x((size_t)B * C * H * W), t((size_t)O * C * bh * bw), w(t.size());
    if (missing) {
        fill_uniform(x, 1234, -0.5f, 0.5f);
        fill_normal(t, 2345, 0.1f);
        fill_uniform(w, 3456, 0.5f, 1.5f);
    } else {
        fill_normal(x, 1234, 1.0f);
        fill_normal(t, 2345, 1.0f);
        fill_uniform(w, 3456, 0.1f, 2.0f);
    }
    dump(tag + "_x", x); dump(tag + "_t", t); dump(tag + "_w", w);
    c.x = upload(x); c.t = upload(t); c.w = upload(w);
    HIP_OK(hipMalloc(&c.y, (size_t)c.out[0] * c.out[1] * c.out[2] * c.out[3] * sizeof(float)));
    SN_OK(simnets_hip_similarity_workspace_bytes(&c.a, c.in, c.tp, &c.ws_bytes));
    HIP_OK(hipMalloc(&c.ws, std::max<size_t>(c.ws_bytes, 256)));
    return c;
}

struct MexCase {
    simnets_mex_attrs a;
    int in[4], out[4], off[5];
    float *x, *o, *y;
    void *ws;
    size_t ws_bytes, off_count;
};

static MexCase make_mex(const std::string &tag, int B, int C, int HW, int M, bool shared1, const float *input)
{
    MexCase c;
    simnets_mex_attrs_default(&c.a);
    c.a.num_instances = M;
    c.a.softmax_mode = 1;
    c.a.blocks[0] = C; c.a.strides[0] = C;
    c.a.normalize_offsets = 1;
    if (shared1) {
        c.a.shared_offset_region[0] = 1;
    } else {
        c.a.unshared_offset_region[0] = 2;
    }
    const int in[4] = {B, C, HW, HW};
    memcpy(c.in, in, sizeof(in));
    SN_OK(simnets_mex_out_shape(&c.a, c.in, c.out, c.off));
    c.off_count = (size_t)c.off[0] * c.off[1] * c.off[2] * c.off[3] * c.off[4];
    std::vector<float> off(c.off_count);
    fill_normal(off, 4567 + C, 0.1f);
    dump(tag + "_off", off);
    c.o = upload(off);
    if (input) {
        c.x = const_cast<float *>(input);
    } else {
        std::vector<float> x((size_t)B * C * HW * HW);
        fill_normal(x, 1234, 1.0f);
        dump(tag + "_x", x);
        c.x = upload(x);
    }
    HIP_OK(hipMalloc(&c.y, (size_t)c.out[0] * c.out[1] * c.out[2] * c.out[3] * sizeof(float)));
    SN_OK(simnets_hip_mex_workspace_bytes(&c.a, c.in, &c.ws_bytes));
    HIP_OK(hipMalloc(&c.ws, std::max<size_t>(c.ws_bytes, 256)));
    return c;
}

static void run_sim(SimCase &c, hipStream_t s)
{
    SN_OK(simnets_hip_similarity_fwd(&c.a, c.in, c.tp, c.tp, c.x, c.t, c.w, c.y, c.ws, c.ws_bytes, s));
}
static void run_mex(MexCase &c, hipStream_t s)
{
    SN_OK(simnets_hip_mex_fwd(&c.a, c.in, c.x, c.o, c.off_count, c.y, c.ws, c.ws_bytes, s));
}

static void report(const char *name, double gmac, double bytes, double flop_per_gmac, float ms, int steps)
{
    const double gmacs = gmac / (ms * 1e-3);
    printf("{\"config\": \"%s\", \"ms\": %.4f, \"steps\": %d, \"gmac_per_s_G\": %.1f, \"tflops\": %.2f, "
           "\"frac_fp32_peak_157.3\": %.4f, \"hbm_frac_8TBs\": %.4f}\n",
           name, ms, steps, gmacs / 1e9, gmacs * flop_per_gmac / 1e12, gmacs * flop_per_gmac / 157.3e12,
           bytes / (ms * 1e-3) / 8e12);
}

int main(int argc, char **argv)
{
    int config = 0, steps = 20, warmup = 5, algo = SIMNETS_ALGO_AUTO;
    bool peaks = false;
    for (int i = 1; i < argc; ++i) {
        std::string a = argv[i];
        if (a == "--peaks") peaks = true;
        else if (a == "--config" && i + 1 < argc) config = atoi(argv[++i]);
        else if (a == "--steps" && i + 1 < argc) steps = atoi(argv[++i]);
        else if (a == "--warmup" && i + 1 < argc) warmup = atoi(argv[++i]);
        else if (a == "--dump" && i + 1 < argc) g_dump_dir = argv[++i];
        else if (a == "--algo" && i + 1 < argc) {
            std::string v = argv[++i];
            algo = v == "direct" ? SIMNETS_ALGO_DIRECT : v == "sqrtw" ? SIMNETS_ALGO_SQRTW : v == "mfma" ? SIMNETS_ALGO_MFMA : SIMNETS_ALGO_AUTO;
        } else {
            fprintf(stderr, "usage: %s --peaks | --config N [--algo direct|sqrtw|mfma] [--steps K] [--warmup W] [--dump DIR]\n", argv[0]);
            return 2;
        }
    }
    hipStream_t s;
    HIP_OK(hipStreamCreate(&s));
    if (peaks)
        run_peaks(s);
    if (config == 1) {
        SimCase c = make_similarity("c1", 64, 1, 28, 28, 32, 2, 2, 2, 2, true, algo, 0);
        for (int i = 0; i < warmup; ++i) run_sim(c, s);
        float ms = time_ms(s, steps, [&] { run_sim(c, s); });
        report("config1 similarity L2 norm ignore-nan 64x1x28x28 -> 64x32x16x16", 2097152.0, 2298880.0, 6, ms, steps);
        checksum("config1", c.y, count4(c.out), s);
        HIP_OK(hipMemsetAsync(c.y, 0xff, count4(c.out) * sizeof(float), s));
        SN_OK(simnets_hip_similarity_prepare(&c.a, c.in, c.tp, c.tp, c.t, c.w, c.ws, c.ws_bytes, s));
        auto prepared = [&] { SN_OK(simnets_hip_similarity_fwd_prepared(&c.a, c.in, c.tp, c.x, c.ws, c.ws_bytes, c.y, s)); };
        for (int i = 0; i < warmup; ++i) prepared();
        ms = time_ms(s, 10 * steps, prepared);
        report("config1, parameters prepared once (simnets_hip_similarity_fwd_prepared)", 2097152.0, 2298880.0, 6, ms, 10 * steps);
        checksum("config1 prepared", c.y, count4(c.out), s);
    } else if (config == 2) {
        MexCase c = make_mex("c2", 64, 32, 16, 64, false, nullptr);
        for (int i = 0; i < warmup; ++i) run_mex(c, s);
        float ms = time_ms(s, steps, [&] { run_mex(c, s); });
        report("config2 mex 64x32x16x16 -> 64x64x16x16", 33554432.0, 6324224.0, 5, ms, steps);
        checksum("config2", c.y, count4(c.out), s);
        HIP_OK(hipMemsetAsync(c.y, 0xff, count4(c.out) * sizeof(float), s));
        SN_OK(simnets_hip_mex_prepare(&c.a, c.in, c.o, c.off_count, c.ws, c.ws_bytes, s));
        auto prepared = [&] { SN_OK(simnets_hip_mex_fwd_prepared(&c.a, c.in, c.x, c.ws, c.ws_bytes, c.y, s)); };
        for (int i = 0; i < warmup; ++i) prepared();
        ms = time_ms(s, 10 * steps, prepared);
        report("config2, offsets prepared once (simnets_hip_mex_fwd_prepared)", 33554432.0, 6324224.0, 5, ms, 10 * steps);
        checksum("config2 prepared", c.y, count4(c.out), s);
    } else if (config == 3) {
        for (int l1 = 0; l1 < 2; ++l1) {
            if (l1 && algo != SIMNETS_ALGO_AUTO && algo != SIMNETS_ALGO_DIRECT)
                break;
            SimCase c = make_similarity("c3", 256, 64, 32, 32, 128, 3, 3, 1, 1, false, algo, l1);
            for (int i = 0; i < warmup; ++i) run_sim(c, s);
            float ms = time_ms(s, steps, [&] { run_sim(c, s); });
            report(l1 ? "config3 similarity L1 256x64x32x32 x 128 templates 3x3" : "config3 similarity L2 256x64x32x32 x 128 templates 3x3",
                   19327352832.0, 201916416.0, l1 ? 3 : 4, ms, steps);
            SN_OK(simnets_hip_similarity_prepare(&c.a, c.in, c.tp, c.tp, c.t, c.w, c.ws, c.ws_bytes, s));
            ms = time_ms(s, steps, [&] { SN_OK(simnets_hip_similarity_fwd_prepared(&c.a, c.in, c.tp, c.x, c.ws, c.ws_bytes, c.y, s)); });
            report(l1 ? "config3 similarity L1, parameters prepared once" : "config3 similarity L2, parameters prepared once",
                   19327352832.0, 201916416.0, l1 ? 3 : 4, ms, steps);
            checksum(l1 ? "config3 L1" : "config3 L2", c.y, count4(c.out), s);
            HIP_OK(hipFree(c.x)); HIP_OK(hipFree(c.y)); HIP_OK(hipFree(c.ws));
        }
    } else if (config == 4) {
        const int B = 512;
        SimCase sc = make_similarity("c4", B, 1, 28, 28, 32, 2, 2, 2, 2, true, algo, 0);
        std::vector<MexCase> mex;
        std::vector<float *> pooled;
        const float *cur = sc.y;
        int ch = 32, hw = 16;
        for (int l = 0; l < 4; ++l) {
            mex.push_back(make_mex("c4_mex" + std::to_string(l), B, ch, hw, 2 * ch, false, cur));
            float *p;
            HIP_OK(hipMalloc(&p, (size_t)B * 2 * ch * (hw / 2) * (hw / 2) * sizeof(float)));
            pooled.push_back(p);
            cur = p;
            ch *= 2;
            hw /= 2;
        }
        mex.push_back(make_mex("c4_mex4", B, ch, 1, 10, true, cur));
        const size_t n_final = count4(mex[4].out);
        auto stack = [&] {
            run_sim(sc, s);
            for (int l = 0; l < 4; ++l) {
                run_mex(mex[l], s);
                SN_OK(simnets_hip_sum_pool_fwd(mex[l].out, 2, 2, mex[l].y, pooled[l], s));
            }
            run_mex(mex[4], s);
        };
        for (int i = 0; i < warmup; ++i) stack();
        float ms = time_ms(s, steps, stack);
        report("config4 missing-data stack batch 512", 512.0 * 32 * 256 * 4 + 4 * 268435456.0 + 512.0 * 10 * 512, 0, 5, ms, steps);
        checksum("config4 separate calls", mex[4].y, n_final, s);
        HIP_OK(hipMemsetAsync(mex[4].y, 0xff, n_final * sizeof(float), s));
        // the same stack with each MEX + pooling pair as one call (simnets_hip_mex_sum_pool_fwd)
        std::vector<void *> fws(4);
        std::vector<size_t> fbytes(4);
        for (int l = 0; l < 4; ++l) {
            SN_OK(simnets_hip_mex_sum_pool_workspace_bytes(&mex[l].a, mex[l].in, 2, 2, &fbytes[l]));
            HIP_OK(hipMalloc(&fws[l], std::max<size_t>(fbytes[l], 256)));
        }
        auto fused = [&] {
            run_sim(sc, s);
            for (int l = 0; l < 4; ++l)
                SN_OK(simnets_hip_mex_sum_pool_fwd(&mex[l].a, mex[l].in, mex[l].x, mex[l].o, mex[l].off_count, 2, 2,
                                                   pooled[l], fws[l], fbytes[l], s));
            run_mex(mex[4], s);
        };
        for (int i = 0; i < warmup; ++i) fused();
        ms = time_ms(s, steps, fused);
        report("config4 missing-data stack batch 512, MEX + pooling fused", 512.0 * 32 * 256 * 4 + 4 * 268435456.0 + 512.0 * 10 * 512, 0, 5, ms, steps);
        checksum("config4 fused pooling", mex[4].y, n_final, s);
        HIP_OK(hipMemsetAsync(mex[4].y, 0xff, n_final * sizeof(float), s));
        // ... and with the Similarity layer evaluated inside the first of those kernels
        size_t f0bytes = 0;
        SN_OK(simnets_hip_similarity_mex_sum_pool_workspace_bytes(&sc.a, sc.in, sc.tp, &mex[0].a, 2, 2, &f0bytes));
        void *f0ws;
        HIP_OK(hipMalloc(&f0ws, std::max<size_t>(f0bytes, 256)));
        auto fused3 = [&] {
            SN_OK(simnets_hip_similarity_mex_sum_pool_fwd(&sc.a, sc.in, sc.tp, sc.x, sc.t, sc.w, &mex[0].a, mex[0].o,
                                                          mex[0].off_count, 2, 2, pooled[0], f0ws, f0bytes, s));
            for (int l = 1; l < 4; ++l)
                SN_OK(simnets_hip_mex_sum_pool_fwd(&mex[l].a, mex[l].in, mex[l].x, mex[l].o, mex[l].off_count, 2, 2,
                                                   pooled[l], fws[l], fbytes[l], s));
            run_mex(mex[4], s);
        };
        for (int i = 0; i < warmup; ++i) fused3();
        ms = time_ms(s, steps, fused3);
        report("config4 missing-data stack batch 512, Similarity + MEX + pooling fused", 512.0 * 32 * 256 * 4 + 4 * 268435456.0 + 512.0 * 10 * 512, 0, 5, ms, steps);
        checksum("config4 fused similarity and pooling", mex[4].y, n_final, s);
        HIP_OK(hipMemsetAsync(mex[4].y, 0xff, n_final * sizeof(float), s));
        // ... and with every layer's parameters packed once (the *_prepare / *_fwd_prepared entry points): the
        // workspaces above double as the prepared buffers, five launches per stack
        SN_OK(simnets_hip_similarity_mex_sum_pool_prepare(&sc.a, sc.in, sc.tp, sc.t, sc.w, &mex[0].a, mex[0].o,
                                                          mex[0].off_count, 2, 2, f0ws, f0bytes, s));
        for (int l = 1; l < 4; ++l)
            SN_OK(simnets_hip_mex_sum_pool_prepare(&mex[l].a, mex[l].in, mex[l].o, mex[l].off_count, 2, 2, fws[l],
                                                   fbytes[l], s));
        SN_OK(simnets_hip_mex_prepare(&mex[4].a, mex[4].in, mex[4].o, mex[4].off_count, mex[4].ws, mex[4].ws_bytes, s));
        auto prepared = [&] {
            SN_OK(simnets_hip_similarity_mex_sum_pool_fwd_prepared(&sc.a, sc.in, sc.tp, sc.x, &mex[0].a, 2, 2, f0ws, f0bytes,
                                                                   pooled[0], s));
            for (int l = 1; l < 4; ++l)
                SN_OK(simnets_hip_mex_sum_pool_fwd_prepared(&mex[l].a, mex[l].in, mex[l].x, 2, 2, fws[l], fbytes[l],
                                                            pooled[l], s));
            SN_OK(simnets_hip_mex_fwd_prepared(&mex[4].a, mex[4].in, mex[4].x, mex[4].ws, mex[4].ws_bytes, mex[4].y, s));
        };
        for (int i = 0; i < warmup; ++i) prepared();
        ms = time_ms(s, steps, prepared);
        report("config4 missing-data stack batch 512, fused, parameters prepared once", 512.0 * 32 * 256 * 4 + 4 * 268435456.0 + 512.0 * 10 * 512, 117e6, 5, ms, steps);
        checksum("config4 fused prepared", mex[4].y, n_final, s);
        HIP_OK(hipMemsetAsync(mex[4].y, 0xff, n_final * sizeof(float), s));
        // ... and the same five launches recorded once and replayed as a HIP graph (a serving loop: the calls are
        // kernel launches on the caller's stream and nothing else, so a capture holds exactly those)
        hipGraph_t graph;
        hipGraphExec_t exec;
        HIP_OK(hipStreamSynchronize(s));
        HIP_OK(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
        prepared();
        HIP_OK(hipStreamEndCapture(s, &graph));
        HIP_OK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
        auto replay = [&] { HIP_OK(hipGraphLaunch(exec, s)); };
        for (int i = 0; i < warmup; ++i) replay();
        ms = time_ms(s, steps, replay);
        report("config4 missing-data stack batch 512, fused, parameters prepared once, replayed from a HIP graph", 512.0 * 32 * 256 * 4 + 4 * 268435456.0 + 512.0 * 10 * 512, 117e6, 5, ms, steps);
        checksum("config4 fused prepared graph", mex[4].y, n_final, s);
        HIP_OK(hipGraphExecDestroy(exec));
        HIP_OK(hipGraphDestroy(graph));
    }
    else if (config == 5) {
        // backward at the config-3 and config-2 shapes, upstream gradients ~N(0,1)
        for (int l1 = 0; l1 < 2; ++l1) {
            SimCase c = make_similarity("c5", 256, 64, 32, 32, 128, 3, 3, 1, 1, false, SIMNETS_ALGO_AUTO, l1);
            const size_t n_out = (size_t)c.out[0] * c.out[1] * c.out[2] * c.out[3];
            std::vector<float> g(n_out);
            fill_normal(g, 6789, 1.0f);
            dump("c5_g", g);
            float *dg = upload(g), *dx, *dt, *dw;
            HIP_OK(hipMalloc(&dx, (size_t)256 * 64 * 32 * 32 * sizeof(float)));
            HIP_OK(hipMalloc(&dt, (size_t)128 * 64 * 9 * sizeof(float)));
            HIP_OK(hipMalloc(&dw, (size_t)128 * 64 * 9 * sizeof(float)));
            size_t wx = 0, wp = 0;
            SN_OK(simnets_hip_similarity_grad_workspace_bytes(&c.a, c.in, c.tp, &wx, &wp));
            void *ws;
            HIP_OK(hipMalloc(&ws, std::max<size_t>(std::max(wx, wp), 256)));
            auto gx = [&] { SN_OK(simnets_hip_similarity_input_grad(&c.a, c.in, c.tp, c.tp, c.x, c.t, c.w, dg, dx, ws, wx, s)); };
            auto gp = [&] { SN_OK(simnets_hip_similarity_params_grad(&c.a, c.in, c.tp, c.tp, c.x, c.t, c.w, dg, dt, dw, ws, wp, s)); };
            for (int i = 0; i < warmup; ++i) { gx(); gp(); }
            float ms = time_ms(s, steps, gx);
            // input grad: read g and x, write dx; 2 flop per term for L2 (fma, fma), 5 for L1
            report(l1 ? "config5 similarity input grad L1 (config-3 shape)" : "config5 similarity input grad L2 (config-3 shape)",
                   19327352832.0, (n_out + 2.0 * 256 * 64 * 32 * 32) * 4, l1 ? 5 : 4, ms, steps);
            ms = time_ms(s, steps, gp);
            report(l1 ? "config5 similarity params grad L1 (config-3 shape)" : "config5 similarity params grad L2 (config-3 shape)",
                   19327352832.0, (n_out + 256.0 * 64 * 32 * 32) * 4, l1 ? 6 : 5, ms, steps);
            checksum(l1 ? "config5 L1 input grad" : "config5 L2 input grad", dx, (size_t)256 * 64 * 32 * 32, s);
            checksum(l1 ? "config5 L1 templates grad" : "config5 L2 templates grad", dt, (size_t)128 * 64 * 9, s);
            checksum(l1 ? "config5 L1 weights grad" : "config5 L2 weights grad", dw, (size_t)128 * 64 * 9, s);
            HIP_OK(hipFree(dg)); HIP_OK(hipFree(dx)); HIP_OK(hipFree(dt)); HIP_OK(hipFree(dw)); HIP_OK(hipFree(ws));
            HIP_OK(hipFree(c.x)); HIP_OK(hipFree(c.y));
        }
        {
            MexCase c = make_mex("c5_mex", 64, 32, 16, 64, false, nullptr);
            run_mex(c, s);
            const size_t n_out = (size_t)c.out[0] * c.out[1] * c.out[2] * c.out[3];
            std::vector<float> g(n_out);
            fill_normal(g, 6789, 1.0f);
            dump("c5_mex_g", g);
            float *dg = upload(g), *dx, *doff;
            HIP_OK(hipMalloc(&dx, (size_t)64 * 32 * 16 * 16 * sizeof(float)));
            HIP_OK(hipMalloc(&doff, c.off_count * sizeof(float)));
            size_t wx = 0, wo = 0;
            SN_OK(simnets_hip_mex_grad_workspace_bytes(&c.a, c.in, &wx, &wo));
            void *ws;
            HIP_OK(hipMalloc(&ws, std::max<size_t>(std::max(wx, wo), 256)));
            auto gx = [&] { SN_OK(simnets_hip_mex_input_grad(&c.a, c.in, c.x, c.o, c.off_count, c.y, dg, dx, ws, wx, s)); };
            auto go = [&] { SN_OK(simnets_hip_mex_offsets_grad(&c.a, c.in, c.x, c.o, c.off_count, c.y, dg, doff, ws, wo, s)); };
            for (int i = 0; i < warmup; ++i) { gx(); go(); }
            float ms = time_ms(s, steps, gx);
            report("config5 mex input grad (config-2 shape)", 33554432.0, (2.0 * n_out + 2.0 * 64 * 32 * 256) * 4, 5, ms, steps);
            ms = time_ms(s, steps, go);
            report("config5 mex offsets grad (config-2 shape)", 33554432.0, (2.0 * n_out + 64.0 * 32 * 256) * 4, 5, ms, steps);
            checksum("config5 mex input grad", dx, (size_t)64 * 32 * 16 * 16, s);
            checksum("config5 mex offsets grad", doff, c.off_count, s);
        }
    }
    HIP_OK(hipStreamSynchronize(s));
    HIP_OK(hipStreamDestroy(s));
    return 0;
}
