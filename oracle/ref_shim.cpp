// extern "C" doorway onto the reference's own header-only CPU building blocks.
//
// Test infrastructure.  This translation unit is compiled against the headers where they
// lie in the reference checkout (-I<reference>/include, see oracle/Makefile) and produces
// oracle/_ref/libsimnets_ref.so.  It contains no reference code: it only instantiates the
// reference templates
//     ggemm_cpu, ggemm_readc_cpu, interlace_cpu            include/utils/ggemm_cpu.hpp
//     sim_l1_forward, sim_l2_forward, sim_l2_normalized_forward   include/utils/similarity_utils.hpp
//     mex_forward_exp, mex_forward_out, split_patches_cpu,
//     sim_*_backward_weights, sim_*_backward_bottom (similarity_utils.hpp:82-150),
//     mex_backward_bottom_finite/infinite (mex_utils.hpp:31-46)   include/utils/mex_utils.hpp
// with the template arguments their callers use (src/kernels/similarity_kernel_cpu.cpp:84-116,
// src/kernels/mex_kernel_cpu.cpp:15-37, :134-157) so that the C restatement in
// simnets_oracle.c can be compared with them bit for bit.
//
// Only these three headers build here: every other file of the reference's CPU path
// includes TensorFlow headers, which this image does not have.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>

#include "utils/ggemm_cpu.hpp"
#include "utils/similarity_utils.hpp"
#include "utils/mex_utils.hpp"

namespace {

template <typename T>
void ggemm_similarity(int mode, int M, int N, int K, const T *A_interlaced, const T *B, T *C, T fudge)
{
    using V2 = typename vec<T>::vec2;
    const V2 *A = reinterpret_cast<const V2 *>(A_interlaced);
    switch (mode) {
    case 0:
        ggemm_cpu<V2, T, T, uint8_t, sim_l1_forward<T>, ggemm_add<T>, false>(M, N, K, A, B, C, 0, 0);
        break;
    case 1:
        ggemm_cpu<V2, T, T, uint8_t, sim_l2_forward<T, false>, ggemm_add<T>, false>(M, N, K, A, B, C, 0, 0);
        break;
    case 2:
        ggemm_cpu<V2, T, T, T, sim_l2_normalized_forward<T, false, false>, ggemm_add<T>, false>(M, N, K, A, B, C,
                                                                                                0, fudge);
        break;
    default:
        ggemm_cpu<V2, T, T, T, sim_l2_normalized_forward<T, false, true>, ggemm_add<T>, false>(M, N, K, A, B, C,
                                                                                               0, fudge);
        break;
    }
}

// The call sequence of mex_forward_cpu (src/kernels/mex_kernel_cpu.cpp:11-38), which itself
// sits in a TensorFlow-dependent file, re-issued against the reference templates.
template <typename T>
void mex_forward(int M, int N, int K, bool softmax_mode, T epsilon, const T *offsets, const T *in, T *out,
                 int batch)
{
    const T init_value = epsilon > 0 ? -INFINITY : INFINITY;
    if (epsilon > 0) {
        ggemm_cpu<T, T, T, uint8_t, ggemm_add<T, uint8_t>, ggemm_max<T>, false, true, true, true>(
            M, N, K, offsets, in, out, init_value, 0, batch);
    } else {
        ggemm_cpu<T, T, T, uint8_t, ggemm_add<T, uint8_t>, ggemm_min<T>, false, true, true, true>(
            M, N, K, offsets, in, out, init_value, 0, batch);
    }
    if (std::isfinite(epsilon)) {
        ggemm_readc_cpu<false, false, T, T, T, typename vec<T>::vec2, mex_forward_exp<T>, ggemm_add<T>, true,
                        mex_forward_out<T>, true, true, true, true>(
            M, N, K, offsets, in, out, out, 0, make_vec2<T>(epsilon, softmax_mode ? T(0) : (T)-std::log(K)),
            batch);
    }
}

} // namespace

namespace {
template <typename T>
void sim_backward_weights(int mode, T err, T x, T t, T w, T fudge, T *out2)
{
    using V2 = typename vec<T>::vec2;
    V2 p = make_vec2<T>(t, w), r;
    switch (mode) {
    case 0: r = sim_l1_backward_weights<T>(err, x, p, 0); break;
    case 1: r = sim_l2_backward_weights<T, false>(err, x, p, 0); break;
    case 2: r = sim_l2_normalized_backward_weights<T, false, false>(err, x, p, fudge); break;
    default: r = sim_l2_normalized_backward_weights<T, false, true>(err, x, p, fudge); break;
    }
    out2[0] = r.x;
    out2[1] = r.y;
}
template <typename T>
T sim_backward_bottom(int mode, T t, T w, T err, T data)
{
    using V2 = typename vec<T>::vec2;
    V2 p = make_vec2<T>(t, w);
    switch (mode) {
    case 0: return sim_l1_backward_bottom<T>(p, err, data, 0);
    case 1: return sim_l2_backward_bottom<T, false>(p, err, data, 0);
    case 2: return sim_l2_normalized_backward_bottom<T, false, false>(p, err, data, T(0));
    default: return sim_l2_normalized_backward_bottom<T, false, true>(p, err, data, T(0));
    }
}
template <typename T>
T mex_backward_term(int finite, T offset, T top_data, T top_diff, T data, T ex, T ey)
{
    using V2 = typename vec<T>::vec2;
    if (finite)
        return mex_backward_bottom_finite<T>(offset, make_vec2<T>(top_data, top_diff), data, make_vec2<T>(ex, ey));
    return mex_backward_bottom_infinite<T>(offset, make_vec2<T>(top_data, top_diff), data, 0);
}
} // namespace

extern "C" {

void ref_sim_backward_weights_fn_f32(int mode, float err, float x, float t, float w, float fudge, float *o) { sim_backward_weights<float>(mode, err, x, t, w, fudge, o); }
void ref_sim_backward_weights_fn_f64(int mode, double err, double x, double t, double w, double fudge, double *o) { sim_backward_weights<double>(mode, err, x, t, w, fudge, o); }
float ref_sim_backward_bottom_fn_f32(int mode, float t, float w, float err, float data) { return sim_backward_bottom<float>(mode, t, w, err, data); }
double ref_sim_backward_bottom_fn_f64(int mode, double t, double w, double err, double data) { return sim_backward_bottom<double>(mode, t, w, err, data); }
float ref_mex_backward_term_fn_f32(int finite, float offset, float top_data, float top_diff, float data, float ex, float ey) { return mex_backward_term<float>(finite, offset, top_data, top_diff, data, ex, ey); }
double ref_mex_backward_term_fn_f64(int finite, double offset, double top_data, double top_diff, double data, double ex, double ey) { return mex_backward_term<double>(finite, offset, top_data, top_diff, data, ex, ey); }

int ref_ggemm_padded_output_size(int M, int N) { return ggemm_padded_output_size(M, N); }

void ref_interlace_f32(int n, const float *a, const float *b, float *o)
{
    interlace_cpu<float>(n, a, b, reinterpret_cast<vec<float>::vec2 *>(o));
}

void ref_ggemm_similarity_f32(int mode, int M, int N, int K, const float *A, const float *B, float *C, float fudge)
{
    ggemm_similarity<float>(mode, M, N, K, A, B, C, fudge);
}
void ref_ggemm_similarity_f64(int mode, int M, int N, int K, const double *A, const double *B, double *C,
                              double fudge)
{
    ggemm_similarity<double>(mode, M, N, K, A, B, C, fudge);
}

void ref_mex_forward_f32(int M, int N, int K, int softmax_mode, float epsilon, const float *offsets,
                         const float *in, float *out, int batch)
{
    mex_forward<float>(M, N, K, softmax_mode != 0, epsilon, offsets, in, out, batch);
}
void ref_mex_forward_f64(int M, int N, int K, int softmax_mode, double epsilon, const double *offsets,
                         const double *in, double *out, int batch)
{
    mex_forward<double>(M, N, K, softmax_mode != 0, epsilon, offsets, in, out, batch);
}

void ref_split_patches_f32(int reverse, int N, int Dim, int W, int H, int C, int W_Gs, int H_Gs, int C_Gs,
                           int W_Step, int H_Step, int C_Step, float *in, float *out, int use_unshared)
{
    if (reverse)
        split_patches_cpu<float, true>(N, Dim, W, H, C, W_Gs, H_Gs, C_Gs, W_Step, H_Step, C_Step, in, out,
                                       use_unshared != 0);
    else
        split_patches_cpu<float, false>(N, Dim, W, H, C, W_Gs, H_Gs, C_Gs, W_Step, H_Step, C_Step, in, out,
                                        use_unshared != 0);
}
void ref_split_patches_f64(int reverse, int N, int Dim, int W, int H, int C, int W_Gs, int H_Gs, int C_Gs,
                           int W_Step, int H_Step, int C_Step, double *in, double *out, int use_unshared)
{
    if (reverse)
        split_patches_cpu<double, true>(N, Dim, W, H, C, W_Gs, H_Gs, C_Gs, W_Step, H_Step, C_Step, in, out,
                                        use_unshared != 0);
    else
        split_patches_cpu<double, false>(N, Dim, W, H, C, W_Gs, H_Gs, C_Gs, W_Step, H_Step, C_Step, in, out,
                                         use_unshared != 0);
}
}
