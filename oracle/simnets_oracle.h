/*
 * CPU oracle for the SimNets Similarity and MEX forward operators.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, loop for loop, the CPU
 * code path of HUJI-Deep/simnets-tf so that the HIP library can be checked against it and
 * so that a CPU baseline can be timed beside the GPU numbers.  Only the test-suite, the
 * smoke check and the cpu_baseline leg of the benchmark may link or load it; the shipped
 * library never calls into it and has no CPU fallback.
 *
 * Every function names the reference file:line it follows (paths relative to the
 * reference checkout).  Each entry point exists in an fp32 flavour (suffix _f32, the
 * precision the HIP path computes in, bit-faithful to the reference's float instantiation
 * when built without FP contraction) and an fp64 flavour (suffix _f64, the reference's
 * double instantiation, used as the high-precision yardstick).
 *
 * How each part is pinned (see tests/test_oracle_*.py):
 *   - ggemm / ggemm_readc / combine functors / interlace / split_patches: bit-exact against
 *     the reference's own headers compiled into oracle/_ref (tests skip if absent).
 *   - im2col_3d: torch.nn.functional.unfold (zero padding), an independent per-element
 *     index formula for NaN padding, closed-form NaN counts.
 *   - dimension_out_size / MEX region arithmetic: the known-answer shapes held by the
 *     reference's Keras tests, the 2025-region sanity case, tiling invariants.
 *   - Similarity / MEX orchestration: cross-checked against the brute-force restatements
 *     of SimilarityRef / MexRef (the comparison the reference's own tests make) and against
 *     library routines (cdist, logsumexp) on the special cases that reduce to them.
 *   No function of this oracle is "parity unpinned".
 */
#ifndef SIMNETS_ORACLE_H
#define SIMNETS_ORACLE_H

#ifdef __cplusplus
extern "C" {
#endif

enum { SO_SIM_L1 = 0, SO_SIM_L2 = 1 };

/* include/utils/im2col.hpp:101-108 */
int so_dimension_out_size(int image_size, int pad_size, int patch_size, int stride, int round_down);

/* include/utils/ggemm_cpu.hpp:456-460 */
int so_ggemm_padded_output_size(int M, int N);

typedef struct so_similarity_args {
    int batch, channels, height, width; /* input  [B,C,H,W]                            */
    int num_instances;                  /* templates/weights [O,C,bh,bw]               */
    int block_h, block_w;               /* attr blocks                                 */
    int stride_h, stride_w;             /* attr strides                                */
    int pad_h, pad_w;                   /* attr padding                                */
    int similarity_function;            /* SO_SIM_L1 | SO_SIM_L2                       */
    int normalization_term;
    float normalization_term_fudge;
    int ignore_nan_input;
    float out_of_bounds_value;
    /* 1: add the -0.5*K*log(2pi) constant to the WHOLE output tensor once per batch
     *    iteration, exactly as similarity_kernel_cpu.cpp:69,118-120 does (image n ends up
     *    with it (B-n) times).  0: add it once per output, the SimilarityRef semantics
     *    (similarity_ref_kernel_cpu.cpp:89-93).  Identical for batch 1. */
    int norm_const_every_iteration;
    int threads;                        /* >1: spread the batch loop over pthreads (NOT reference behaviour) */
} so_similarity_args;

/* out dims: similarity_kernel_common.hpp:147-158.  Returns 0, or <0 on invalid arguments
 * (similarity_kernel_common.hpp:85-110,160-163). */
int so_similarity_out_dims(const so_similarity_args *a, int *out_h, int *out_w);

/* src/kernels/similarity_kernel_cpu.cpp:19-122 (interlace -> per image im2col_3d -> ggemm). */
int so_similarity_fwd_f32(const so_similarity_args *a, const float *input, const float *templates,
                          const float *weights, float *output);
int so_similarity_fwd_f64(const so_similarity_args *a, const double *input, const double *templates,
                          const double *weights, double *output);
/* src/kernels/similarity_ref_kernel_cpu.cpp:61-102 (seven nested loops). */
int so_similarity_ref_f32(const so_similarity_args *a, const float *input, const float *templates,
                          const float *weights, float *output);
int so_similarity_ref_f64(const so_similarity_args *a, const double *input, const double *templates,
                          const double *weights, double *output);

typedef struct so_mex_args {
    int batch, channels, height, width;
    int num_instances;
    int softmax_mode;
    int n_padding;  int padding[3];     /* 2 or 3 entries; -1 -> image dim (mex_kernel_common.cpp:8-27) */
    int n_strides;  int strides[3];
    int n_blocks;   int blocks[3];
    float epsilon;                      /* may be +-inf */
    float blocks_out_of_bounds_value;
    int blocks_round_down;
    int use_unshared_regions;
    int n_shared;   int shared_offset_region[3];    /* 1 or 3 entries */
    int n_unshared; int unshared_offset_region[3];  /* 1 or 3 entries */
    int threads;
} so_mex_args;

/* Everything MexDimensionsData::CalculateDimensions derives (mex_kernel_common.cpp:63-158). */
typedef struct so_mex_dims {
    int pad_c, pad_h, pad_w, stride_c, stride_h, stride_w, block_c, block_h, block_w;
    int channels_out, height_out, width_out, channels_out_total;
    int shared_region_c, shared_region_h, shared_region_w;
    int offsets_c, offsets_h, offsets_w;
    int num_regions, region_size;
    int M, K, N;
    int is_1x1;
} so_mex_dims;

int so_mex_calc_dims(const so_mex_args *a, so_mex_dims *d);

/* src/kernels/mex_kernel_cpu.cpp:60-159 (im2col_3d -> split_patches -> two-pass LSE -> scatter). */
int so_mex_fwd_f32(const so_mex_args *a, const float *input, const float *offsets, float *output);
int so_mex_fwd_f64(const so_mex_args *a, const double *input, const double *offsets, double *output);
/* src/kernels/mex_kernel_cpu.cpp:166-207, 218-287 (MexRef). */
int so_mex_ref_f32(const so_mex_args *a, const float *input, const float *offsets, float *output);
int so_mex_ref_f64(const so_mex_args *a, const double *input, const double *offsets, double *output);

/* python/simnets/keras.py:155-160: offsets[r,m,:] -= logsumexp(offsets[r,m,:]); rows = R*M, K = block volume.
 * fp32 flavour follows the usual max-shifted evaluation of reduce_logsumexp. */
void so_normalize_offsets_f32(int rows, int K, const float *in, float *out);
void so_normalize_offsets_f64(int rows, int K, const double *in, double *out);

/* Building blocks, exported so that they can be compared one by one with the reference's
 * own headers (oracle/_ref) and with library routines. */
/* src/utils/im2col.cpp:247-280 */
void so_im2col_3d_f32(const float *im, int channels, int height, int width, int patch_c, int patch_h,
                      int patch_w, int pad_c, int pad_h, int pad_w, int stride_c, int stride_h,
                      int stride_w, float *col, int round_down, float oob);
void so_im2col_3d_f64(const double *im, int channels, int height, int width, int patch_c, int patch_h,
                      int patch_w, int pad_c, int pad_h, int pad_w, int stride_c, int stride_h,
                      int stride_w, double *col, int round_down, double oob);
/* include/utils/mex_utils.hpp:69-116 */
void so_split_patches_f32(int reverse, int N, int Dim, int W, int H, int C, int W_Gs, int H_Gs, int C_Gs,
                          int W_Step, int H_Step, int C_Step, float *in, float *out, int use_unshared);
void so_split_patches_f64(int reverse, int N, int Dim, int W, int H, int C, int W_Gs, int H_Gs, int C_Gs,
                          int W_Step, int H_Step, int C_Step, double *in, double *out, int use_unshared);
/* ggemm_cpu with the Similarity combines (ggemm_cpu.hpp:462-511 + similarity_utils.hpp:17-80).
 * mode: 0 L1, 1 L2, 2 L2 normalized, 3 L2 normalized + ignore NaN.  A is the interlaced
 * (template, weight) array of M*K pairs. */
void so_ggemm_similarity_f32(int mode, int M, int N, int K, const float *A_interlaced, const float *B,
                             float *C, float fudge);
void so_ggemm_similarity_f64(int mode, int M, int N, int K, const double *A_interlaced, const double *B,
                             double *C, double fudge);
/* mex_forward_cpu (mex_kernel_cpu.cpp:11-38): batched max pass + exp/sum/log pass. */
void so_mex_forward_f32(int M, int N, int K, int softmax_mode, float epsilon, const float *offsets,
                        const float *in, float *out, int batch);
void so_mex_forward_f64(int M, int N, int K, int softmax_mode, double epsilon, const double *offsets,
                        const double *in, double *out, int batch);

/* ---- backward operators --------------------------------------------------------------------
 * src/kernels/similarity_grad_kernel_cpu.cpp:158-270 / :23-146, src/kernels/mex_grad_kernel_cpu.cpp:32-208 / :220-369.
 * Pinned by central differences of the fp64 forward oracle and by torch.autograd on the closed forms
 * (tests/test_oracle_pins.py); the backward functors are pinned bit-exactly against oracle/_ref. */
int so_similarity_input_grad_f32(const so_similarity_args *a, const float *input, const float *templates,
                                 const float *weights, const float *output_grad, float *input_grad);
int so_similarity_input_grad_f64(const so_similarity_args *a, const double *input, const double *templates,
                                 const double *weights, const double *output_grad, double *input_grad);
int so_similarity_params_grad_f32(const so_similarity_args *a, const float *input, const float *templates,
                                  const float *weights, const float *output_grad, float *templates_grad,
                                  float *weights_grad);
int so_similarity_params_grad_f64(const so_similarity_args *a, const double *input, const double *templates,
                                  const double *weights, const double *output_grad, double *templates_grad,
                                  double *weights_grad);
int so_mex_input_grad_f32(const so_mex_args *a, const float *input, const float *offsets, const float *output,
                          const float *output_grad, float *input_grad);
int so_mex_input_grad_f64(const so_mex_args *a, const double *input, const double *offsets, const double *output,
                          const double *output_grad, double *input_grad);
int so_mex_offsets_grad_f32(const so_mex_args *a, const float *input, const float *offsets, const float *output,
                            const float *output_grad, float *offsets_grad);
int so_mex_offsets_grad_f64(const so_mex_args *a, const double *input, const double *offsets, const double *output,
                            const double *output_grad, double *offsets_grad);
/* src/utils/im2col.cpp:297-328 */
void so_col2im_3d_f32(const float *col, int channels, int height, int width, int patch_c, int patch_h, int patch_w,
                      int pad_c, int pad_h, int pad_w, int stride_c, int stride_h, int stride_w, float *im,
                      int round_down);
void so_col2im_3d_f64(const double *col, int channels, int height, int width, int patch_c, int patch_h, int patch_w,
                      int pad_c, int pad_h, int pad_w, int stride_c, int stride_h, int stride_w, double *im,
                      int round_down);
/* the backward combine functors one call at a time (similarity_utils.hpp:82-150, mex_utils.hpp:31-46);
 * mode as in so_ggemm_similarity, out2 = (d/dtemplate, d/dweight) */
void so_sim_backward_weights_fn_f32(int mode, float err, float x, float t, float w, float fudge, float *out2);
void so_sim_backward_weights_fn_f64(int mode, double err, double x, double t, double w, double fudge, double *out2);
float so_sim_backward_bottom_fn_f32(int mode, float t, float w, float err, float data);
double so_sim_backward_bottom_fn_f64(int mode, double t, double w, double err, double data);
float so_mex_backward_term_fn_f32(int finite, float offset, float top_data, float top_diff, float data, float ex,
                                  float ey);
double so_mex_backward_term_fn_f64(int finite, double offset, double top_data, double top_diff, double data,
                                   double ex, double ey);

#ifdef __cplusplus
}
#endif
#endif
