/*
 * simnets_hip.h - C ABI of the MI355X (gfx950) implementation of the SimNets forward operators.
 *
 * This is the boundary an operator layer binds instead of the kernels of HUJI-Deep/simnets-tf:
 * where that project's TensorFlow OpKernel::Compute methods call im2col_3d + ggemm, an op
 * layer calls simnets_hip_similarity_fwd / simnets_hip_mex_fwd with device pointers and the
 * operator attributes.  Citations below name the reference interface each entry point
 * replaces (paths relative to the reference checkout).
 *
 * Conventions
 *   - All tensors are dense, row-major, fp32, NCHW, resident in device memory; the caller
 *     owns every buffer.  The library never allocates, frees or keeps device memory: scratch
 *     comes from the caller's workspace (size from the *_workspace_bytes query).
 *   - Work is enqueued on the given stream (a hipStream_t passed as void*; NULL = the null
 *     stream) and the call returns without synchronising.  Calls are re-entrant.
 *   - Return value: SIMNETS_OK (0) or a negative simnets_status.  Attribute and shape
 *     validation happens on the host before anything is launched, so the error paths do not
 *     need a GPU.  simnets_hip_strerror() gives the message; where the reference raises
 *     InvalidArgument the message is the reference's own text.
 *   - There is no CPU fallback: on a machine without a usable HIP device the compute entry
 *     points return SIMNETS_ERR_HIP.
 */
#ifndef SIMNETS_HIP_H
#define SIMNETS_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SIMNETS_HIP_ABI_VERSION 1

typedef enum simnets_status {
    SIMNETS_OK = 0,
    SIMNETS_ERR_NULL_POINTER = -1,
    SIMNETS_ERR_PADDING_LENGTH = -2,        /* similarity_kernel_common.hpp:86 / mex ExpandDimSpec */
    SIMNETS_ERR_BLOCKS_LENGTH = -3,         /* similarity_kernel_common.hpp:89, mex_kernel_common.cpp:43 */
    SIMNETS_ERR_STRIDES_LENGTH = -4,        /* similarity_kernel_common.hpp:92, mex_kernel_common.cpp:39 */
    SIMNETS_ERR_SIMILARITY_FUNCTION = -5,   /* similarity_kernel_common.hpp:95-101 */
    SIMNETS_ERR_NORMALIZATION_NEEDS_L2 = -6,/* similarity_kernel_common.hpp:106 */
    SIMNETS_ERR_IGNORE_NAN_NEEDS_NORM = -7, /* similarity_kernel_common.hpp:108 */
    SIMNETS_ERR_TEMPLATE_CHANNELS = -8,     /* similarity_kernel_common.hpp:160 */
    SIMNETS_ERR_WEIGHTS_CHANNELS = -9,      /* similarity_kernel_common.hpp:162 */
    SIMNETS_ERR_STRIDE_NOT_POSITIVE = -10,  /* im2col.hpp:116-118 */
    SIMNETS_ERR_NUM_INSTANCES = -11,        /* mex_kernel_common.cpp:34 */
    SIMNETS_ERR_UNSHARED_REGION_LENGTH = -12, /* mex_kernel_common.cpp:54 */
    SIMNETS_ERR_SHARED_REGION_LENGTH = -13, /* mex_kernel_common.cpp:56 */
    SIMNETS_ERR_BLOCK_DEPTH = -14,          /* mex_kernel_common.cpp:169 */
    SIMNETS_ERR_SHAPE = -15,                /* a tensor shape disagrees with the attributes */
    SIMNETS_ERR_EMPTY_OUTPUT = -16,         /* an output dimension would be <= 0 */
    SIMNETS_ERR_WORKSPACE = -17,            /* workspace missing, too small or misaligned */
    SIMNETS_ERR_ALGO = -18,                 /* requested algorithm cannot serve these attributes */
    SIMNETS_ERR_TOO_LARGE = -19,            /* a dimension product exceeds 32-bit indexing */
    SIMNETS_ERR_HIP = -20,                  /* a HIP call or kernel launch failed */
    SIMNETS_ERR_STATIC_SCRATCH = -21        /* the call needs more scratch than SIMNETS_HIP_STATIC_SCRATCH_BYTES */
} simnets_status;

const char *simnets_hip_strerror(int status);
int simnets_hip_abi_version(void);

/* ------------------------------------------------------------------------------------------
 * Similarity:  REGISTER_OP("Similarity")  src/ops/similarity_op.cpp:61-75
 * ------------------------------------------------------------------------------------------ */
enum { SIMNETS_SIM_L1 = 0, SIMNETS_SIM_L2 = 1 };

/* How the weighted distance is evaluated.  All choices implement the same operator. */
enum {
    SIMNETS_ALGO_AUTO = 0,   /* SQRTW for plain L2 (no normalization term), DIRECT for every other mode */
    SIMNETS_ALGO_DIRECT = 1, /* d = t - x; acc += (-w*d)*d   (L1: acc += -w*|d|), NaN-capable, every mode */
    SIMNETS_ALGO_SQRTW = 2,  /* plain L2 only: d = sqrt(w)*t - sqrt(w)*x in one fma; acc += -d*d.  The rounding of d
                                could exceed 4e-6 relative only for outputs closer to zero than sum_k w t^2 / 1024.
                                The terms all have one sign, so a wave (64 pixel groups x 8 templates) whose partial
                                sums after the first channel chunk all lie beyond that bound is safe; a wave with one
                                that does not (or with a template of negative or NaN weight) stops there and a second
                                pass of its workgroup recomputes all its outputs with DIRECT's arithmetic,
                                bit-identical to SIMNETS_ALGO_DIRECT */
    SIMNETS_ALGO_MFMA = 3    /* plain L2 only, inputs free of NaN/Inf: sum w x^2 - 2 sum (w t) x + sum w t^2
                                as dense fp32 matrix-core contractions */
};

typedef struct simnets_similarity_attrs {
    int similarity_function;         /* attr similarity_function: {'L1','L2'} = 'L2'          */
    int n_blocks;  int blocks[2];    /* attr blocks  = [3,3]   (README calls it ksize)        */
    int n_strides; int strides[2];   /* attr strides = [2,2]                                  */
    int n_padding; int padding[2];   /* attr padding = [0,0]                                  */
    int normalization_term;          /* attr normalization_term = false                      */
    float normalization_term_fudge;  /* attr normalization_term_fudge = 0.001                */
    int ignore_nan_input;            /* attr ignore_nan_input = false                        */
    float out_of_bounds_value;       /* attr out_of_bounds_value = 0.0 (may be NaN)          */
    /* -- extensions; zero keeps the documented operator semantics -- */
    int algo;                        /* SIMNETS_ALGO_*                                       */
    /* Non-zero reproduces SimilarityKernelCPU::Compute literally for
     * L2 + normalization_term + !ignore_nan_input: the constant -0.5*K*log(2 pi) is added to the
     * whole output once per batch iteration (similarity_kernel_cpu.cpp:69,118-120), so image n
     * carries it (B - n) times.  Zero adds it once per output, which is what SimilarityRef
     * (similarity_ref_kernel_cpu.cpp:89-93) and the op documentation define. */
    int norm_const_every_iteration;
} simnets_similarity_attrs;

/* Fills in the REGISTER_OP defaults (src/ops/similarity_op.cpp:67-74). */
void simnets_similarity_attrs_default(simnets_similarity_attrs *attrs);

/* Shape function: SimilarityShape (src/ops/similarity_op.cpp:8-53) and
 * SimilarityKernelCommon::CalculateDimensions (include/kernels/similarity_kernel_common.hpp:113-164).
 * input_shape = [B,C,H,W], templates_shape = weights_shape = [O,C,bh,bw]; output_shape <- [B,O,oh,ow].
 * Performs every attribute / shape check of the operator. */
int simnets_similarity_out_shape(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                 const int templates_shape[4], const int weights_shape[4], int output_shape[4]);

/* Scratch the forward call needs (packed parameters), in bytes. */
int simnets_hip_similarity_workspace_bytes(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                           const int templates_shape[4], size_t *bytes);

/* Forward: replaces SimilarityKernelGPU<float>::Compute (src/kernels/similarity_kernel_gpu.cu:24-133),
 * i.e. interlace_gpu + per-image im2col_3d_gpu + ggemm_gpu + the normalization constant.
 * weights must be non-negative (the reference's Keras layer applies abs, python/simnets/keras.py:65). */
int simnets_hip_similarity_fwd(const simnets_similarity_attrs *attrs, const int input_shape[4],
                               const int templates_shape[4], const int weights_shape[4], const float *input,
                               const float *templates, const float *weights, float *output, void *workspace,
                               size_t workspace_bytes, void *stream);

/* The same forward with the parameter-only work taken out of the steady-state call, for callers whose templates and
 * weights stay fixed across calls (inference): where SimilarityKernelGPU::Compute interlaces the parameters on
 * every call (src/kernels/similarity_kernel_gpu.cu:70), simnets_hip_similarity_prepare does the packing once
 * (packed parameters, tables, and for the sqrt-weight form the second packed copy and the thresholds) into a
 * caller-owned buffer of simnets_hip_similarity_workspace_bytes bytes (256-byte aligned), and
 * simnets_hip_similarity_fwd_prepared runs only the forward kernels on it.  attrs, input_shape (batch size
 * included: the tiling depends on it) and templates_shape must be the ones the buffer was prepared with; results
 * are those of simnets_hip_similarity_fwd bit for bit.  The buffer may also hold a few bytes of per-call scratch (the
 * workgroup flags of the sqrt-weight form on small maps), so calls that share one prepared buffer must not overlap. */
int simnets_hip_similarity_prepare(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                   const int templates_shape[4], const int weights_shape[4], const float *templates,
                                   const float *weights, void *prepared, size_t prepared_bytes, void *stream);
int simnets_hip_similarity_fwd_prepared(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                        const int templates_shape[4], const float *input, void *prepared,
                                        size_t prepared_bytes, float *output, void *stream);

/* simnets_hip_similarity_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc) and so have no workspace to pass.  It has no counterpart in the
 * reference.  Same arguments minus the workspace, same kernels, same results bit for bit; the scratch is a fixed
 * device array of SIMNETS_HIP_STATIC_SCRATCH_BYTES inside the library (one copy per GPU, held until the process
 * ends) and the call allocates nothing.  Calls whose simnets_hip_similarity_workspace_bytes exceeds that size
 * return SIMNETS_ERR_STATIC_SCRATCH before anything is launched.  All calls on one GPU share that GPU's array:
 * calls that may overlap on one GPU (different streams, different threads) race; order them on one stream.  The
 * first call on a device looks up the array's address (hipGetSymbolAddress): make it outside graph capture. */
#define SIMNETS_HIP_STATIC_SCRATCH_BYTES (4u << 20)
int simnets_hip_similarity_fwd_static(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                      const int templates_shape[4], const int weights_shape[4], const float *input,
                                      const float *templates, const float *weights, float *output, void *stream);

/* Backward.  Scratch sizes of the two gradient calls (either pointer may be NULL). */
int simnets_hip_similarity_grad_workspace_bytes(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                                const int templates_shape[4], size_t *input_grad_bytes,
                                                size_t *params_grad_bytes);

/* REGISTER_OP("SimilarityInputGrad") (src/ops/similarity_op.cpp:141-156): replaces
 * SimilarityInputGradKernelGPU<float>::Compute (src/kernels/similarity_grad_kernel_gpu.cu), i.e. per image
 * im2col_3d_gpu + ggemm_readc_gpu<TRANSPOSE_A> with sim_*_backward_bottom + col2im_3d_gpu.
 * output_grad has the forward output's shape, input_grad the input's.  attrs->algo: SIMNETS_ALGO_DIRECT sums
 * the reference's terms one by one in every case; otherwise the L2 modes with 24 channels or more (strides no
 * larger than the window, padding smaller than the window) evaluate A - (x - c) B with A = sum g s w (t - c),
 * B = sum g s w on the fp32 matrix cores (same sum, other rounding; c = the channel's mean template value).
 * Small grids split that sum over workgroups and add the parts in a fixed order: results do not vary from
 * run to run. */
int simnets_hip_similarity_input_grad(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                      const int templates_shape[4], const int weights_shape[4], const float *input,
                                      const float *templates, const float *weights, const float *output_grad,
                                      float *input_grad, void *workspace, size_t workspace_bytes, void *stream);

/* REGISTER_OP("SimilarityParametersGrad") (src/ops/similarity_op.cpp:158-174): replaces
 * SimilarityParametersGradKernelGPU<float>::Compute, i.e. per image im2col_3d_gpu + ggemm_readc_gpu with
 * sim_*_backward_weights accumulated over the batch + deinterlace.  templates_grad and weights_grad have
 * the templates' shape.  The sums over pixels are formed in a fixed order: results are reproducible.
 * attrs->algo: SIMNETS_ALGO_DIRECT sums the reference's terms one by one; otherwise the L2 modes accumulate the
 * moments sum g (x - c), sum g (x - c)^2, sum g about a centre c near the templates on the fp32 matrix cores and
 * combine them in double precision, and L1 takes sign and magnitude from 2^64 (x - t) (bit-identical to the
 * term-by-term sums unless 0 < |x - t| < 2^-64). */
int simnets_hip_similarity_params_grad(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                       const int templates_shape[4], const int weights_shape[4], const float *input,
                                       const float *templates, const float *weights, const float *output_grad,
                                       float *templates_grad, float *weights_grad, void *workspace,
                                       size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------------------------------
 * MEX:  REGISTER_OP("Mex")  src/ops/mex_op.cpp:58-74
 * ------------------------------------------------------------------------------------------ */
typedef struct simnets_mex_attrs {
    int num_instances;                   /* attr num_instances (required)                     */
    int softmax_mode;                    /* attr softmax_mode = false                         */
    int n_padding; int padding[3];       /* attr padding = [0,0,0]; 2 entries get -1 prepended; -1 -> image dim */
    int n_strides; int strides[3];       /* attr strides = [1,1,1]; -1 -> image dim           */
    int n_blocks;  int blocks[3];        /* attr blocks  = [1,1,1]                            */
    float epsilon;                       /* attr epsilon = 1.0, may be +-inf                  */
    float blocks_out_of_bounds_value;    /* attr blocks_out_of_bounds_value = 0.0             */
    int blocks_round_down;               /* attr blocks_round_down = true                     */
    int use_unshared_regions;            /* attr use_unshared_regions = true                  */
    int n_shared;   int shared_offset_region[3];    /* attr shared_offset_region = [-1]   (1 or 3) */
    int n_unshared; int unshared_offset_region[3];  /* attr unshared_offset_region = [-1] (1 or 3) */
    /* -- extension -- */
    /* Non-zero: offsets[r,m,:] -= logsumexp(offsets[r,m,:]) before use, what the reference's Keras
     * layer does in Python for normalize_offsets=True (python/simnets/keras.py:155-160). */
    int normalize_offsets;
} simnets_mex_attrs;

/* Fills in the REGISTER_OP defaults (src/ops/mex_op.cpp:62-73); num_instances is set to 1. */
void simnets_mex_attrs_default(simnets_mex_attrs *attrs);

/* Everything MexDimensionsData::CalculateDimensions derives (src/kernels/mex_kernel_common.cpp:63-158). */
typedef struct simnets_mex_dims {
    int pad_c, pad_h, pad_w, stride_c, stride_h, stride_w, block_c, block_h, block_w;
    int channels_out, height_out, width_out, channels_out_total;
    int shared_region_c, shared_region_h, shared_region_w;
    int offsets_c, offsets_h, offsets_w;
    int num_regions, region_size;
    int M, K, N;
    int is_1x1;
} simnets_mex_dims;

/* MexDimensionsData::CalculateDimensions + the checks of MEXKernelCommon's constructor
 * (src/kernels/mex_kernel_common.cpp:29-58, :63-158, :169).  image_chw = [C,H,W]. */
int simnets_mex_calc_dims(const simnets_mex_attrs *attrs, const int image_chw[3], simnets_mex_dims *dims);

/* Shape function: MexShape (src/ops/mex_op.cpp:8-55).  input_shape = [B,C,H,W];
 * output_shape <- [B, channels_out*num_instances, oh, ow]; offsets_shape <- [R,M,bc,bh,bw]
 * (either output may be NULL). */
int simnets_mex_out_shape(const simnets_mex_attrs *attrs, const int input_shape[4], int output_shape[4],
                          int offsets_shape[5]);

/* Binary-compatible twin of the reference's only C-ABI symbol (src/kernels/mex_dims_helper.cpp:8-44),
 * so python/simnets/ops/mex.py:17-38 can bind this library unchanged.  Returns num_regions, or -1
 * when n_blocks != 3. */
int get_mex_offsets_nregions(int n_input_dim, const int *input_dim, int n_padding, const int *padding,
                             int n_strides, const int *strides, int num_instances, int blocks_round_down,
                             int use_unshared_regions, int n_blocks, const int *blocks,
                             int n_shared_offset_region, const int *shared_offset_region,
                             int n_unshared_offset_region, const int *unshared_offset_region);

int simnets_hip_mex_workspace_bytes(const simnets_mex_attrs *attrs, const int input_shape[4], size_t *bytes);

/* Forward: replaces MEXKernelGPU<float>::Compute (src/kernels/mex_kernel_gpu.cu:60-159), i.e. the
 * offsets copy + per-image im2col_3d_gpu + split_patches_gpu + ggemm_gpu (max pass) +
 * ggemm_readc_gpu (exp/sum/log pass) + reverse split_patches_gpu.
 * offsets_count = number of floats behind `offsets`; must be >= num_regions*num_instances*K.
 * `input` may have any float alignment; on layers with 2x2 unshared offsets over whole-channel patches a 16-byte
 * aligned input takes a faster kernel, whose results differ from the general kernel's in the last bits. */
int simnets_hip_mex_fwd(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                        const float *offsets, size_t offsets_count, float *output, void *workspace,
                        size_t workspace_bytes, void *stream);

/* The same forward with the offsets-only work taken out of the steady-state call (fixed offsets, inference): where
 * MEXKernelGPU::Compute copies the offsets on every call (src/kernels/mex_kernel_gpu.cu:98-112),
 * simnets_hip_mex_prepare packs them once (normalised if attrs say so, scaled, k-major per instance group, with their
 * exponentials, row maxima and ranges, and the patch element table) into a caller-owned buffer of
 * simnets_hip_mex_workspace_bytes bytes (256-byte aligned) and simnets_hip_mex_fwd_prepared runs only the forward
 * kernel on it.  attrs and input_shape (batch size included) must be the ones the buffer was prepared with; results
 * are those of simnets_hip_mex_fwd (on an input of the same alignment) bit for bit. */
int simnets_hip_mex_prepare(const simnets_mex_attrs *attrs, const int input_shape[4], const float *offsets,
                            size_t offsets_count, void *prepared, size_t prepared_bytes, void *stream);
int simnets_hip_mex_fwd_prepared(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                 void *prepared, size_t prepared_bytes, float *output, void *stream);

/* Backward.  Scratch sizes of the two gradient calls (either pointer may be NULL). */
int simnets_hip_mex_grad_workspace_bytes(const simnets_mex_attrs *attrs, const int input_shape[4],
                                         size_t *input_grad_bytes, size_t *offsets_grad_bytes);

/* REGISTER_OP("MexInputGrad") (src/ops/mex_op.cpp:134-151): replaces MEXGradInputKernelGPU<float>::Compute
 * (src/kernels/mex_grad_kernel_gpu.cu), i.e. per image im2col_3d_gpu + split_patches + ggemm_readc_gpu with
 * mex_backward_bottom_finite/_infinite + reverse split_patches + col2im_3d_gpu.
 * output = the forward result for the same input/offsets/attrs, output_grad has its shape, input_grad the
 * input's.  When blocks overlap (block > stride) the patches' contributions to an element are added in
 * ascending (c, h, w) order of the patches, like col2im_3d does: results are reproducible. */
int simnets_hip_mex_input_grad(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                               const float *offsets, size_t offsets_count, const float *output,
                               const float *output_grad, float *input_grad, void *workspace, size_t workspace_bytes,
                               void *stream);

/* REGISTER_OP("MexOffsetsGrad") (src/ops/mex_op.cpp:153-170): replaces MEXGradOffsetsKernelGPU<float>::Compute.
 * offsets_grad has the offsets' shape [R,M,bc,bh,bw]; sums run in a fixed order (reproducible).
 * With attrs->normalize_offsets the forward op saw o - logsumexp(o); the gradient returned is the one
 * w.r.t. the raw offsets o (the chain rule through python/simnets/keras.py:155-160 is applied). */
int simnets_hip_mex_offsets_grad(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                 const float *offsets, size_t offsets_count, const float *output,
                                 const float *output_grad, float *offsets_grad, void *workspace,
                                 size_t workspace_bytes, void *stream);

/* Both gradients of one MEX layer in one call, as the gradient registered for the Mex op needs them
 * (python/simnets/ops/mex.py:47-81 calls MexInputGrad and MexOffsetsGrad on the same tensors): the results are those
 * of simnets_hip_mex_input_grad and simnets_hip_mex_offsets_grad, bit for bit; the offsets as the forward op used
 * them, their packed form and the per-pixel factors are prepared once for both. */
int simnets_hip_mex_grads_workspace_bytes(const simnets_mex_attrs *attrs, const int input_shape[4], size_t *bytes);
int simnets_hip_mex_grads(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                          const float *offsets, size_t offsets_count, const float *output, const float *output_grad,
                          float *input_grad, float *offsets_grad, void *workspace, size_t workspace_bytes,
                          void *stream);

/* ------------------------------------------------------------------------------------------
 * Glue of the missing-data network between MEX layers: non-overlapping sum pooling, which the
 * reference example builds from AveragePooling2D * pool area (README.md:108-111,
 * examples/mnist_ght_model_missing_data.py:60-66).  input [B,C,H,W] -> output [B,C,H/ph,W/pw]
 * ('valid': a trailing partial window is dropped).
 * ------------------------------------------------------------------------------------------ */
int simnets_hip_sum_pool_fwd(const int input_shape[4], int pool_h, int pool_w, const float *input, float *output,
                             void *stream);

/* Its gradient (what the framework's AveragePooling2D gradient times the pool area gives in the reference example,
 * examples/mnist_ght_model_missing_data.py:60-66): input_grad [B,C,H,W] <- output_grad [B,C,H/ph,W/pw] of the
 * element's window; elements of a dropped trailing row or column get 0. */
int simnets_hip_sum_pool_input_grad(const int input_shape[4], int pool_h, int pool_w, const float *output_grad,
                                    float *input_grad, void *stream);

/* MEX followed by that sum pooling, as one call: output [B, M*channels_out, height_out/pool_h, width_out/pool_w]
 * = simnets_hip_sum_pool_fwd(simnets_hip_mex_fwd(...)).  The pair the reference's networks run back to back
 * (README.md:108-129: MEX with unshared_offset_region = the pooling window, then pooling).  When the offsets are
 * unshared with regions [1, pool_h, pool_w] (a pooling window is then one pixel of every region), epsilon is finite
 * and the window has 2 or 4 pixels, one kernel computes the MEX values of a window in one lane, adds them in the
 * window's row-major order and writes only the pooled tensor; any other geometry runs the two kernels through
 * scratch memory.  No gradient entry point takes the pooled tensor alone: training uses the _both form below. */
int simnets_hip_mex_sum_pool_workspace_bytes(const simnets_mex_attrs *attrs, const int input_shape[4], int pool_h,
                                             int pool_w, size_t *bytes);
int simnets_hip_mex_sum_pool_fwd(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                 const float *offsets, size_t offsets_count, int pool_h, int pool_w, float *output,
                                 void *workspace, size_t workspace_bytes, void *stream);

/* The same call for training: it also stores the MEX output before pooling (mex_output, the shape
 * simnets_mex_out_shape gives), which MexInputGrad / MexOffsetsGrad take as their `output` argument
 * (src/ops/mex_op.cpp:134-170), so that a training step keeps the fused kernel and runs no pooling launch.  Both
 * tensors hold the values of the two separate calls. */
int simnets_hip_mex_sum_pool_fwd_both(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                      const float *offsets, size_t offsets_count, int pool_h, int pool_w,
                                      float *mex_output, float *output, void *workspace, size_t workspace_bytes,
                                      void *stream);

/* The gradients of that pair in one call: MexInputGrad and MexOffsetsGrad (src/ops/mex_op.cpp:134-170) applied to the
 * gradient of the pooling (the reference's AveragePooling2D x area, README.md:108-111), from the gradient of the POOLED
 * output `pooled_output_grad` [B, M*C_out, H_out/pool_h, W_out/pool_w] and the unpooled MEX output `mex_output`
 * (what simnets_hip_mex_sum_pool_fwd_both stores).  With 2 x 2 windows over an output of even height and width and one
 * output channel per instance (every output pixel then has a window: the layers of the reference's networks) the
 * gradient kernels read the window gradients themselves; elsewhere the pooling gradient is expanded into the
 * workspace first.  Either gradient pointer may be NULL.  The values are those of simnets_hip_sum_pool_input_grad followed by simnets_hip_mex_grads, bit for bit. */
int simnets_hip_mex_sum_pool_grads_workspace_bytes(const simnets_mex_attrs *attrs, const int input_shape[4], int pool_h,
                                                   int pool_w, size_t *bytes);
int simnets_hip_mex_sum_pool_grads(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                   const float *offsets, size_t offsets_count, int pool_h, int pool_w,
                                   const float *mex_output, const float *pooled_output_grad, float *input_grad,
                                   float *offsets_grad, void *workspace, size_t workspace_bytes, void *stream);

/* A training step runs the forward op and then its gradients on the same offsets (python/simnets/ops/mex.py:47-81:
 * the registered gradient receives the forward op's inputs and output).  Both sides re-order the offsets first
 * (scaled, row maxima and ranges, exponentials, the normalised copy of normalize_offsets), in different group sizes.
 * The *_saving forward calls leave the gradient kernels' form in `saved` (simnets_hip_mex_saved_bytes; 256-byte
 * aligned; 0 bytes = this layer's gradient kernels read the offsets as they are, `saved` may then be NULL; layers of few
 * instances over long patches keep the normalised copy alone) from the
 * launch that packs the forward's own, and the *_saved gradient calls read it instead of packing again.  Outputs
 * and gradients are those of the plain calls, bit for bit.  `saved` is valid for the attributes, input shape and
 * offsets VALUES of the forward call that wrote it; a gradient call given saved == NULL packs for itself. */
int simnets_hip_mex_saved_bytes(const simnets_mex_attrs *attrs, const int input_shape[4], size_t *bytes);
int simnets_hip_mex_fwd_saving(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                               const float *offsets, size_t offsets_count, float *output, void *saved,
                               size_t saved_bytes, void *workspace, size_t workspace_bytes, void *stream);
int simnets_hip_mex_sum_pool_fwd_saving(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                        const float *offsets, size_t offsets_count, int pool_h, int pool_w,
                                        float *mex_output, float *output, void *saved, size_t saved_bytes,
                                        void *workspace, size_t workspace_bytes, void *stream);
int simnets_hip_mex_grads_saved(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                const float *offsets, size_t offsets_count, const float *output,
                                const float *output_grad, const void *saved, size_t saved_bytes, float *input_grad,
                                float *offsets_grad, void *workspace, size_t workspace_bytes, void *stream);
int simnets_hip_mex_sum_pool_grads_saved(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                         const float *offsets, size_t offsets_count, int pool_h, int pool_w,
                                         const float *mex_output, const float *pooled_output_grad, const void *saved,
                                         size_t saved_bytes, float *input_grad, float *offsets_grad, void *workspace,
                                         size_t workspace_bytes, void *stream);

/* ... simnets_hip_mex_sum_pool_fwd in two halves, like simnets_hip_mex_prepare / simnets_hip_mex_fwd_prepared: the
 * buffer has simnets_hip_mex_sum_pool_workspace_bytes bytes; when the geometry runs the two kernels through scratch memory the
 * buffer holds that scratch as well, so calls that share one prepared buffer must not overlap. */
int simnets_hip_mex_sum_pool_prepare(const simnets_mex_attrs *attrs, const int input_shape[4], const float *offsets,
                                     size_t offsets_count, int pool_h, int pool_w, void *prepared,
                                     size_t prepared_bytes, void *stream);
int simnets_hip_mex_sum_pool_fwd_prepared(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                          int pool_h, int pool_w, void *prepared, size_t prepared_bytes, float *output,
                                          void *stream);

/* Similarity, MEX over its output, sum pooling, as one call: the first layers of the reference's networks
 * (README.md:108-129: Similarity on the image, MEX over all of its channels per pixel, pooling).  output =
 * simnets_hip_sum_pool_fwd(simnets_hip_mex_fwd(simnets_hip_similarity_fwd(...))); mex_attrs describe the MEX layer
 * over the Similarity output [B, O, oh, ow]; weights have the templates' shape.  When the MEX + pooling pair is
 * fusable (above), the MEX blocks are [O, 1, 1] without padding and a Similarity patch has at most 16 elements, one
 * kernel evaluates the Similarity channels inside its staging (same arithmetic and order as the Similarity kernel,
 * term by term as SIMNETS_ALGO_DIRECT) and neither intermediate tensor exists; any other combination runs the
 * separate kernels through scratch memory.  Forward only. */
int simnets_hip_similarity_mex_sum_pool_workspace_bytes(const simnets_similarity_attrs *sim_attrs,
                                                        const int input_shape[4], const int templates_shape[4],
                                                        const simnets_mex_attrs *mex_attrs, int pool_h, int pool_w,
                                                        size_t *bytes);
int simnets_hip_similarity_mex_sum_pool_fwd(const simnets_similarity_attrs *sim_attrs, const int input_shape[4],
                                            const int templates_shape[4], const float *input, const float *templates,
                                            const float *weights, const simnets_mex_attrs *mex_attrs,
                                            const float *offsets, size_t offsets_count, int pool_h, int pool_w,
                                            float *output, void *workspace, size_t workspace_bytes, void *stream);

/* ... in two halves: templates, weights and offsets are packed once into a buffer of
 * simnets_hip_similarity_mex_sum_pool_workspace_bytes bytes; the steady-state call takes the input only.  Same
 * conditions as the other prepared calls (same attrs and shapes; no overlapping calls on one buffer). */
int simnets_hip_similarity_mex_sum_pool_prepare(const simnets_similarity_attrs *sim_attrs, const int input_shape[4],
                                                const int templates_shape[4], const float *templates,
                                                const float *weights, const simnets_mex_attrs *mex_attrs,
                                                const float *offsets, size_t offsets_count, int pool_h, int pool_w,
                                                void *prepared, size_t prepared_bytes, void *stream);
int simnets_hip_similarity_mex_sum_pool_fwd_prepared(const simnets_similarity_attrs *sim_attrs,
                                                     const int input_shape[4], const int templates_shape[4],
                                                     const float *input, const simnets_mex_attrs *mex_attrs, int pool_h,
                                                     int pool_w, void *prepared, size_t prepared_bytes, float *output,
                                                     void *stream);

#ifdef __cplusplus
}
#endif
#endif /* SIMNETS_HIP_H */
