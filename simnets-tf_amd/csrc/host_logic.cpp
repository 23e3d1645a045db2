// Host-side half of libsimnets_hip: attribute defaults, validation, dimension arithmetic and the
// C-ABI entry points that never touch the device.  Mirrors, check for check, what the reference's
// operator layer does before it launches anything:
//   Similarity  include/kernels/similarity_kernel_common.hpp:82-111 (attrs), :113-164 (dims),
//               src/ops/similarity_op.cpp:8-53 (shape function)
//   MEX         src/kernels/mex_kernel_common.cpp:8-27 (ExpandDimSpec), :29-58 (attrs),
//               :63-158 (CalculateDimensions), :169; src/ops/mex_op.cpp:8-55 (shape function)
//   dims helper src/kernels/mex_dims_helper.cpp:8-44
#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>

#include "internal.h"

namespace simnets {

// include/utils/im2col.hpp:101-108
static int dimension_out_size(int image_size, int pad_size, int patch_size, int stride, bool round_down)
{
    if (round_down)
        return (image_size + 2 * pad_size - patch_size) / stride + 1;
    return static_cast<int>(std::ceil(static_cast<float>(image_size + 2 * pad_size - patch_size) / stride)) + 1;
}

// include/utils/ggemm_cpu.hpp:451-454
static int ceiled_div(int a, int b) { return (a / b) + ((a % b) > 0); }

static bool fits_int32(long long v) { return v >= 0 && v <= std::numeric_limits<int>::max(); }

int sim_make_plan(const simnets_similarity_attrs *a, const int in[4], const int tp[4], const int wt[4], SimPlan *p)
{
    if (!a || !in || !tp || !wt || !p)
        return SIMNETS_ERR_NULL_POINTER;
    if (a->n_padding != 2)
        return SIMNETS_ERR_PADDING_LENGTH;
    if (a->n_blocks != 2)
        return SIMNETS_ERR_BLOCKS_LENGTH;
    if (a->n_strides != 2)
        return SIMNETS_ERR_STRIDES_LENGTH;
    if (a->similarity_function != SIMNETS_SIM_L1 && a->similarity_function != SIMNETS_SIM_L2)
        return SIMNETS_ERR_SIMILARITY_FUNCTION;
    if (a->normalization_term && a->similarity_function != SIMNETS_SIM_L2)
        return SIMNETS_ERR_NORMALIZATION_NEEDS_L2;
    if (a->ignore_nan_input && !a->normalization_term)
        return SIMNETS_ERR_IGNORE_NAN_NEEDS_NORM;
    for (int i = 0; i < 4; ++i)
        if (in[i] < 0 || tp[i] < 0 || wt[i] < 0)
            return SIMNETS_ERR_SHAPE;
    if (in[1] != tp[1])
        return SIMNETS_ERR_TEMPLATE_CHANNELS;
    if (in[1] != wt[1])
        return SIMNETS_ERR_WEIGHTS_CHANNELS;
    if (a->strides[0] <= 0 || a->strides[1] <= 0)
        return SIMNETS_ERR_STRIDE_NOT_POSITIVE;
    // The reference sizes the output from the template tensor in its shape function and from the
    // blocks attribute in its kernel; the two must agree for the op to be well defined.
    if (tp[2] != a->blocks[0] || tp[3] != a->blocks[1] || a->blocks[0] <= 0 || a->blocks[1] <= 0)
        return SIMNETS_ERR_SHAPE;
    if (wt[0] != tp[0] || wt[2] != tp[2] || wt[3] != tp[3])
        return SIMNETS_ERR_SHAPE;
    if (a->padding[0] < 0 || a->padding[1] < 0)
        return SIMNETS_ERR_SHAPE;

    p->B = in[0]; p->C = in[1]; p->H = in[2]; p->W = in[3];
    p->O = tp[0];
    p->bh = a->blocks[0]; p->bw = a->blocks[1];
    p->sh = a->strides[0]; p->sw = a->strides[1];
    p->ph = a->padding[0]; p->pw = a->padding[1];
    p->oh = dimension_out_size(p->H, p->ph, p->bh, p->sh, true);
    p->ow = dimension_out_size(p->W, p->pw, p->bw, p->sw, true);
    if (p->oh <= 0 || p->ow <= 0 || p->O <= 0 || p->C <= 0 || p->H <= 0 || p->W <= 0)
        return SIMNETS_ERR_EMPTY_OUTPUT;
    const long long K = 1LL * p->C * p->bh * p->bw;
    if (!fits_int32(K) || !fits_int32(1LL * p->C * p->H * p->W) || !fits_int32(1LL * p->O * p->oh * p->ow) ||
        !fits_int32(1LL * p->O * K * 4) || !fits_int32(1LL * p->B * p->oh * p->ow))
        return SIMNETS_ERR_TOO_LARGE;
    p->K = static_cast<int>(K);
    if (a->similarity_function == SIMNETS_SIM_L1)
        p->mode = SIM_MODE_L1;
    else if (!a->normalization_term)
        p->mode = SIM_MODE_L2;
    else
        p->mode = a->ignore_nan_input ? SIM_MODE_L2_NORM_IGNORE_NAN : SIM_MODE_L2_NORM;
    p->fudge = a->normalization_term_fudge;
    p->oob = a->out_of_bounds_value;
    p->norm_const_every_iteration = a->norm_const_every_iteration != 0;
    p->exact_terms = a->algo == SIMNETS_ALGO_DIRECT;
    switch (a->algo) {
    case SIMNETS_ALGO_AUTO:
        // plain L2: the two-instruction sqrt-weight form, with its small outputs recomputed exactly
        p->algo = p->mode == SIM_MODE_L2 ? SIMNETS_ALGO_SQRTW : SIMNETS_ALGO_DIRECT;
        break;
    case SIMNETS_ALGO_DIRECT:
        p->algo = SIMNETS_ALGO_DIRECT;
        break;
    case SIMNETS_ALGO_SQRTW:
    case SIMNETS_ALGO_MFMA:
        if (p->mode != SIM_MODE_L2)
            return SIMNETS_ERR_ALGO;
        p->algo = a->algo;
        break;
    default:
        return SIMNETS_ERR_ALGO;
    }
    return SIMNETS_OK;
}

// src/kernels/mex_kernel_common.cpp:8-27
static void expand_dim_spec(const int image_chw[3], int n, const int *spec, int out[3])
{
    int i0 = 0;
    if (n == 2) {
        out[0] = -1;
        i0 = 1;
    }
    for (int i = 0; i + i0 < 3 && i < n; ++i)
        out[i + i0] = spec[i];
    for (int i = 0; i < 3; ++i)
        if (out[i] == -1)
            out[i] = image_chw[i];
}

static int mex_calc_dims_impl(const simnets_mex_attrs *a, const int image[3], simnets_mex_dims *d, bool check_depth)
{
    if (!a || !image || !d)
        return SIMNETS_ERR_NULL_POINTER;
    if (a->num_instances <= 0)
        return SIMNETS_ERR_NUM_INSTANCES;
    if (a->n_padding != 3 && a->n_padding != 2)
        return SIMNETS_ERR_PADDING_LENGTH;
    if (a->n_strides != 3)
        return SIMNETS_ERR_STRIDES_LENGTH;
    if (a->n_blocks != 3)
        return SIMNETS_ERR_BLOCKS_LENGTH;
    if (a->n_unshared != 3 && a->n_unshared != 1)
        return SIMNETS_ERR_UNSHARED_REGION_LENGTH;
    if (a->n_shared != 3 && a->n_shared != 1)
        return SIMNETS_ERR_SHARED_REGION_LENGTH;
    if (image[0] <= 0 || image[1] <= 0 || image[2] <= 0)
        return SIMNETS_ERR_EMPTY_OUTPUT;
    int pad[3], str[3];
    expand_dim_spec(image, a->n_padding, a->padding, pad);
    expand_dim_spec(image, a->n_strides, a->strides, str);
    if (str[0] <= 0 || str[1] <= 0 || str[2] <= 0)
        return SIMNETS_ERR_STRIDE_NOT_POSITIVE;
    if (a->blocks[0] <= 0 || a->blocks[1] <= 0 || a->blocks[2] <= 0 || pad[0] < 0 || pad[1] < 0 || pad[2] < 0)
        return SIMNETS_ERR_SHAPE;
    std::memset(d, 0, sizeof(*d));
    d->pad_c = pad[0]; d->pad_h = pad[1]; d->pad_w = pad[2];
    d->stride_c = str[0]; d->stride_h = str[1]; d->stride_w = str[2];
    d->block_c = a->blocks[0]; d->block_h = a->blocks[1]; d->block_w = a->blocks[2];
    if (check_depth && d->block_c > image[0])
        return SIMNETS_ERR_BLOCK_DEPTH;
    const bool rd = a->blocks_round_down != 0;
    d->height_out = dimension_out_size(image[1], d->pad_h, d->block_h, d->stride_h, rd);
    d->width_out = dimension_out_size(image[2], d->pad_w, d->block_w, d->stride_w, rd);
    d->channels_out = dimension_out_size(image[0], d->pad_c, d->block_c, d->stride_c, rd);
    if (d->height_out <= 0 || d->width_out <= 0 || d->channels_out <= 0)
        return SIMNETS_ERR_EMPTY_OUTPUT;

    auto resolve = [](int spec, int full) {
        if (spec < 0)
            spec = full;
        return std::min(spec, full);
    };
    if (!a->use_unshared_regions) {
        int sc, sh, sw;
        if (a->n_shared == 3) {
            sc = a->shared_offset_region[0]; sh = a->shared_offset_region[1]; sw = a->shared_offset_region[2];
        } else {
            sw = sh = a->shared_offset_region[0];
            sc = -1;
        }
        sh = resolve(sh, d->height_out); sw = resolve(sw, d->width_out); sc = resolve(sc, d->channels_out);
        if (sh == 0 || sw == 0 || sc == 0)
            return SIMNETS_ERR_SHAPE;
        d->shared_region_c = sc; d->shared_region_h = sh; d->shared_region_w = sw;
        d->offsets_h = ceiled_div(d->height_out, sh);
        d->offsets_w = ceiled_div(d->width_out, sw);
        d->offsets_c = ceiled_div(d->channels_out, sc);
    } else {
        int uc, uh, uw;
        if (a->n_unshared == 3) {
            uc = a->unshared_offset_region[0]; uh = a->unshared_offset_region[1]; uw = a->unshared_offset_region[2];
        } else {
            uw = uh = a->unshared_offset_region[0];
            uc = -1;
        }
        uh = resolve(uh, d->height_out); uw = resolve(uw, d->width_out); uc = resolve(uc, d->channels_out);
        if (uh == 0 || uw == 0 || uc == 0)
            return SIMNETS_ERR_SHAPE;
        d->offsets_h = uh; d->offsets_w = uw; d->offsets_c = uc;
        d->shared_region_h = ceiled_div(d->height_out, uh);
        d->shared_region_w = ceiled_div(d->width_out, uw);
        d->shared_region_c = ceiled_div(d->channels_out, uc);
    }
    const long long R = 1LL * d->offsets_h * d->offsets_w * d->offsets_c;
    const long long K = 1LL * d->block_c * d->block_h * d->block_w;
    const long long N = 1LL * d->height_out * d->width_out * d->channels_out;
    if (!fits_int32(R) || !fits_int32(K) || !fits_int32(N) || !fits_int32(N * a->num_instances) ||
        !fits_int32(R * a->num_instances) || !fits_int32(1LL * image[0] * image[1] * image[2]))
        return SIMNETS_ERR_TOO_LARGE;
    d->num_regions = static_cast<int>(R);
    d->region_size = d->shared_region_w * d->shared_region_h * d->shared_region_c;
    d->channels_out_total = d->channels_out * a->num_instances;
    d->M = a->num_instances;
    d->K = static_cast<int>(K);
    d->N = static_cast<int>(N);
    d->is_1x1 = (d->block_c == image[0] || (d->block_c == 1 && d->stride_c == 1)) && d->block_w == 1 &&
                d->block_h == 1 && d->stride_h == 1 && d->stride_w == 1 && d->pad_c == 0 && d->pad_h == 0 &&
                d->pad_w == 0;
    return SIMNETS_OK;
}

int mex_make_plan(const simnets_mex_attrs *a, const int in[4], MexPlan *p)
{
    if (!a || !in || !p)
        return SIMNETS_ERR_NULL_POINTER;
    if (in[0] < 0)
        return SIMNETS_ERR_SHAPE;
    const int rc = mex_calc_dims_impl(a, in + 1, &p->d, true);
    if (rc)
        return rc;
    p->B = in[0]; p->C = in[1]; p->H = in[2]; p->W = in[3];
    p->softmax_mode = a->softmax_mode != 0;
    p->epsilon = a->epsilon;
    p->oob = a->blocks_out_of_bounds_value;
    p->use_unshared = a->use_unshared_regions != 0;
    p->normalize_offsets = a->normalize_offsets != 0;
    p->grad_pack = nullptr;
    if (std::isnan(a->epsilon) || a->epsilon == 0.0f)
        return SIMNETS_ERR_SHAPE;
    if (!fits_int32(1LL * p->B * p->d.region_size) || !fits_int32(1LL * p->d.num_regions * p->d.M * 1LL) )
        return SIMNETS_ERR_TOO_LARGE;
    return SIMNETS_OK;
}

}  // namespace simnets

using namespace simnets;

extern "C" {

int simnets_hip_abi_version(void) { return SIMNETS_HIP_ABI_VERSION; }

const char *simnets_hip_strerror(int status)
{
    switch (status) {
    case SIMNETS_OK: return "ok";
    case SIMNETS_ERR_NULL_POINTER: return "a required pointer argument is NULL";
    case SIMNETS_ERR_PADDING_LENGTH: return "padding must be a list with two elements (Similarity) or two/three elements (Mex)";
    case SIMNETS_ERR_BLOCKS_LENGTH: return "blocks must be a list with two elements (Similarity) / blocks should be a list with 3 elements (Mex)";
    case SIMNETS_ERR_STRIDES_LENGTH: return "stride must be a list with two elements (Similarity) / strides should be a list with 3 elements (Mex)";
    case SIMNETS_ERR_SIMILARITY_FUNCTION: return "similarity_function must be L1 or L2";
    case SIMNETS_ERR_NORMALIZATION_NEEDS_L2: return "normalization_term is relevant only if similarity_function is L2";
    case SIMNETS_ERR_IGNORE_NAN_NEEDS_NORM: return "ignore_nan is relevant only if normalization_term is true";
    case SIMNETS_ERR_TEMPLATE_CHANNELS: return "Number of channels mismatch between input and template";
    case SIMNETS_ERR_WEIGHTS_CHANNELS: return "Number of channels mismatch between input and weights";
    case SIMNETS_ERR_STRIDE_NOT_POSITIVE: return "Stride must be > 0";
    case SIMNETS_ERR_NUM_INSTANCES: return "num_instances must be positive";
    case SIMNETS_ERR_UNSHARED_REGION_LENGTH: return "unshared_offset_region should be a list with 1 or 3 elements";
    case SIMNETS_ERR_SHARED_REGION_LENGTH: return "shared_offset_region should be a list with 1 or 3 elements";
    case SIMNETS_ERR_BLOCK_DEPTH: return "block depth must be smaller than input depth";
    case SIMNETS_ERR_SHAPE: return "tensor shape or attribute value inconsistent with the operator definition";
    case SIMNETS_ERR_EMPTY_OUTPUT: return "an input or output dimension is not positive";
    case SIMNETS_ERR_WORKSPACE: return "workspace is missing, too small or not 256-byte aligned";
    case SIMNETS_ERR_ALGO: return "the requested algorithm does not support these attributes";
    case SIMNETS_ERR_TOO_LARGE: return "a per-image dimension product exceeds 32-bit indexing";
    case SIMNETS_ERR_HIP: return "a HIP runtime call or kernel launch failed (no usable gfx950 device?)";
    case SIMNETS_ERR_STATIC_SCRATCH: return "the call needs more scratch than the library's static device buffer holds (SIMNETS_HIP_STATIC_SCRATCH_BYTES); use the entry point that takes a workspace";
    default: return "unknown simnets status";
    }
}

void simnets_similarity_attrs_default(simnets_similarity_attrs *a)
{
    if (!a)
        return;
    std::memset(a, 0, sizeof(*a));
    a->similarity_function = SIMNETS_SIM_L2;
    a->n_blocks = 2; a->blocks[0] = 3; a->blocks[1] = 3;
    a->n_strides = 2; a->strides[0] = 2; a->strides[1] = 2;
    a->n_padding = 2; a->padding[0] = 0; a->padding[1] = 0;
    a->normalization_term = 0;
    a->normalization_term_fudge = 0.001f;
    a->ignore_nan_input = 0;
    a->out_of_bounds_value = 0.0f;
}

int simnets_similarity_out_shape(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                 const int templates_shape[4], const int weights_shape[4], int output_shape[4])
{
    SimPlan p;
    const int rc = sim_make_plan(attrs, input_shape, templates_shape, weights_shape, &p);
    if (rc)
        return rc;
    if (!output_shape)
        return SIMNETS_ERR_NULL_POINTER;
    output_shape[0] = p.B; output_shape[1] = p.O; output_shape[2] = p.oh; output_shape[3] = p.ow;
    return SIMNETS_OK;
}

int simnets_hip_similarity_workspace_bytes(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                           const int templates_shape[4], size_t *bytes)
{
    SimPlan p;
    const int rc = sim_make_plan(attrs, input_shape, templates_shape, templates_shape, &p);
    if (rc)
        return rc;
    if (!bytes)
        return SIMNETS_ERR_NULL_POINTER;
    *bytes = sim_workspace_bytes(p);
    return SIMNETS_OK;
}

int simnets_hip_similarity_grad_workspace_bytes(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                                const int templates_shape[4], size_t *input_grad_bytes,
                                                size_t *params_grad_bytes)
{
    SimPlan p;
    const int rc = sim_make_plan(attrs, input_shape, templates_shape, templates_shape, &p);
    if (rc)
        return rc;
    if (input_grad_bytes)
        *input_grad_bytes = sim_grad_input_workspace_bytes(p);
    if (params_grad_bytes)
        *params_grad_bytes = sim_grad_params_workspace_bytes(p);
    return SIMNETS_OK;
}

void simnets_mex_attrs_default(simnets_mex_attrs *a)
{
    if (!a)
        return;
    std::memset(a, 0, sizeof(*a));
    a->num_instances = 1;
    a->softmax_mode = 0;
    a->n_padding = 3;
    a->n_strides = 3; a->strides[0] = a->strides[1] = a->strides[2] = 1;
    a->n_blocks = 3; a->blocks[0] = a->blocks[1] = a->blocks[2] = 1;
    a->epsilon = 1.0f;
    a->blocks_out_of_bounds_value = 0.0f;
    a->blocks_round_down = 1;
    a->use_unshared_regions = 1;
    a->n_shared = 1; a->shared_offset_region[0] = -1;
    a->n_unshared = 1; a->unshared_offset_region[0] = -1;
}

int simnets_mex_calc_dims(const simnets_mex_attrs *attrs, const int image_chw[3], simnets_mex_dims *dims)
{
    return mex_calc_dims_impl(attrs, image_chw, dims, true);
}

int simnets_mex_out_shape(const simnets_mex_attrs *attrs, const int input_shape[4], int output_shape[4],
                          int offsets_shape[5])
{
    MexPlan p;
    const int rc = mex_make_plan(attrs, input_shape, &p);
    if (rc)
        return rc;
    if (output_shape) {
        output_shape[0] = p.B; output_shape[1] = p.d.channels_out_total;
        output_shape[2] = p.d.height_out; output_shape[3] = p.d.width_out;
    }
    if (offsets_shape) {
        offsets_shape[0] = p.d.num_regions; offsets_shape[1] = p.d.M;
        offsets_shape[2] = p.d.block_c; offsets_shape[3] = p.d.block_h; offsets_shape[4] = p.d.block_w;
    }
    return SIMNETS_OK;
}

int get_mex_offsets_nregions(int n_input_dim, const int *input_dim, int n_padding, const int *padding, int n_strides,
                             const int *strides, int num_instances, int blocks_round_down, int use_unshared_regions,
                             int n_blocks, const int *blocks, int n_shared_offset_region,
                             const int *shared_offset_region, int n_unshared_offset_region,
                             const int *unshared_offset_region)
{
    (void)n_input_dim;
    if (n_blocks != 3)
        return -1;  // mex_dims_helper.cpp:25-27
    if (!input_dim || !padding || !strides || !blocks || !shared_offset_region || !unshared_offset_region)
        return -1;
    simnets_mex_attrs a;
    simnets_mex_attrs_default(&a);
    auto fill = [](int n, const int *src, int *dst) {
        for (int i = 0; i < n && i < 3; ++i)
            dst[i] = src[i];
        return n;
    };
    a.num_instances = num_instances;
    a.n_padding = fill(n_padding, padding, a.padding);
    a.n_strides = fill(n_strides, strides, a.strides);
    a.n_blocks = fill(n_blocks, blocks, a.blocks);
    a.n_shared = fill(n_shared_offset_region, shared_offset_region, a.shared_offset_region);
    a.n_unshared = fill(n_unshared_offset_region, unshared_offset_region, a.unshared_offset_region);
    a.blocks_round_down = blocks_round_down > 0;
    a.use_unshared_regions = use_unshared_regions > 0;
    // The reference helper accepts the one-element defaults padding=[0] / strides=[1] that
    // python/simnets/ops/mex.py:19 passes when the caller omits them; widen them the same way
    // a three-element list of that value would behave for the region count.
    if (a.n_padding == 1) { a.padding[1] = a.padding[2] = a.padding[0]; a.n_padding = 3; }
    if (a.n_strides == 1) { a.strides[1] = a.strides[2] = a.strides[0]; a.n_strides = 3; }
    simnets_mex_dims d;
    const int rc = mex_calc_dims_impl(&a, input_dim, &d, false);
    if (rc)
        return -1;
    return d.num_regions;
}

int simnets_hip_mex_workspace_bytes(const simnets_mex_attrs *attrs, const int input_shape[4], size_t *bytes)
{
    MexPlan p;
    const int rc = mex_make_plan(attrs, input_shape, &p);
    if (rc)
        return rc;
    if (!bytes)
        return SIMNETS_ERR_NULL_POINTER;
    *bytes = mex_workspace_bytes(p);
    return SIMNETS_OK;
}

int simnets_hip_mex_grad_workspace_bytes(const simnets_mex_attrs *attrs, const int input_shape[4],
                                         size_t *input_grad_bytes, size_t *offsets_grad_bytes)
{
    MexPlan p;
    const int rc = mex_make_plan(attrs, input_shape, &p);
    if (rc)
        return rc;
    if (input_grad_bytes)
        *input_grad_bytes = mex_grad_input_workspace_bytes(p);
    if (offsets_grad_bytes)
        *offsets_grad_bytes = mex_grad_offsets_workspace_bytes(p);
    return SIMNETS_OK;
}

}  // extern "C"
