/*
 * CPU oracle for the SimNets Similarity / MEX forward operators: dimension logic and the
 * two instantiations (fp32, fp64) of the arithmetic in simnets_oracle_impl.inc.
 * Test infrastructure only; see simnets_oracle.h for the rules and for how it is pinned.
 *
 * Build: gcc -O2 -std=c11 -ffp-contract=off -fno-fast-math -fPIC -shared (oracle/Makefile).
 */
#define _GNU_SOURCE
#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#include "simnets_oracle.h"

#ifndef M_PI
#define M_PI 3.14159265358979323846
#endif

/* include/utils/im2col.hpp:101-108 */
int so_dimension_out_size(int image_size, int pad_size, int patch_size, int stride, int round_down)
{
    if (round_down)
        return (image_size + 2 * pad_size - patch_size) / stride + 1;
    return (int)ceilf((float)(image_size + 2 * pad_size - patch_size) / stride) + 1;
}

/* include/utils/ggemm_cpu.hpp:451-460 (BLOCK_WIDTH = BLOCK_HEIGHT = 16) */
static int so_ceiled_div(int a, int b) { return (a / b) + ((a % b) > 0); }
int so_ggemm_padded_output_size(int M, int N)
{
    const int newN = so_ceiled_div(N, 16) * 16;
    const int newM = so_ceiled_div(M, 16) * 16;
    return newN * newM - M * N;
}

/* include/kernels/similarity_kernel_common.hpp:82-111 (attribute checks), :113-164 (dims);
 * stride > 0 from include/utils/im2col.hpp:116-118. */
int so_similarity_out_dims(const so_similarity_args *a, int *out_h, int *out_w)
{
    if (a->similarity_function != SO_SIM_L1 && a->similarity_function != SO_SIM_L2)
        return -1;
    if (a->normalization_term && a->similarity_function != SO_SIM_L2)
        return -2; /* "normalization_term is relevant only if similarity_function is L2" */
    if (a->ignore_nan_input && !a->normalization_term)
        return -3; /* "ignore_nan is relevant only if normalization_term is true" */
    if (a->stride_h <= 0 || a->stride_w <= 0)
        return -4;
    *out_h = so_dimension_out_size(a->height, a->pad_h, a->block_h, a->stride_h, 1);
    *out_w = so_dimension_out_size(a->width, a->pad_w, a->block_w, a->stride_w, 1);
    return 0;
}

/* src/kernels/mex_kernel_common.cpp:8-27 */
static void so_expand_dim_spec(const int image_chw[3], int n, const int *spec, int out[3])
{
    int i0 = 0;
    if (n == 2) {
        out[0] = -1;
        i0 = 1;
    }
    for (int i = 0; i < n && i0 + i < 3; ++i)
        out[i0 + i] = spec[i];
    for (int i = 0; i < 3; ++i)
        if (out[i] == -1)
            out[i] = image_chw[i];
}

static int so_min(int a, int b) { return a < b ? a : b; }

/* src/kernels/mex_kernel_common.cpp:29-58 (attribute checks), :63-158 (CalculateDimensions),
 * :169 (block depth check). */
int so_mex_calc_dims(const so_mex_args *a, so_mex_dims *d)
{
    if (a->num_instances <= 0)
        return -1;
    if (a->n_strides != 3)
        return -2;
    if (a->n_blocks != 3)
        return -3;
    if (a->n_unshared != 3 && a->n_unshared != 1)
        return -4;
    if (a->n_shared != 3 && a->n_shared != 1)
        return -5;
    if (a->n_padding != 3 && a->n_padding != 2)
        return -6;
    const int image[3] = {a->channels, a->height, a->width};
    int pad[3], str[3];
    so_expand_dim_spec(image, a->n_padding, a->padding, pad);
    so_expand_dim_spec(image, a->n_strides, a->strides, str);
    if (str[0] <= 0 || str[1] <= 0 || str[2] <= 0)
        return -7;
    memset(d, 0, sizeof(*d));
    d->pad_c = pad[0]; d->pad_h = pad[1]; d->pad_w = pad[2];
    d->stride_c = str[0]; d->stride_h = str[1]; d->stride_w = str[2];
    d->block_c = a->blocks[0]; d->block_h = a->blocks[1]; d->block_w = a->blocks[2];

    d->height_out = so_dimension_out_size(a->height, d->pad_h, d->block_h, d->stride_h, a->blocks_round_down);
    d->width_out = so_dimension_out_size(a->width, d->pad_w, d->block_w, d->stride_w, a->blocks_round_down);
    d->channels_out = so_dimension_out_size(a->channels, d->pad_c, d->block_c, d->stride_c, a->blocks_round_down);
    /* A block larger than the padded image leaves an output extent of zero or less; the reference goes on and divides
     * by the region extent it derives from it (an integer division by zero).  The checker reports it instead. */
    if (d->height_out <= 0 || d->width_out <= 0 || d->channels_out <= 0)
        return -9;

    if (!a->use_unshared_regions) {
        int sc, sh, sw;
        if (a->n_shared == 3) {
            sc = a->shared_offset_region[0]; sh = a->shared_offset_region[1]; sw = a->shared_offset_region[2];
        } else {
            sw = sh = a->shared_offset_region[0];
            sc = -1;
        }
        if (sh < 0) sh = d->height_out;
        sh = so_min(sh, d->height_out);
        if (sw < 0) sw = d->width_out;
        sw = so_min(sw, d->width_out);
        if (sc < 0) sc = d->channels_out;
        sc = so_min(sc, d->channels_out);
        if (sc == 0 || sh == 0 || sw == 0)
            return -9; /* (a region extent of zero: the same division) */
        d->shared_region_c = sc; d->shared_region_h = sh; d->shared_region_w = sw;
        d->offsets_h = so_ceiled_div(d->height_out, sh);
        d->offsets_w = so_ceiled_div(d->width_out, sw);
        d->offsets_c = so_ceiled_div(d->channels_out, sc);
    } else {
        int uc, uh, uw;
        if (a->n_unshared == 3) {
            uc = a->unshared_offset_region[0]; uh = a->unshared_offset_region[1]; uw = a->unshared_offset_region[2];
        } else {
            uw = uh = a->unshared_offset_region[0];
            uc = -1;
        }
        if (uh < 0) uh = d->height_out;
        uh = so_min(uh, d->height_out);
        if (uw < 0) uw = d->width_out;
        uw = so_min(uw, d->width_out);
        if (uc < 0) uc = d->channels_out;
        uc = so_min(uc, d->channels_out);
        if (uc == 0 || uh == 0 || uw == 0)
            return -9;
        d->offsets_h = uh; d->offsets_w = uw; d->offsets_c = uc;
        d->shared_region_h = so_ceiled_div(d->height_out, uh);
        d->shared_region_w = so_ceiled_div(d->width_out, uw);
        d->shared_region_c = so_ceiled_div(d->channels_out, uc);
    }
    d->num_regions = d->offsets_h * d->offsets_w * d->offsets_c;
    d->region_size = d->shared_region_w * d->shared_region_h * d->shared_region_c;
    d->channels_out_total = d->channels_out * a->num_instances;
    d->M = a->num_instances;
    d->K = d->block_c * d->block_h * d->block_w;
    d->N = d->height_out * d->width_out * d->channels_out;
    d->is_1x1 = (d->block_c == a->channels || (d->block_c == 1 && d->stride_c == 1)) && d->block_w == 1 &&
                d->block_h == 1 && d->stride_h == 1 && d->stride_w == 1 && d->pad_c == 0 && d->pad_h == 0 &&
                d->pad_w == 0;
    if (d->block_c > a->channels)
        return -8; /* "block depth must be smaller than input depth" */
    return 0;
}

#define REAL float
#define SFX(n) n##_f32
#define R_LOG logf
#define R_EXP expf
#define R_ABS fabsf
#include "simnets_oracle_impl.inc"
#undef REAL
#undef SFX
#undef R_LOG
#undef R_EXP
#undef R_ABS

#define REAL double
#define SFX(n) n##_f64
#define R_LOG log
#define R_EXP exp
#define R_ABS fabs
#include "simnets_oracle_impl.inc"
#undef REAL
#undef SFX
#undef R_LOG
#undef R_EXP
#undef R_ABS
