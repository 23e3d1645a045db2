// Compute entry points of the C ABI (include/simnets_hip.h): validate on the host, then enqueue.
#include <hip/hip_runtime.h>

#include <atomic>

#include "internal.h"

namespace simnets {

int sim_direct_launch(const SimPlan &p, const float *input, const float *templates, const float *weights,
                      float *output, void *workspace, size_t workspace_bytes, hipStream_t s);
size_t sim_mfma_workspace_bytes(const SimPlan &p);
int sim_mfma_launch(const SimPlan &p, const float *input, const float *templates, const float *weights, float *output,
                    void *workspace, size_t workspace_bytes, hipStream_t s);

int sim_direct_prepare(const SimPlan &p, const float *templates, const float *weights, void *workspace,
                       size_t workspace_bytes, hipStream_t s);
int sim_direct_run(const SimPlan &p, const float *input, float *output, void *workspace, size_t workspace_bytes,
                   hipStream_t s);
int sim_mfma_prepare(const SimPlan &p, const float *templates, const float *weights, void *workspace,
                     size_t workspace_bytes, hipStream_t s);
int sim_mfma_run(const SimPlan &p, const float *input, float *output, void *workspace, size_t workspace_bytes,
                 hipStream_t s);

size_t sim_workspace_bytes(const SimPlan &p)
{
    if (p.algo == SIMNETS_ALGO_MFMA)
        return sim_mfma_workspace_bytes(p);
    return sim_direct_workspace_bytes(p);
}

int sim_launch(const SimPlan &p, const float *input, const float *templates, const float *weights, float *output,
               void *workspace, size_t workspace_bytes, void *stream)
{
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (p.algo == SIMNETS_ALGO_MFMA)
        return sim_mfma_launch(p, input, templates, weights, output, workspace, workspace_bytes, s);
    return sim_direct_launch(p, input, templates, weights, output, workspace, workspace_bytes, s);
}

int sim_prepare(const SimPlan &p, const float *templates, const float *weights, void *prepared, size_t prepared_bytes,
                void *stream)
{
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (p.algo == SIMNETS_ALGO_MFMA)
        return sim_mfma_prepare(p, templates, weights, prepared, prepared_bytes, s);
    return sim_direct_prepare(p, templates, weights, prepared, prepared_bytes, s);
}

int sim_run(const SimPlan &p, const float *input, float *output, void *prepared, size_t prepared_bytes, void *stream)
{
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    if (p.algo == SIMNETS_ALGO_MFMA)
        return sim_mfma_run(p, input, output, prepared, prepared_bytes, s);
    return sim_direct_run(p, input, output, prepared, prepared_bytes, s);
}

}  // namespace simnets

using namespace simnets;

static bool workspace_ok(const void *workspace, size_t have, size_t need)
{
    return need == 0 || (workspace && have >= need && (reinterpret_cast<uintptr_t>(workspace) & 255) == 0);
}

// Scratch of simnets_hip_similarity_fwd_static: a fixed device array instead of a caller workspace.  Every GPU the
// library runs on holds its own copy, at its own address, until the process ends.  In host code the array's name
// is only a handle for hipGetSymbolAddress: the device address it yields (per device) is what kernels receive.
static __device__ __align__(256) unsigned char scratch[SIMNETS_HIP_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device, looked up once per device.
int static_scratch(void **ptr)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        return SIMNETS_ERR_HIP;
    void *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p)
            return SIMNETS_ERR_HIP;
        g_scratch_ptr[dev].store(p, std::memory_order_release);  // racing threads store the same address
    }
    *ptr = p;
    return SIMNETS_OK;
}
}  // namespace

extern "C" {

int simnets_hip_similarity_fwd_static(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                      const int templates_shape[4], const int weights_shape[4], const float *input,
                                      const float *templates, const float *weights, float *output, void *stream)
{
    SimPlan p;
    const int rc = sim_make_plan(attrs, input_shape, templates_shape, weights_shape, &p);
    if (rc)
        return rc;
    const size_t need = sim_workspace_bytes(p);
    if (need > SIMNETS_HIP_STATIC_SCRATCH_BYTES)
        return SIMNETS_ERR_STATIC_SCRATCH;
    if (p.B == 0)
        return SIMNETS_OK;
    if (!input || !templates || !weights || !output)
        return SIMNETS_ERR_NULL_POINTER;
    void *ws = nullptr;
    const int rs = static_scratch(&ws);
    if (rs)
        return rs;
    // the pack kernel rewrites every part of the scratch the main kernel reads (parameters, tables, thresholds)
    // and the main kernel writes every flag the recomputing pass reads, so nothing of an earlier call survives
    return sim_launch(p, input, templates, weights, output, ws, SIMNETS_HIP_STATIC_SCRATCH_BYTES, stream);
}

int simnets_hip_similarity_fwd(const simnets_similarity_attrs *attrs, const int input_shape[4],
                               const int templates_shape[4], const int weights_shape[4], const float *input,
                               const float *templates, const float *weights, float *output, void *workspace,
                               size_t workspace_bytes, void *stream)
{
    SimPlan p;
    const int rc = sim_make_plan(attrs, input_shape, templates_shape, weights_shape, &p);
    if (rc)
        return rc;
    if (p.B == 0)
        return SIMNETS_OK;
    if (!input || !templates || !weights || !output)
        return SIMNETS_ERR_NULL_POINTER;
    if (!workspace_ok(workspace, workspace_bytes, sim_workspace_bytes(p)))
        return SIMNETS_ERR_WORKSPACE;
    return sim_launch(p, input, templates, weights, output, workspace, workspace_bytes, stream);
}

int simnets_hip_similarity_prepare(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                   const int templates_shape[4], const int weights_shape[4], const float *templates,
                                   const float *weights, void *prepared, size_t prepared_bytes, void *stream)
{
    SimPlan p;
    const int rc = sim_make_plan(attrs, input_shape, templates_shape, weights_shape, &p);
    if (rc)
        return rc;
    if (!templates || !weights)
        return SIMNETS_ERR_NULL_POINTER;
    if (!workspace_ok(prepared, prepared_bytes, sim_workspace_bytes(p)))
        return SIMNETS_ERR_WORKSPACE;
    return sim_prepare(p, templates, weights, prepared, prepared_bytes, stream);
}

int simnets_hip_similarity_fwd_prepared(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                        const int templates_shape[4], const float *input, void *prepared,
                                        size_t prepared_bytes, float *output, void *stream)
{
    SimPlan p;
    const int rc = sim_make_plan(attrs, input_shape, templates_shape, templates_shape, &p);
    if (rc)
        return rc;
    if (p.B == 0)
        return SIMNETS_OK;
    if (!input || !output)
        return SIMNETS_ERR_NULL_POINTER;
    if (!workspace_ok(prepared, prepared_bytes, sim_workspace_bytes(p)))
        return SIMNETS_ERR_WORKSPACE;
    return sim_run(p, input, output, prepared, prepared_bytes, stream);
}

int simnets_hip_similarity_input_grad(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                      const int templates_shape[4], const int weights_shape[4], const float *input,
                                      const float *templates, const float *weights, const float *output_grad,
                                      float *input_grad, void *workspace, size_t workspace_bytes, void *stream)
{
    SimPlan p;
    const int rc = sim_make_plan(attrs, input_shape, templates_shape, weights_shape, &p);
    if (rc)
        return rc;
    if (p.B == 0)
        return SIMNETS_OK;
    if (!input || !templates || !weights || !output_grad || !input_grad)
        return SIMNETS_ERR_NULL_POINTER;
    if (!workspace_ok(workspace, workspace_bytes, sim_grad_input_workspace_bytes(p)))
        return SIMNETS_ERR_WORKSPACE;
    return sim_grad_input(p, input, templates, weights, output_grad, input_grad, workspace, workspace_bytes, stream);
}

int simnets_hip_similarity_params_grad(const simnets_similarity_attrs *attrs, const int input_shape[4],
                                       const int templates_shape[4], const int weights_shape[4], const float *input,
                                       const float *templates, const float *weights, const float *output_grad,
                                       float *templates_grad, float *weights_grad, void *workspace,
                                       size_t workspace_bytes, void *stream)
{
    SimPlan p;
    const int rc = sim_make_plan(attrs, input_shape, templates_shape, weights_shape, &p);
    if (rc)
        return rc;
    if (!templates || !weights || !templates_grad || !weights_grad || (p.B > 0 && (!input || !output_grad)))
        return SIMNETS_ERR_NULL_POINTER;
    if (!workspace_ok(workspace, workspace_bytes, sim_grad_params_workspace_bytes(p)))
        return SIMNETS_ERR_WORKSPACE;
    return sim_grad_params(p, input, templates, weights, output_grad, templates_grad, weights_grad, workspace,
                           workspace_bytes, stream);
}

static int mex_grad_checks(const simnets_mex_attrs *attrs, const int input_shape[4], size_t offsets_count,
                           MexPlan *p)
{
    const int rc = mex_make_plan(attrs, input_shape, p);
    if (rc)
        return rc;
    if (offsets_count < (size_t)p->d.num_regions * p->d.M * p->d.K)
        return SIMNETS_ERR_SHAPE;
    return SIMNETS_OK;
}

int simnets_hip_mex_input_grad(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                               const float *offsets, size_t offsets_count, const float *output,
                               const float *output_grad, float *input_grad, void *workspace, size_t workspace_bytes,
                               void *stream)
{
    MexPlan p;
    const int rc = mex_grad_checks(attrs, input_shape, offsets_count, &p);
    if (rc)
        return rc;
    if (p.B == 0)
        return SIMNETS_OK;
    if (!input || !offsets || !output || !output_grad || !input_grad)
        return SIMNETS_ERR_NULL_POINTER;
    if (!workspace_ok(workspace, workspace_bytes, mex_grad_input_workspace_bytes(p)))
        return SIMNETS_ERR_WORKSPACE;
    return mex_grad_input(p, input, offsets, output, output_grad, input_grad, workspace, workspace_bytes, stream);
}

int simnets_hip_mex_offsets_grad(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                 const float *offsets, size_t offsets_count, const float *output,
                                 const float *output_grad, float *offsets_grad, void *workspace,
                                 size_t workspace_bytes, void *stream)
{
    MexPlan p;
    const int rc = mex_grad_checks(attrs, input_shape, offsets_count, &p);
    if (rc)
        return rc;
    if (!offsets || !offsets_grad || (p.B > 0 && (!input || !output || !output_grad)))
        return SIMNETS_ERR_NULL_POINTER;
    if (!workspace_ok(workspace, workspace_bytes, mex_grad_offsets_workspace_bytes(p)))
        return SIMNETS_ERR_WORKSPACE;
    return mex_grad_offsets(p, input, offsets, output, output_grad, offsets_grad, workspace, workspace_bytes, stream);
}

int simnets_hip_mex_grads_workspace_bytes(const simnets_mex_attrs *attrs, const int input_shape[4], size_t *bytes)
{
    if (!bytes)
        return SIMNETS_ERR_NULL_POINTER;
    MexPlan p;
    const int rc = mex_make_plan(attrs, input_shape, &p);
    if (rc)
        return rc;
    *bytes = mex_grads_workspace_bytes(p, true, true);
    return SIMNETS_OK;
}

// the buffer a saving forward call filled, if the caller has one and the layer's gradient kernels read one
static int saved_pack(const MexPlan &p, const void *saved, size_t saved_bytes, const void **use)
{
    *use = nullptr;
    const size_t need = mex_grad_pack_bytes(p);
    if (saved == nullptr || need == 0)
        return SIMNETS_OK;
    if (!workspace_ok(saved, saved_bytes, need))
        return SIMNETS_ERR_WORKSPACE;
    *use = saved;
    return SIMNETS_OK;
}

int simnets_hip_mex_grads_saved(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                const float *offsets, size_t offsets_count, const float *output,
                                const float *output_grad, const void *saved, size_t saved_bytes, float *input_grad,
                                float *offsets_grad, void *workspace, size_t workspace_bytes, void *stream)
{
    MexPlan p;
    int rc = mex_grad_checks(attrs, input_shape, offsets_count, &p);
    if (rc)
        return rc;
    if (!offsets || !offsets_grad || (p.B > 0 && (!input || !output || !output_grad || !input_grad)))
        return SIMNETS_ERR_NULL_POINTER;
    if (!workspace_ok(workspace, workspace_bytes, mex_grads_workspace_bytes(p, true, true)))
        return SIMNETS_ERR_WORKSPACE;
    const void *pack;
    if ((rc = saved_pack(p, saved, saved_bytes, &pack)) != SIMNETS_OK)
        return rc;
    return mex_grads(p, input, offsets, output, output_grad, input_grad, offsets_grad, workspace, workspace_bytes,
                     stream, false, pack);
}

int simnets_hip_mex_grads(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                          const float *offsets, size_t offsets_count, const float *output, const float *output_grad,
                          float *input_grad, float *offsets_grad, void *workspace, size_t workspace_bytes,
                          void *stream)
{
    return simnets_hip_mex_grads_saved(attrs, input_shape, input, offsets, offsets_count, output, output_grad, nullptr,
                                       0, input_grad, offsets_grad, workspace, workspace_bytes, stream);
}

// scratch of simnets_hip_mex_sum_pool_grads: the gradient kernels' workspace, then the expanded pooling gradient
static size_t mex_pool_grads_scratch(const MexPlan &p, size_t *expanded_at)
{
    const size_t grads = align_up(mex_grads_workspace_bytes(p, true, true), 256);
    *expanded_at = grads;
    return grads + align_up((size_t)p.B * p.d.M * p.d.channels_out * p.d.height_out * p.d.width_out * sizeof(float), 256);
}

int simnets_hip_mex_sum_pool_grads_workspace_bytes(const simnets_mex_attrs *attrs, const int input_shape[4], int pool_h,
                                                   int pool_w, size_t *bytes)
{
    if (!bytes)
        return SIMNETS_ERR_NULL_POINTER;
    MexPlan p;
    const int rc = mex_make_plan(attrs, input_shape, &p);
    if (rc)
        return rc;
    if (pool_h <= 0 || pool_w <= 0)
        return SIMNETS_ERR_SHAPE;
    size_t at;
    *bytes = mex_pool_grads_scratch(p, &at);
    return SIMNETS_OK;
}

int simnets_hip_mex_sum_pool_grads(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                   const float *offsets, size_t offsets_count, int pool_h, int pool_w,
                                   const float *mex_output, const float *pooled_output_grad, float *input_grad,
                                   float *offsets_grad, void *workspace, size_t workspace_bytes, void *stream)
{
    return simnets_hip_mex_sum_pool_grads_saved(attrs, input_shape, input, offsets, offsets_count, pool_h, pool_w,
                                                mex_output, pooled_output_grad, nullptr, 0, input_grad, offsets_grad,
                                                workspace, workspace_bytes, stream);
}

int simnets_hip_mex_sum_pool_grads_saved(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                         const float *offsets, size_t offsets_count, int pool_h, int pool_w,
                                         const float *mex_output, const float *pooled_output_grad, const void *saved,
                                         size_t saved_bytes, float *input_grad, float *offsets_grad, void *workspace,
                                         size_t workspace_bytes, void *stream)
{
    MexPlan p;
    int rc = mex_grad_checks(attrs, input_shape, offsets_count, &p);
    if (rc)
        return rc;
    if (pool_h <= 0 || pool_w <= 0)
        return SIMNETS_ERR_SHAPE;
    if (p.d.height_out / pool_h <= 0 || p.d.width_out / pool_w <= 0)
        return SIMNETS_ERR_EMPTY_OUTPUT;
    if (!offsets || (!offsets_grad && !input_grad) ||
        (p.B > 0 && (!input || !mex_output || !pooled_output_grad)))
        return SIMNETS_ERR_NULL_POINTER;
    size_t expanded_at;
    const size_t need = mex_pool_grads_scratch(p, &expanded_at);
    if (!workspace_ok(workspace, workspace_bytes, need))
        return SIMNETS_ERR_WORKSPACE;
    const void *pack;
    if ((rc = saved_pack(p, saved, saved_bytes, &pack)) != SIMNETS_OK)
        return rc;
    if (p.B > 0 && pool_h == 2 && pool_w == 2 && mex_grads_take_pooled(p, input, mex_output, pooled_output_grad, input_grad))
        return mex_grads(p, input, offsets, mex_output, pooled_output_grad, input_grad, offsets_grad, workspace,
                         expanded_at, stream, true, pack);
    float *expanded = reinterpret_cast<float *>(reinterpret_cast<char *>(workspace) + expanded_at);
    if (p.B > 0) {
        const int erc = sum_pool_grad_launch(p.B, p.d.M * p.d.channels_out, p.d.height_out, p.d.width_out, pool_h, pool_w,
                                             pooled_output_grad, expanded, stream);
        if (erc)
            return erc;
    }
    return mex_grads(p, input, offsets, mex_output, expanded, input_grad, offsets_grad, workspace, expanded_at, stream,
                     false, pack);
}

// A forward call that also leaves the offsets as the gradient kernels read them in `saved`: the plan asks the
// forward's pack launch to write them; a forward that launched none (it packs inside its kernel) is followed by the
// gradient kernels' own pack launch.
static int saving_begin(MexPlan &p, MexGradPack *gp, void *saved, size_t saved_bytes)
{
    gp->buffer = nullptr; gp->written = false;
    const size_t need = mex_grad_pack_bytes(p);
    if (need == 0)
        return SIMNETS_OK;
    if (!workspace_ok(saved, saved_bytes, need))
        return SIMNETS_ERR_WORKSPACE;
    gp->buffer = saved;
    p.grad_pack = gp;
    return SIMNETS_OK;
}
static int saving_end(const MexPlan &p, const MexGradPack &gp, const float *offsets, void *stream)
{
    if (gp.buffer == nullptr || gp.written)
        return SIMNETS_OK;
    return mex_grad_pack_launch(p, offsets, gp.buffer, stream);
}

int simnets_hip_mex_saved_bytes(const simnets_mex_attrs *attrs, const int input_shape[4], size_t *bytes)
{
    if (!bytes)
        return SIMNETS_ERR_NULL_POINTER;
    MexPlan p;
    const int rc = mex_make_plan(attrs, input_shape, &p);
    if (rc)
        return rc;
    *bytes = mex_grad_pack_bytes(p);
    return SIMNETS_OK;
}

static int mex_fwd_phase(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                         const float *offsets, size_t offsets_count, float *output, void *workspace,
                         size_t workspace_bytes, void *stream, int phase, bool saving = false, void *saved = nullptr,
                         size_t saved_bytes = 0)
{
    MexPlan p;
    int rc = mex_make_plan(attrs, input_shape, &p);
    if (rc)
        return rc;
    if ((phase & kMexPrepare) && offsets_count < (size_t)p.d.num_regions * p.d.M * p.d.K)
        return SIMNETS_ERR_SHAPE;
    if (p.B == 0 && phase != kMexPrepare)
        return SIMNETS_OK;
    if (((phase & kMexRun) && (!input || !output)) || ((phase & kMexPrepare) && !offsets))
        return SIMNETS_ERR_NULL_POINTER;
    if (!workspace_ok(workspace, workspace_bytes, mex_workspace_bytes(p)))
        return SIMNETS_ERR_WORKSPACE;
    MexGradPack gp;
    if (saving && (rc = saving_begin(p, &gp, saved, saved_bytes)) != SIMNETS_OK)
        return rc;
    rc = mex_launch(p, input, offsets, output, workspace, workspace_bytes, stream, phase);
    return rc != SIMNETS_OK || !saving ? rc : saving_end(p, gp, offsets, stream);
}

int simnets_hip_mex_fwd_saving(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                               const float *offsets, size_t offsets_count, float *output, void *saved,
                               size_t saved_bytes, void *workspace, size_t workspace_bytes, void *stream)
{
    return mex_fwd_phase(attrs, input_shape, input, offsets, offsets_count, output, workspace, workspace_bytes, stream,
                         kMexWhole, true, saved, saved_bytes);
}

int simnets_hip_mex_fwd(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                        const float *offsets, size_t offsets_count, float *output, void *workspace,
                        size_t workspace_bytes, void *stream)
{
    return mex_fwd_phase(attrs, input_shape, input, offsets, offsets_count, output, workspace, workspace_bytes, stream,
                         kMexWhole);
}

int simnets_hip_mex_prepare(const simnets_mex_attrs *attrs, const int input_shape[4], const float *offsets,
                            size_t offsets_count, void *prepared, size_t prepared_bytes, void *stream)
{
    return mex_fwd_phase(attrs, input_shape, nullptr, offsets, offsets_count, nullptr, prepared, prepared_bytes, stream,
                         kMexPrepare);
}

int simnets_hip_mex_fwd_prepared(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                 void *prepared, size_t prepared_bytes, float *output, void *stream)
{
    return mex_fwd_phase(attrs, input_shape, input, nullptr, 0, output, prepared, prepared_bytes, stream, kMexRun);
}

int simnets_hip_sum_pool_fwd(const int input_shape[4], int pool_h, int pool_w, const float *input, float *output,
                             void *stream)
{
    if (!input_shape)
        return SIMNETS_ERR_NULL_POINTER;
    if (pool_h <= 0 || pool_w <= 0 || input_shape[0] < 0 || input_shape[1] <= 0 || input_shape[2] <= 0 ||
        input_shape[3] <= 0)
        return SIMNETS_ERR_SHAPE;
    if (input_shape[2] / pool_h <= 0 || input_shape[3] / pool_w <= 0)
        return SIMNETS_ERR_EMPTY_OUTPUT;
    if (input_shape[0] == 0)
        return SIMNETS_OK;
    if (!input || !output)
        return SIMNETS_ERR_NULL_POINTER;
    return sum_pool_launch(input_shape[0], input_shape[1], input_shape[2], input_shape[3], pool_h, pool_w, input,
                           output, stream);
}

int simnets_hip_sum_pool_input_grad(const int input_shape[4], int pool_h, int pool_w, const float *output_grad,
                                    float *input_grad, void *stream)
{
    if (!input_shape)
        return SIMNETS_ERR_NULL_POINTER;
    if (pool_h <= 0 || pool_w <= 0 || input_shape[0] < 0 || input_shape[1] <= 0 || input_shape[2] <= 0 ||
        input_shape[3] <= 0)
        return SIMNETS_ERR_SHAPE;
    if (input_shape[2] / pool_h <= 0 || input_shape[3] / pool_w <= 0)
        return SIMNETS_ERR_EMPTY_OUTPUT;
    if (input_shape[0] == 0)
        return SIMNETS_OK;
    if (!output_grad || !input_grad)
        return SIMNETS_ERR_NULL_POINTER;
    return sum_pool_grad_launch(input_shape[0], input_shape[1], input_shape[2], input_shape[3], pool_h, pool_w,
                                output_grad, input_grad, stream);
}

int simnets_hip_mex_sum_pool_workspace_bytes(const simnets_mex_attrs *attrs, const int input_shape[4], int pool_h,
                                             int pool_w, size_t *bytes)
{
    if (!bytes)
        return SIMNETS_ERR_NULL_POINTER;
    MexPlan p;
    const int rc = mex_make_plan(attrs, input_shape, &p);
    if (rc)
        return rc;
    if (pool_h <= 0 || pool_w <= 0)
        return SIMNETS_ERR_SHAPE;
    if (p.d.height_out / pool_h <= 0 || p.d.width_out / pool_w <= 0)
        return SIMNETS_ERR_EMPTY_OUTPUT;
    *bytes = mex_pool_workspace_bytes(p, pool_h, pool_w);
    return SIMNETS_OK;
}

static int mex_sum_pool_phase(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                              const float *offsets, size_t offsets_count, int pool_h, int pool_w, float *output,
                              void *workspace, size_t workspace_bytes, void *stream, int phase,
                              float *mex_output = nullptr, bool saving = false, void *saved = nullptr,
                              size_t saved_bytes = 0)
{
    MexPlan p;
    int rc = mex_make_plan(attrs, input_shape, &p);
    if (rc)
        return rc;
    if (pool_h <= 0 || pool_w <= 0 ||
        ((phase & kMexPrepare) && offsets_count < (size_t)p.d.num_regions * p.d.M * p.d.K))
        return SIMNETS_ERR_SHAPE;
    if (p.d.height_out / pool_h <= 0 || p.d.width_out / pool_w <= 0)
        return SIMNETS_ERR_EMPTY_OUTPUT;
    if (p.B == 0 && phase != kMexPrepare)
        return SIMNETS_OK;
    if (((phase & kMexRun) && (!input || !output)) || ((phase & kMexPrepare) && !offsets))
        return SIMNETS_ERR_NULL_POINTER;
    if (!workspace_ok(workspace, workspace_bytes, mex_pool_workspace_bytes(p, pool_h, pool_w)))
        return SIMNETS_ERR_WORKSPACE;
    MexGradPack gp;
    if (saving && (rc = saving_begin(p, &gp, saved, saved_bytes)) != SIMNETS_OK)
        return rc;
    rc = mex_pool_launch(p, pool_h, pool_w, input, offsets, output, workspace, workspace_bytes, stream, phase,
                         mex_output);
    return rc != SIMNETS_OK || !saving ? rc : saving_end(p, gp, offsets, stream);
}

int simnets_hip_mex_sum_pool_fwd_saving(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                        const float *offsets, size_t offsets_count, int pool_h, int pool_w,
                                        float *mex_output, float *output, void *saved, size_t saved_bytes,
                                        void *workspace, size_t workspace_bytes, void *stream)
{
    if (!mex_output && input_shape[0] != 0)
        return SIMNETS_ERR_NULL_POINTER;
    return mex_sum_pool_phase(attrs, input_shape, input, offsets, offsets_count, pool_h, pool_w, output, workspace,
                              workspace_bytes, stream, kMexWhole, mex_output, true, saved, saved_bytes);
}

int simnets_hip_mex_sum_pool_fwd_both(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                      const float *offsets, size_t offsets_count, int pool_h, int pool_w,
                                      float *mex_output, float *output, void *workspace, size_t workspace_bytes,
                                      void *stream)
{
    if (!mex_output && input_shape[0] != 0)
        return SIMNETS_ERR_NULL_POINTER;
    return mex_sum_pool_phase(attrs, input_shape, input, offsets, offsets_count, pool_h, pool_w, output, workspace,
                              workspace_bytes, stream, kMexWhole, mex_output);
}

int simnets_hip_mex_sum_pool_fwd(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                 const float *offsets, size_t offsets_count, int pool_h, int pool_w, float *output,
                                 void *workspace, size_t workspace_bytes, void *stream)
{
    return mex_sum_pool_phase(attrs, input_shape, input, offsets, offsets_count, pool_h, pool_w, output, workspace,
                              workspace_bytes, stream, kMexWhole);
}

int simnets_hip_mex_sum_pool_prepare(const simnets_mex_attrs *attrs, const int input_shape[4], const float *offsets,
                                     size_t offsets_count, int pool_h, int pool_w, void *prepared,
                                     size_t prepared_bytes, void *stream)
{
    return mex_sum_pool_phase(attrs, input_shape, nullptr, offsets, offsets_count, pool_h, pool_w, nullptr, prepared,
                              prepared_bytes, stream, kMexPrepare);
}

int simnets_hip_mex_sum_pool_fwd_prepared(const simnets_mex_attrs *attrs, const int input_shape[4], const float *input,
                                          int pool_h, int pool_w, void *prepared, size_t prepared_bytes, float *output,
                                          void *stream)
{
    return mex_sum_pool_phase(attrs, input_shape, input, nullptr, 0, pool_h, pool_w, output, prepared, prepared_bytes,
                              stream, kMexRun);
}

static int sim_mex_pool_plans(const simnets_similarity_attrs *sim_attrs, const int input_shape[4],
                              const int templates_shape[4], const simnets_mex_attrs *mex_attrs, int pool_h, int pool_w,
                              SimPlan *sp, MexPlan *mp)
{
    int rc = sim_make_plan(sim_attrs, input_shape, templates_shape, templates_shape, sp);
    if (rc)
        return rc;
    const int mid[4] = {sp->B, sp->O, sp->oh, sp->ow};
    rc = mex_make_plan(mex_attrs, mid, mp);
    if (rc)
        return rc;
    if (pool_h <= 0 || pool_w <= 0)
        return SIMNETS_ERR_SHAPE;
    if (mp->d.height_out / pool_h <= 0 || mp->d.width_out / pool_w <= 0)
        return SIMNETS_ERR_EMPTY_OUTPUT;
    return SIMNETS_OK;
}

int simnets_hip_similarity_mex_sum_pool_workspace_bytes(const simnets_similarity_attrs *sim_attrs,
                                                        const int input_shape[4], const int templates_shape[4],
                                                        const simnets_mex_attrs *mex_attrs, int pool_h, int pool_w,
                                                        size_t *bytes)
{
    if (!bytes)
        return SIMNETS_ERR_NULL_POINTER;
    SimPlan sp;
    MexPlan mp;
    const int rc = sim_mex_pool_plans(sim_attrs, input_shape, templates_shape, mex_attrs, pool_h, pool_w, &sp, &mp);
    if (rc)
        return rc;
    *bytes = sim_mex_pool_workspace_bytes(sp, mp, pool_h, pool_w);
    return SIMNETS_OK;
}

static int sim_mex_pool_phase(const simnets_similarity_attrs *sim_attrs, const int input_shape[4],
                              const int templates_shape[4], const float *input, const float *templates,
                              const float *weights, const simnets_mex_attrs *mex_attrs, const float *offsets,
                              size_t offsets_count, int pool_h, int pool_w, float *output, void *workspace,
                              size_t workspace_bytes, void *stream, int phase)
{
    SimPlan sp;
    MexPlan mp;
    const int rc = sim_mex_pool_plans(sim_attrs, input_shape, templates_shape, mex_attrs, pool_h, pool_w, &sp, &mp);
    if (rc)
        return rc;
    if ((phase & kMexPrepare) && offsets_count < (size_t)mp.d.num_regions * mp.d.M * mp.d.K)
        return SIMNETS_ERR_SHAPE;
    if (sp.B == 0 && phase != kMexPrepare)
        return SIMNETS_OK;
    if (((phase & kMexRun) && (!input || !output)) || ((phase & kMexPrepare) && (!templates || !weights || !offsets)))
        return SIMNETS_ERR_NULL_POINTER;
    if (!workspace_ok(workspace, workspace_bytes, sim_mex_pool_workspace_bytes(sp, mp, pool_h, pool_w)))
        return SIMNETS_ERR_WORKSPACE;
    return sim_mex_pool_launch(sp, mp, pool_h, pool_w, input, templates, weights, offsets, output, workspace,
                               workspace_bytes, stream, phase);
}

int simnets_hip_similarity_mex_sum_pool_fwd(const simnets_similarity_attrs *sim_attrs, const int input_shape[4],
                                            const int templates_shape[4], const float *input, const float *templates,
                                            const float *weights, const simnets_mex_attrs *mex_attrs,
                                            const float *offsets, size_t offsets_count, int pool_h, int pool_w,
                                            float *output, void *workspace, size_t workspace_bytes, void *stream)
{
    return sim_mex_pool_phase(sim_attrs, input_shape, templates_shape, input, templates, weights, mex_attrs, offsets,
                              offsets_count, pool_h, pool_w, output, workspace, workspace_bytes, stream, kMexWhole);
}

int simnets_hip_similarity_mex_sum_pool_prepare(const simnets_similarity_attrs *sim_attrs, const int input_shape[4],
                                                const int templates_shape[4], const float *templates,
                                                const float *weights, const simnets_mex_attrs *mex_attrs,
                                                const float *offsets, size_t offsets_count, int pool_h, int pool_w,
                                                void *prepared, size_t prepared_bytes, void *stream)
{
    return sim_mex_pool_phase(sim_attrs, input_shape, templates_shape, nullptr, templates, weights, mex_attrs, offsets,
                              offsets_count, pool_h, pool_w, nullptr, prepared, prepared_bytes, stream, kMexPrepare);
}

int simnets_hip_similarity_mex_sum_pool_fwd_prepared(const simnets_similarity_attrs *sim_attrs,
                                                     const int input_shape[4], const int templates_shape[4],
                                                     const float *input, const simnets_mex_attrs *mex_attrs, int pool_h,
                                                     int pool_w, void *prepared, size_t prepared_bytes, float *output,
                                                     void *stream)
{
    return sim_mex_pool_phase(sim_attrs, input_shape, templates_shape, input, nullptr, nullptr, mex_attrs, nullptr, 0,
                              pool_h, pool_w, output, prepared, prepared_bytes, stream, kMexRun);
}

}  // extern "C"
