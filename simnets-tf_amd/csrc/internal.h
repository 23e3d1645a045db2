// Internal declarations shared by the host logic and the kernel launchers of libsimnets_hip.
#pragma once

#include <cstddef>
#include <cstdint>

#include "simnets_hip.h"

namespace simnets {

// Which combine the Similarity ggemm applies (the dispatch of
// src/kernels/similarity_kernel_cpu.cpp:84-116 in the reference).
enum SimMode { SIM_MODE_L1 = 0, SIM_MODE_L2 = 1, SIM_MODE_L2_NORM = 2, SIM_MODE_L2_NORM_IGNORE_NAN = 3,
               SIM_MODE_L2_SQRTW = 4 /* internal: plain L2 evaluated as -(sqrt(w) t - sqrt(w) x)^2 */ };

struct SimPlan {
    int B, C, H, W, O;
    int bh, bw, sh, sw, ph, pw;
    int oh, ow, K;
    int mode;  // SimMode
    int algo;  // resolved SIMNETS_ALGO_* (never AUTO)
    int exact_terms;  // the caller named SIMNETS_ALGO_DIRECT: gradients, too, sum the reference's terms one by one
    float fudge, oob;
    int norm_const_every_iteration;
};

// Validates like SimilarityKernelCommon (ctor + CalculateDimensions) and fills the plan.
int sim_make_plan(const simnets_similarity_attrs *attrs, const int input_shape[4], const int templates_shape[4],
                  const int weights_shape[4], SimPlan *plan);

size_t sim_workspace_bytes(const SimPlan &p);
size_t sim_direct_workspace_bytes(const SimPlan &p);
int sim_launch(const SimPlan &p, const float *input, const float *templates, const float *weights, float *output,
               void *workspace, size_t workspace_bytes, void *stream);

// The forward call in two halves: everything that depends on the parameters only, and the launches that read it.
int sim_prepare(const SimPlan &p, const float *templates, const float *weights, void *prepared, size_t prepared_bytes,
                void *stream);
int sim_run(const SimPlan &p, const float *input, float *output, void *prepared, size_t prepared_bytes, void *stream);

// where a forward call leaves the offsets as the gradient kernels read them (mex_grad_pack_bytes)
struct MexGradPack {
    void *buffer;
    bool written;   // set by the forward's pack launch when it wrote the buffer
};

struct MexPlan {
    int B, C, H, W;
    simnets_mex_dims d;
    int softmax_mode;
    float epsilon, oob;
    int use_unshared;
    int normalize_offsets;
    MexGradPack *grad_pack;   // forward calls that keep the gradient kernels' offsets layout; else null
};

int mex_make_plan(const simnets_mex_attrs *attrs, const int input_shape[4], MexPlan *plan);
size_t mex_workspace_bytes(const MexPlan &p);
// The forward calls in two halves (`phase`): the launch that depends on the parameters alone, and the launches that
// read what it wrote; the default is the whole call.
enum { kMexPrepare = 1, kMexRun = 2, kMexWhole = 3 };
int mex_launch(const MexPlan &p, const float *input, const float *offsets, float *output, void *workspace,
               size_t workspace_bytes, void *stream, int phase = kMexWhole);

// Backward operators (similarity_grad.hip, mex_grad.hip).  `stream` is a hipStream_t.
// Input gradient of the L2 modes at stride 1 on the matrix cores (similarity_mfma.hip)
bool sim_mfma_grad_input_supported(const SimPlan &p);
size_t sim_mfma_grad_input_workspace_bytes(const SimPlan &p);
int sim_mfma_grad_input_launch(const SimPlan &p, const float *input, const float *templates, const float *weights,
                               const float *output_grad, float *input_grad, void *workspace, size_t workspace_bytes,
                               void *stream);
size_t sim_grad_input_workspace_bytes(const SimPlan &p);
size_t sim_grad_params_workspace_bytes(const SimPlan &p);
int sim_grad_input(const SimPlan &p, const float *input, const float *templates, const float *weights,
                   const float *output_grad, float *input_grad, void *workspace, size_t workspace_bytes, void *stream);
int sim_grad_params(const SimPlan &p, const float *input, const float *templates, const float *weights,
                    const float *output_grad, float *templates_grad, float *weights_grad, void *workspace,
                    size_t workspace_bytes, void *stream);
size_t mex_grad_input_workspace_bytes(const MexPlan &p);
size_t mex_grad_offsets_workspace_bytes(const MexPlan &p);
size_t mex_grads_workspace_bytes(const MexPlan &p, bool want_input, bool want_offsets);
// either gradient or both: a null gradient pointer skips one
// grad_is_pooled: output_grad is the gradient of the 2 x 2 sum-pooled output (only where mex_grads_take_pooled says so)
int mex_grads(const MexPlan &p, const float *input, const float *offsets, const float *output,
              const float *output_grad, float *input_grad, float *offsets_grad, void *workspace,
              size_t workspace_bytes, void *stream, bool grad_is_pooled = false, const void *saved = nullptr);
// `saved`: the buffer (mex_grad_pack_bytes, declared with the packing in mex_common.h) that a forward call of the same
// layer and offsets filled, through MexPlan::grad_pack or mex_grad_pack_launch; the call then packs nothing.
size_t mex_grad_pack_bytes(const MexPlan &p);   // 0: the layer's gradient kernels read no packed offsets
// whether they read the packed layout at all (finite epsilon, not the kernel for few instances over long patches,
// which takes the offsets - or the normalised copy, which the buffer then holds alone - as they are)
bool mex_grads_read_packed(const MexPlan &p);
int mex_grad_pack_launch(const MexPlan &p, const float *offsets, void *buffer, void *stream);
// whether the gradient kernels of this layer read the pooled gradient themselves (one output channel per instance,
// even output height and width: every output pixel then has a window; input_grad may be null)
bool mex_grads_take_pooled(const MexPlan &p, const float *input, const float *output, const float *pooled_grad,
                           const float *input_grad);
int mex_grad_input(const MexPlan &p, const float *input, const float *offsets, const float *output,
                   const float *output_grad, float *input_grad, void *workspace, size_t workspace_bytes, void *stream);
int mex_grad_offsets(const MexPlan &p, const float *input, const float *offsets, const float *output,
                     const float *output_grad, float *offsets_grad, void *workspace, size_t workspace_bytes,
                     void *stream);

int sum_pool_launch(int B, int C, int H, int W, int ph, int pw, const float *input, float *output, void *stream);
int sum_pool_grad_launch(int B, int C, int H, int W, int ph, int pw, const float *output_grad, float *input_grad,
                         void *stream);
// MEX followed by non-overlapping sum pooling: one fused kernel when a pooling window is one pixel of every
// offsets region, else MEX into scratch + pooling
size_t mex_pool_workspace_bytes(const MexPlan &p, int ph, int pw);
// `full` (optional): the launch also stores the MEX output before pooling there (what the gradient operators read)
int mex_pool_launch(const MexPlan &p, int ph, int pw, const float *input, const float *offsets, float *pooled,
                    void *workspace, size_t workspace_bytes, void *stream, int phase = kMexWhole,
                    float *full = nullptr);
// Similarity, then MEX over its output, then sum pooling; `mp` is the MEX plan for the Similarity output's shape.
// One kernel when the MEX patch of a pixel is exactly the Similarity channels of that pixel (and the MEX + pooling
// pair is fusable), else the separate kernels through scratch memory.
size_t sim_mex_pool_workspace_bytes(const SimPlan &sp, const MexPlan &mp, int ph, int pw);
int sim_mex_pool_launch(const SimPlan &sp, const MexPlan &mp, int ph, int pw, const float *input,
                        const float *templates, const float *weights, const float *offsets, float *pooled,
                        void *workspace, size_t workspace_bytes, void *stream, int phase = kMexWhole);

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

}  // namespace simnets
