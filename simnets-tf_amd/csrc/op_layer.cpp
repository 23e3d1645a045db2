// Compiled operator layer: the caller-side C++ that stands where the reference's op layer stands
// (REGISTER_OP / REGISTER_KERNEL_BUILDER and the Compute wrappers: src/ops/similarity_op.cpp:61-174,
// src/ops/mex_op.cpp:58-170, src/kernels/similarity_kernel_gpu.cu:24-146, src/kernels/mex_kernel_gpu.cu:60-171),
// with torch tensors as device memory.  Host code only: it checks the tensors, fills the attribute structs,
// allocates outputs, keeps one scratch buffer per (device, stream) and calls the C ABI of libsimnets_hip.so.
//
// Two faces over the same functions:
//   * TORCH_LIBRARY(simnets): simnets::similarity, simnets::mex and their four gradient operators, registered with
//     the dispatcher for HIP devices (torch's CUDA key), every attribute explicit as in the reference's op schema;
//     shape inference ("fake" kernels) and the autograd formulas are attached in torch_ops.py;
//   * a Python module (_simnets_native) with the same calls taking the reference's optional keyword attributes
//     (None = the registered default), the fused and prepared forms, and out= arguments: what ops.py forwards to.
//     A call through it costs the host a few microseconds less than building ctypes arguments does, which matters
//     for layers whose kernels run for 4-10 us.
#include <torch/extension.h>
#include <torch/library.h>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/hip/HIPGraphsC10Utils.h>

#include <cstdint>
#include <mutex>
#include <string>
#include <unordered_map>

#include "simnets_hip.h"

namespace py = pybind11;

namespace {

// ---------------------------------------------------------------------------------------------- errors
struct SimnetsStatus : std::exception {
    int code;
    explicit SimnetsStatus(int c) : code(c) {}
    const char *what() const noexcept override { return simnets_hip_strerror(code); }
};
py::object g_error_class;   // ops.SimnetsError, set by ops.py

inline void check(int code)
{
    if (code != 0)
        throw SimnetsStatus(code);
}

// ---------------------------------------------------------------------------------------------- tensors
const at::Tensor &need_f32_hip(const char *name, const at::Tensor &t)
{
    TORCH_CHECK_TYPE(t.scalar_type() == at::kFloat, name, " must be float32 (the HIP path computes in fp32), got ",
                     t.scalar_type());
    TORCH_CHECK(t.is_cuda(), name, " must live on a HIP device: simnets_tf_amd has no CPU fallback");
    return t;
}
inline at::Tensor dense(const char *name, const at::Tensor &t) { return need_f32_hip(name, t).contiguous(); }

struct Shape4 {
    int v[4];
};
inline Shape4 shape4(const at::Tensor &t)
{
    if (t.dim() != 4)
        throw SimnetsStatus(SIMNETS_ERR_SHAPE);
    Shape4 s;
    for (int i = 0; i < 4; ++i) {
        TORCH_CHECK(t.size(i) <= INT32_MAX, "tensor extent beyond 32 bits");
        s.v[i] = (int)t.size(i);
    }
    return s;
}
inline float *ptr(const at::Tensor &t) { return t.data_ptr<float>(); }

// One scratch buffer per (device, stream, capturing): the kernels that use it are ordered on that stream; a buffer
// first allocated during stream capture lives in that graph's private pool and is kept apart from the eager one.
struct WsKey {
    int device;
    void *stream;
    bool capturing;
    bool operator==(const WsKey &o) const { return device == o.device && stream == o.stream && capturing == o.capturing; }
};
struct WsHash {
    size_t operator()(const WsKey &k) const
    {
        return std::hash<void *>()(k.stream) ^ (size_t)(k.device * 2 + (k.capturing ? 1 : 0)) * 0x9e3779b97f4a7c15ULL;
    }
};
std::mutex g_ws_mutex;
std::unordered_map<WsKey, at::Tensor, WsHash> g_workspaces;

struct Launch {
    c10::hip::HIPGuardMasqueradingAsCUDA guard;
    hipStream_t stream;
    int device;
    explicit Launch(const at::Tensor &on) : guard(on.device()), device(on.device().index())
    {
        stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(device).stream();
    }
    // scratch of at least `nbytes` for this call
    std::pair<void *, size_t> workspace(size_t nbytes, const at::Tensor &like)
    {
        const bool capturing = c10::hip::currentStreamCaptureStatusMayInitCtx() != c10::hip::CaptureStatus::None;
        const WsKey key{device, (void *)stream, capturing};
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        at::Tensor &ws = g_workspaces[key];
        if (!ws.defined() || (size_t)ws.numel() < nbytes)
            ws = at::empty({(int64_t)std::max<size_t>(nbytes, (size_t)1 << 20)}, like.options().dtype(at::kByte));
        return {ws.data_ptr(), (size_t)ws.numel()};
    }
};

at::Tensor output_like(const at::Tensor &like, const int (&shape)[4], const c10::optional<at::Tensor> &out)
{
    if (out.has_value() && out->defined()) {
        const at::Tensor &o = *out;
        TORCH_CHECK(o.is_contiguous() && o.scalar_type() == at::kFloat && o.device() == like.device() && o.dim() == 4 &&
                        o.size(0) == shape[0] && o.size(1) == shape[1] && o.size(2) == shape[2] && o.size(3) == shape[3],
                    "out must be a contiguous float32 tensor of shape [", shape[0], ", ", shape[1], ", ", shape[2], ", ",
                    shape[3], "] on ", like.device());
        return o;
    }
    return at::empty({shape[0], shape[1], shape[2], shape[3]}, like.options());
}

// ---------------------------------------------------------------------------------------------- attributes
template <int CAP>
int fill(int (&dst)[CAP], at::IntArrayRef values)
{
    for (size_t i = 0; i < values.size() && i < (size_t)CAP; ++i)
        dst[i] = (int)values[i];
    return (int)values.size();
}

simnets_similarity_attrs sim_attrs(const std::string &function, at::IntArrayRef blocks, at::IntArrayRef strides,
                                   at::IntArrayRef padding, bool normalization_term, double fudge, bool ignore_nan,
                                   double oob, int64_t algo = SIMNETS_ALGO_AUTO, bool every = false)
{
    simnets_similarity_attrs a;
    simnets_similarity_attrs_default(&a);
    a.similarity_function = function == "L1" ? SIMNETS_SIM_L1 : (function == "L2" ? SIMNETS_SIM_L2 : -1);
    a.n_blocks = fill(a.blocks, blocks);
    a.n_strides = fill(a.strides, strides);
    a.n_padding = fill(a.padding, padding);
    a.normalization_term = normalization_term;
    a.normalization_term_fudge = (float)fudge;
    a.ignore_nan_input = ignore_nan;
    a.out_of_bounds_value = (float)oob;
    a.algo = (int)algo;
    a.norm_const_every_iteration = every;
    return a;
}

simnets_mex_attrs mex_attrs(int64_t num_instances, bool softmax_mode, at::IntArrayRef padding, at::IntArrayRef strides,
                            at::IntArrayRef blocks, double epsilon, double oob, bool round_down, bool unshared,
                            at::IntArrayRef shared_region, at::IntArrayRef unshared_region, bool normalize)
{
    simnets_mex_attrs a;
    simnets_mex_attrs_default(&a);
    a.num_instances = (int)num_instances;
    a.softmax_mode = softmax_mode;
    a.n_padding = fill(a.padding, padding);
    a.n_strides = fill(a.strides, strides);
    a.n_blocks = fill(a.blocks, blocks);
    a.epsilon = (float)epsilon;
    a.blocks_out_of_bounds_value = (float)oob;
    a.blocks_round_down = round_down;
    a.use_unshared_regions = unshared;
    a.n_shared = fill(a.shared_offset_region, shared_region);
    a.n_unshared = fill(a.unshared_offset_region, unshared_region);
    a.normalize_offsets = normalize;
    return a;
}

// the reference's keyword attributes as Python objects: None keeps the registered default
template <int CAP>
void fill_opt(const py::object &o, int (&dst)[CAP], int &n)
{
    if (o.is_none())
        return;
    n = 0;
    for (py::handle h : o) {
        if (n < CAP)
            dst[n] = h.cast<int>();
        ++n;
    }
}
simnets_similarity_attrs sim_attrs_py(const py::object &function, const py::object &blocks, const py::object &strides,
                                      const py::object &padding, const py::object &norm, const py::object &fudge,
                                      const py::object &ignore_nan, const py::object &oob, const py::object &algo,
                                      bool every)
{
    simnets_similarity_attrs a;
    simnets_similarity_attrs_default(&a);
    if (!function.is_none()) {
        const std::string f = py::isinstance<py::bytes>(function) ? std::string(py::bytes(function)) : function.cast<std::string>();
        a.similarity_function = f == "L1" ? SIMNETS_SIM_L1 : (f == "L2" ? SIMNETS_SIM_L2 : -1);
    }
    fill_opt(blocks, a.blocks, a.n_blocks);
    fill_opt(strides, a.strides, a.n_strides);
    fill_opt(padding, a.padding, a.n_padding);
    if (!norm.is_none()) a.normalization_term = py::bool_(norm) ? 1 : 0;
    if (!fudge.is_none()) a.normalization_term_fudge = fudge.cast<float>();
    if (!ignore_nan.is_none()) a.ignore_nan_input = py::bool_(ignore_nan) ? 1 : 0;
    if (!oob.is_none()) a.out_of_bounds_value = oob.cast<float>();
    if (!algo.is_none()) {
        if (py::isinstance<py::str>(algo)) {
            const std::string s = algo.cast<std::string>();
            if (s == "auto") a.algo = SIMNETS_ALGO_AUTO;
            else if (s == "direct") a.algo = SIMNETS_ALGO_DIRECT;
            else if (s == "sqrtw") a.algo = SIMNETS_ALGO_SQRTW;
            else if (s == "mfma") a.algo = SIMNETS_ALGO_MFMA;
            else throw py::key_error(s);
        } else {
            a.algo = algo.cast<int>();
        }
    }
    a.norm_const_every_iteration = every;
    return a;
}
simnets_mex_attrs mex_attrs_py(int num_instances, const py::object &softmax, const py::object &padding,
                               const py::object &strides, const py::object &blocks, const py::object &epsilon,
                               const py::object &oob, const py::object &round_down, const py::object &unshared,
                               const py::object &shared_region, const py::object &unshared_region, bool normalize)
{
    simnets_mex_attrs a;
    simnets_mex_attrs_default(&a);
    a.num_instances = num_instances;
    if (!softmax.is_none()) a.softmax_mode = py::bool_(softmax) ? 1 : 0;
    fill_opt(padding, a.padding, a.n_padding);
    fill_opt(strides, a.strides, a.n_strides);
    fill_opt(blocks, a.blocks, a.n_blocks);
    if (!epsilon.is_none()) a.epsilon = epsilon.cast<float>();
    if (!oob.is_none()) a.blocks_out_of_bounds_value = oob.cast<float>();
    if (!round_down.is_none()) a.blocks_round_down = py::bool_(round_down) ? 1 : 0;
    if (!unshared.is_none()) a.use_unshared_regions = py::bool_(unshared) ? 1 : 0;
    fill_opt(shared_region, a.shared_offset_region, a.n_shared);
    fill_opt(unshared_region, a.unshared_offset_region, a.n_unshared);
    a.normalize_offsets = normalize;
    return a;
}

// ---------------------------------------------------------------------------------------------- the calls
at::Tensor similarity_call(const simnets_similarity_attrs &a, const at::Tensor &input, const at::Tensor &templates,
                           const at::Tensor &weights, const c10::optional<at::Tensor> &out)
{
    const at::Tensor x = dense("input", input), t = dense("templates", templates), w = dense("weights", weights);
    const Shape4 xs = shape4(x), ts = shape4(t), ws = shape4(w);
    int os[4];
    check(simnets_similarity_out_shape(&a, xs.v, ts.v, ws.v, os));
    size_t nbytes = 0;
    check(simnets_hip_similarity_workspace_bytes(&a, xs.v, ts.v, &nbytes));
    at::Tensor y = output_like(x, os, out);
    Launch l(x);
    const auto wsp = l.workspace(nbytes, x);
    check(simnets_hip_similarity_fwd(&a, xs.v, ts.v, ws.v, ptr(x), ptr(t), ptr(w), ptr(y), wsp.first, wsp.second, l.stream));
    return y;
}

void sim_grad_setup(const simnets_similarity_attrs &a, const at::Tensor &x, const at::Tensor &t, const at::Tensor &w,
                    const at::Tensor &g, Shape4 &xs, Shape4 &ts, Shape4 &ws)
{
    xs = shape4(x); ts = shape4(t); ws = shape4(w);
    int os[4];
    check(simnets_similarity_out_shape(&a, xs.v, ts.v, ws.v, os));
    if (g.dim() != 4 || g.size(0) != os[0] || g.size(1) != os[1] || g.size(2) != os[2] || g.size(3) != os[3])
        throw SimnetsStatus(SIMNETS_ERR_SHAPE);
}

at::Tensor similarity_input_grad_call(const simnets_similarity_attrs &a, const at::Tensor &input,
                                      const at::Tensor &templates, const at::Tensor &weights, const at::Tensor &grad)
{
    const at::Tensor x = dense("input", input), t = dense("templates", templates), w = dense("weights", weights),
                     g = dense("output_grad", grad);
    Shape4 xs, ts, ws;
    sim_grad_setup(a, x, t, w, g, xs, ts, ws);
    size_t nbytes = 0;
    check(simnets_hip_similarity_grad_workspace_bytes(&a, xs.v, ts.v, &nbytes, nullptr));
    at::Tensor dx = at::empty_like(x);
    Launch l(x);
    const auto wsp = l.workspace(nbytes, x);
    check(simnets_hip_similarity_input_grad(&a, xs.v, ts.v, ws.v, ptr(x), ptr(t), ptr(w), ptr(g), ptr(dx), wsp.first,
                                            wsp.second, l.stream));
    return dx;
}

std::tuple<at::Tensor, at::Tensor> similarity_params_grad_call(const simnets_similarity_attrs &a, const at::Tensor &input,
                                                               const at::Tensor &templates, const at::Tensor &weights,
                                                               const at::Tensor &grad)
{
    const at::Tensor x = dense("input", input), t = dense("templates", templates), w = dense("weights", weights),
                     g = dense("output_grad", grad);
    Shape4 xs, ts, ws;
    sim_grad_setup(a, x, t, w, g, xs, ts, ws);
    size_t nbytes = 0;
    check(simnets_hip_similarity_grad_workspace_bytes(&a, xs.v, ts.v, nullptr, &nbytes));
    at::Tensor dt = at::empty_like(t), dw = at::empty_like(w);
    Launch l(x);
    const auto wsp = l.workspace(nbytes, x);
    check(simnets_hip_similarity_params_grad(&a, xs.v, ts.v, ws.v, ptr(x), ptr(t), ptr(w), ptr(g), ptr(dt), ptr(dw),
                                             wsp.first, wsp.second, l.stream));
    return {dt, dw};
}

at::Tensor mex_call(const simnets_mex_attrs &a, const at::Tensor &input, const at::Tensor &offsets,
                    const c10::optional<at::Tensor> &out)
{
    const at::Tensor x = dense("input", input), off = dense("offsets", offsets);
    const Shape4 xs = shape4(x);
    int os[4];
    check(simnets_mex_out_shape(&a, xs.v, os, nullptr));
    size_t nbytes = 0;
    check(simnets_hip_mex_workspace_bytes(&a, xs.v, &nbytes));
    at::Tensor y = output_like(x, os, out);
    Launch l(x);
    const auto wsp = l.workspace(nbytes, x);
    check(simnets_hip_mex_fwd(&a, xs.v, ptr(x), ptr(off), (size_t)off.numel(), ptr(y), wsp.first, wsp.second, l.stream));
    return y;
}

// the buffer a saving forward call fills for the gradient call (empty when the layer's gradient kernels read none)
at::Tensor saved_buffer(const simnets_mex_attrs &a, const Shape4 &xs, const at::Tensor &like)
{
    size_t nbytes = 0;
    check(simnets_hip_mex_saved_bytes(&a, xs.v, &nbytes));
    return at::empty({(int64_t)nbytes}, like.options().dtype(at::kByte));
}
std::pair<const void *, size_t> saved_arg(const c10::optional<at::Tensor> &saved)
{
    if (!saved.has_value() || !saved->defined() || saved->numel() == 0)
        return {nullptr, 0};
    if (saved->scalar_type() != at::kByte || !saved->is_contiguous() || !saved->is_cuda())
        throw SimnetsStatus(SIMNETS_ERR_SHAPE);
    return {saved->data_ptr(), (size_t)saved->numel()};
}

// ... for training: (output, the offsets as the gradient call reads them)
std::tuple<at::Tensor, at::Tensor> mex_saving_call(const simnets_mex_attrs &a, const at::Tensor &input,
                                                   const at::Tensor &offsets)
{
    const at::Tensor x = dense("input", input), off = dense("offsets", offsets);
    const Shape4 xs = shape4(x);
    int os[4];
    check(simnets_mex_out_shape(&a, xs.v, os, nullptr));
    size_t nbytes = 0;
    check(simnets_hip_mex_workspace_bytes(&a, xs.v, &nbytes));
    at::Tensor y = output_like(x, os, c10::nullopt), saved = saved_buffer(a, xs, x);
    Launch l(x);
    const auto wsp = l.workspace(nbytes, x);
    check(simnets_hip_mex_fwd_saving(&a, xs.v, ptr(x), ptr(off), (size_t)off.numel(), ptr(y),
                                     saved.numel() ? saved.data_ptr() : nullptr, (size_t)saved.numel(), wsp.first,
                                     wsp.second, l.stream));
    return {y, saved};
}

void mex_grad_setup(const simnets_mex_attrs &a, const at::Tensor &x, const at::Tensor &y, const at::Tensor &g, Shape4 &xs)
{
    xs = shape4(x);
    int os[4];
    check(simnets_mex_out_shape(&a, xs.v, os, nullptr));
    for (const at::Tensor *t : {&y, &g})
        if (t->dim() != 4 || t->size(0) != os[0] || t->size(1) != os[1] || t->size(2) != os[2] || t->size(3) != os[3])
            throw SimnetsStatus(SIMNETS_ERR_SHAPE);
}

at::Tensor mex_input_grad_call(const simnets_mex_attrs &a, const at::Tensor &input, const at::Tensor &offsets,
                               const at::Tensor &output, const at::Tensor &grad)
{
    const at::Tensor x = dense("input", input), off = dense("offsets", offsets), y = dense("output", output),
                     g = dense("output_grad", grad);
    Shape4 xs;
    mex_grad_setup(a, x, y, g, xs);
    size_t nbytes = 0;
    check(simnets_hip_mex_grad_workspace_bytes(&a, xs.v, &nbytes, nullptr));
    at::Tensor dx = at::empty_like(x);
    Launch l(x);
    const auto wsp = l.workspace(nbytes, x);
    check(simnets_hip_mex_input_grad(&a, xs.v, ptr(x), ptr(off), (size_t)off.numel(), ptr(y), ptr(g), ptr(dx), wsp.first,
                                     wsp.second, l.stream));
    return dx;
}

at::Tensor mex_offsets_grad_call(const simnets_mex_attrs &a, const at::Tensor &input, const at::Tensor &offsets,
                                 const at::Tensor &output, const at::Tensor &grad)
{
    const at::Tensor x = dense("input", input), off = dense("offsets", offsets), y = dense("output", output),
                     g = dense("output_grad", grad);
    Shape4 xs;
    mex_grad_setup(a, x, y, g, xs);
    size_t nbytes = 0;
    check(simnets_hip_mex_grad_workspace_bytes(&a, xs.v, nullptr, &nbytes));
    at::Tensor doff = at::empty_like(off);
    Launch l(x);
    const auto wsp = l.workspace(nbytes, x);
    check(simnets_hip_mex_offsets_grad(&a, xs.v, ptr(x), ptr(off), (size_t)off.numel(), ptr(y), ptr(g), ptr(doff),
                                       wsp.first, wsp.second, l.stream));
    return doff;
}

std::tuple<at::Tensor, at::Tensor> mex_grads_call(const simnets_mex_attrs &a, const at::Tensor &input,
                                                  const at::Tensor &offsets, const at::Tensor &output,
                                                  const at::Tensor &grad,
                                                  const c10::optional<at::Tensor> &saved = c10::nullopt)
{
    const at::Tensor x = dense("input", input), off = dense("offsets", offsets), y = dense("output", output),
                     g = dense("output_grad", grad);
    Shape4 xs;
    mex_grad_setup(a, x, y, g, xs);
    size_t nbytes = 0;
    check(simnets_hip_mex_grads_workspace_bytes(&a, xs.v, &nbytes));
    at::Tensor dx = at::empty_like(x), doff = at::empty_like(off);
    Launch l(x);
    const auto wsp = l.workspace(nbytes, x);
    const auto sv = saved_arg(saved);
    check(simnets_hip_mex_grads_saved(&a, xs.v, ptr(x), ptr(off), (size_t)off.numel(), ptr(y), ptr(g), sv.first, sv.second,
                                      ptr(dx), ptr(doff), wsp.first, wsp.second, l.stream));
    return {dx, doff};
}

at::Tensor mex_sum_pool_call(const simnets_mex_attrs &a, const at::Tensor &input, const at::Tensor &offsets, int ph,
                             int pw, const c10::optional<at::Tensor> &out)
{
    const at::Tensor x = dense("input", input), off = dense("offsets", offsets);
    const Shape4 xs = shape4(x);
    int os[4];
    check(simnets_mex_out_shape(&a, xs.v, os, nullptr));
    size_t nbytes = 0;
    check(simnets_hip_mex_sum_pool_workspace_bytes(&a, xs.v, ph, pw, &nbytes));
    const int ps[4] = {os[0], os[1], os[2] / ph, os[3] / pw};
    at::Tensor y = output_like(x, ps, out);
    Launch l(x);
    const auto wsp = l.workspace(nbytes, x);
    check(simnets_hip_mex_sum_pool_fwd(&a, xs.v, ptr(x), ptr(off), (size_t)off.numel(), ph, pw, ptr(y), wsp.first,
                                       wsp.second, l.stream));
    return y;
}

// ... for training: (MEX output before pooling, pooled output) from the one call
std::tuple<at::Tensor, at::Tensor> mex_sum_pool_both_call(const simnets_mex_attrs &a, const at::Tensor &input,
                                                          const at::Tensor &offsets, int ph, int pw)
{
    const at::Tensor x = dense("input", input), off = dense("offsets", offsets);
    const Shape4 xs = shape4(x);
    int os[4];
    check(simnets_mex_out_shape(&a, xs.v, os, nullptr));
    size_t nbytes = 0;
    check(simnets_hip_mex_sum_pool_workspace_bytes(&a, xs.v, ph, pw, &nbytes));
    const int ps[4] = {os[0], os[1], os[2] / ph, os[3] / pw};
    at::Tensor full = output_like(x, os, c10::nullopt), y = output_like(x, ps, c10::nullopt);
    Launch l(x);
    const auto wsp = l.workspace(nbytes, x);
    check(simnets_hip_mex_sum_pool_fwd_both(&a, xs.v, ptr(x), ptr(off), (size_t)off.numel(), ph, pw, ptr(full), ptr(y),
                                            wsp.first, wsp.second, l.stream));
    return {full, y};
}

// ... and the offsets as the gradient call reads them
std::tuple<at::Tensor, at::Tensor, at::Tensor> mex_sum_pool_saving_call(const simnets_mex_attrs &a,
                                                                        const at::Tensor &input,
                                                                        const at::Tensor &offsets, int ph, int pw)
{
    const at::Tensor x = dense("input", input), off = dense("offsets", offsets);
    const Shape4 xs = shape4(x);
    int os[4];
    check(simnets_mex_out_shape(&a, xs.v, os, nullptr));
    size_t nbytes = 0;
    check(simnets_hip_mex_sum_pool_workspace_bytes(&a, xs.v, ph, pw, &nbytes));
    const int ps[4] = {os[0], os[1], os[2] / ph, os[3] / pw};
    at::Tensor full = output_like(x, os, c10::nullopt), y = output_like(x, ps, c10::nullopt),
               saved = saved_buffer(a, xs, x);
    Launch l(x);
    const auto wsp = l.workspace(nbytes, x);
    check(simnets_hip_mex_sum_pool_fwd_saving(&a, xs.v, ptr(x), ptr(off), (size_t)off.numel(), ph, pw, ptr(full), ptr(y),
                                              saved.numel() ? saved.data_ptr() : nullptr, (size_t)saved.numel(),
                                              wsp.first, wsp.second, l.stream));
    return {full, y, saved};
}

// the gradients of that pair from the gradient of the pooled output; a gradient that is not wanted is an undefined tensor
std::tuple<at::Tensor, at::Tensor> mex_sum_pool_grads_call(const simnets_mex_attrs &a, const at::Tensor &input,
                                                           const at::Tensor &offsets, const at::Tensor &mex_output,
                                                           const at::Tensor &pooled_grad, int ph, int pw,
                                                           bool want_input, bool want_offsets,
                                                           const c10::optional<at::Tensor> &saved)
{
    const at::Tensor x = dense("input", input), off = dense("offsets", offsets), y = dense("mex_output", mex_output),
                     g = dense("pooled_output_grad", pooled_grad);
    const Shape4 xs = shape4(x);
    int os[4];
    check(simnets_mex_out_shape(&a, xs.v, os, nullptr));
    if (ph <= 0 || pw <= 0)
        throw SimnetsStatus(SIMNETS_ERR_SHAPE);
    const int ps[4] = {os[0], os[1], os[2] / ph, os[3] / pw};
    for (int i = 0; i < 4; ++i)
        if (y.dim() != 4 || g.dim() != 4 || y.size(i) != os[i] || g.size(i) != ps[i])
            throw SimnetsStatus(SIMNETS_ERR_SHAPE);
    if (!want_input && !want_offsets)
        return {at::Tensor(), at::Tensor()};
    size_t nbytes = 0;
    check(simnets_hip_mex_sum_pool_grads_workspace_bytes(&a, xs.v, ph, pw, &nbytes));
    at::Tensor dx = want_input ? at::empty_like(x) : at::Tensor(), doff = want_offsets ? at::empty_like(off) : at::Tensor();
    Launch l(x);
    const auto wsp = l.workspace(nbytes, x);
    const auto sv = saved_arg(saved);
    check(simnets_hip_mex_sum_pool_grads_saved(&a, xs.v, ptr(x), ptr(off), (size_t)off.numel(), ph, pw, ptr(y), ptr(g),
                                               sv.first, sv.second, want_input ? ptr(dx) : nullptr,
                                               want_offsets ? ptr(doff) : nullptr, wsp.first, wsp.second, l.stream));
    return {dx, doff};
}

at::Tensor similarity_mex_sum_pool_call(const simnets_similarity_attrs &sa, const simnets_mex_attrs &ma,
                                        const at::Tensor &input, const at::Tensor &templates, const at::Tensor &weights,
                                        const at::Tensor &offsets, int ph, int pw, const c10::optional<at::Tensor> &out)
{
    const at::Tensor x = dense("input", input), t = dense("templates", templates), w = dense("weights", weights),
                     off = dense("offsets", offsets);
    const Shape4 xs = shape4(x), ts = shape4(t);
    if (w.sizes() != t.sizes())
        throw SimnetsStatus(SIMNETS_ERR_SHAPE);
    int mid[4], os[4];
    check(simnets_similarity_out_shape(&sa, xs.v, ts.v, ts.v, mid));
    check(simnets_mex_out_shape(&ma, mid, os, nullptr));
    size_t nbytes = 0;
    check(simnets_hip_similarity_mex_sum_pool_workspace_bytes(&sa, xs.v, ts.v, &ma, ph, pw, &nbytes));
    const int ps[4] = {os[0], os[1], os[2] / ph, os[3] / pw};
    at::Tensor y = output_like(x, ps, out);
    Launch l(x);
    const auto wsp = l.workspace(nbytes, x);
    check(simnets_hip_similarity_mex_sum_pool_fwd(&sa, xs.v, ts.v, ptr(x), ptr(t), ptr(w), &ma, ptr(off),
                                                  (size_t)off.numel(), ph, pw, ptr(y), wsp.first, wsp.second, l.stream));
    return y;
}

at::Tensor sum_pooling_call(const at::Tensor &input, int ph, int pw, const c10::optional<at::Tensor> &out)
{
    const at::Tensor x = dense("input", input);
    const Shape4 xs = shape4(x);
    const int os[4] = {xs.v[0], xs.v[1], xs.v[2] / std::max(ph, 1), xs.v[3] / std::max(pw, 1)};
    at::Tensor y = output_like(x, os, out);
    Launch l(x);
    check(simnets_hip_sum_pool_fwd(xs.v, ph, pw, ptr(x), ptr(y), l.stream));
    return y;
}

at::Tensor sum_pooling_input_grad_call(const at::Tensor &grad, std::vector<int64_t> input_shape, int ph, int pw)
{
    const at::Tensor g = dense("output_grad", grad);
    TORCH_CHECK(input_shape.size() == 4, "input_shape must have four entries");
    const int xs[4] = {(int)input_shape[0], (int)input_shape[1], (int)input_shape[2], (int)input_shape[3]};
    if (g.dim() != 4 || g.size(0) != xs[0] || g.size(1) != xs[1] || g.size(2) != xs[2] / std::max(ph, 1) ||
        g.size(3) != xs[3] / std::max(pw, 1))
        throw SimnetsStatus(SIMNETS_ERR_SHAPE);
    at::Tensor dx = at::empty({xs[0], xs[1], xs[2], xs[3]}, g.options());
    Launch l(g);
    check(simnets_hip_sum_pool_input_grad(xs, ph, pw, ptr(g), ptr(dx), l.stream));
    return dx;
}

// ---------------------------------------------------------------------------------------------- prepared calls
// A forward operator bound to packed parameters and one input shape (simnets_hip_*_prepare / *_fwd_prepared): the
// buffer is packed at construction, a call runs only the forward kernels on it.  The buffer also holds the kernels'
// per-call scratch, so calls of one object must not overlap (keep them on one stream).
struct Prepared {
    enum Kind { SIM, MEX, MEX_POOL, SIM_MEX_POOL } kind;
    simnets_similarity_attrs sa;
    simnets_mex_attrs ma;
    int xs[4], ts[4], os[4];
    int ph = 1, pw = 1;
    at::Tensor buffer;
    c10::Device device{c10::kCUDA, 0};

    at::Tensor run(const at::Tensor &input, const c10::optional<at::Tensor> &out)
    {
        if (input.dim() != 4 || input.size(0) != xs[0] || input.size(1) != xs[1] || input.size(2) != xs[2] ||
            input.size(3) != xs[3] || input.device() != device || input.scalar_type() != at::kFloat) {
            need_f32_hip("input", input);
            throw SimnetsStatus(SIMNETS_ERR_SHAPE);
        }
        const at::Tensor x = input.is_contiguous() ? input : input.contiguous();
        at::Tensor y = output_like(x, os, out);
        Launch l(x);
        void *buf = buffer.data_ptr();
        const size_t n = (size_t)buffer.numel();
        int rc;
        switch (kind) {
        case SIM: rc = simnets_hip_similarity_fwd_prepared(&sa, xs, ts, ptr(x), buf, n, ptr(y), l.stream); break;
        case MEX: rc = simnets_hip_mex_fwd_prepared(&ma, xs, ptr(x), buf, n, ptr(y), l.stream); break;
        case MEX_POOL: rc = simnets_hip_mex_sum_pool_fwd_prepared(&ma, xs, ptr(x), ph, pw, buf, n, ptr(y), l.stream); break;
        default:
            rc = simnets_hip_similarity_mex_sum_pool_fwd_prepared(&sa, xs, ts, ptr(x), &ma, ph, pw, buf, n, ptr(y), l.stream);
        }
        check(rc);
        return y;
    }
};

void copy4(int (&dst)[4], const std::vector<int64_t> &src)
{
    if (src.size() != 4)
        throw SimnetsStatus(SIMNETS_ERR_SHAPE);
    for (int i = 0; i < 4; ++i)
        dst[i] = (int)src[i];
}
at::Tensor prepared_buffer(const at::Tensor &like, size_t nbytes)
{
    return at::empty({(int64_t)std::max<size_t>(nbytes, 256)}, like.options().dtype(at::kByte));
}

std::shared_ptr<Prepared> similarity_prepare(const simnets_similarity_attrs &a, const std::vector<int64_t> &input_shape,
                                             const at::Tensor &templates, const at::Tensor &weights)
{
    const at::Tensor t = dense("templates", templates), w = dense("weights", weights);
    auto p = std::make_shared<Prepared>();
    p->kind = Prepared::SIM;
    p->sa = a;
    copy4(p->xs, input_shape);
    const Shape4 ts = shape4(t), ws = shape4(w);
    std::copy(ts.v, ts.v + 4, p->ts);
    check(simnets_similarity_out_shape(&a, p->xs, ts.v, ws.v, p->os));
    size_t nbytes = 0;
    check(simnets_hip_similarity_workspace_bytes(&a, p->xs, ts.v, &nbytes));
    p->buffer = prepared_buffer(t, nbytes);
    p->device = t.device();
    Launch l(t);
    check(simnets_hip_similarity_prepare(&a, p->xs, ts.v, ws.v, ptr(t), ptr(w), p->buffer.data_ptr(),
                                         (size_t)p->buffer.numel(), l.stream));
    return p;
}

std::shared_ptr<Prepared> mex_prepare(const simnets_mex_attrs &a, const std::vector<int64_t> &input_shape,
                                      const at::Tensor &offsets, int ph, int pw, bool pool)
{
    const at::Tensor off = dense("offsets", offsets);
    auto p = std::make_shared<Prepared>();
    p->kind = pool ? Prepared::MEX_POOL : Prepared::MEX;
    p->ma = a;
    p->ph = ph; p->pw = pw;
    copy4(p->xs, input_shape);
    check(simnets_mex_out_shape(&a, p->xs, p->os, nullptr));
    size_t nbytes = 0;
    if (pool) {
        check(simnets_hip_mex_sum_pool_workspace_bytes(&a, p->xs, ph, pw, &nbytes));
        p->os[2] /= ph; p->os[3] /= pw;
    } else {
        check(simnets_hip_mex_workspace_bytes(&a, p->xs, &nbytes));
    }
    p->buffer = prepared_buffer(off, nbytes);
    p->device = off.device();
    Launch l(off);
    if (pool)
        check(simnets_hip_mex_sum_pool_prepare(&a, p->xs, ptr(off), (size_t)off.numel(), ph, pw, p->buffer.data_ptr(),
                                               (size_t)p->buffer.numel(), l.stream));
    else
        check(simnets_hip_mex_prepare(&a, p->xs, ptr(off), (size_t)off.numel(), p->buffer.data_ptr(),
                                      (size_t)p->buffer.numel(), l.stream));
    return p;
}

std::shared_ptr<Prepared> similarity_mex_sum_pool_prepare(const simnets_similarity_attrs &sa, const simnets_mex_attrs &ma,
                                                          const std::vector<int64_t> &input_shape,
                                                          const at::Tensor &templates, const at::Tensor &weights,
                                                          const at::Tensor &offsets, int ph, int pw)
{
    const at::Tensor t = dense("templates", templates), w = dense("weights", weights), off = dense("offsets", offsets);
    if (w.sizes() != t.sizes())
        throw SimnetsStatus(SIMNETS_ERR_SHAPE);
    auto p = std::make_shared<Prepared>();
    p->kind = Prepared::SIM_MEX_POOL;
    p->sa = sa; p->ma = ma; p->ph = ph; p->pw = pw;
    copy4(p->xs, input_shape);
    const Shape4 ts = shape4(t);
    std::copy(ts.v, ts.v + 4, p->ts);
    int mid[4];
    check(simnets_similarity_out_shape(&sa, p->xs, ts.v, ts.v, mid));
    check(simnets_mex_out_shape(&ma, mid, p->os, nullptr));
    p->os[2] /= ph; p->os[3] /= pw;
    size_t nbytes = 0;
    check(simnets_hip_similarity_mex_sum_pool_workspace_bytes(&sa, p->xs, ts.v, &ma, ph, pw, &nbytes));
    p->buffer = prepared_buffer(t, nbytes);
    p->device = t.device();
    Launch l(t);
    check(simnets_hip_similarity_mex_sum_pool_prepare(&sa, p->xs, ts.v, ptr(t), ptr(w), &ma, ptr(off), (size_t)off.numel(),
                                                      ph, pw, p->buffer.data_ptr(), (size_t)p->buffer.numel(), l.stream));
    return p;
}

// ---------------------------------------------------------------------------------------------- dispatcher face
[[noreturn]] void rethrow_status(const SimnetsStatus &e)
{
    TORCH_CHECK_VALUE(false, "simnets_hip status ", e.code, ": ", e.what());
}
#define SIMNETS_OP_TRY(expr)      \
    try {                         \
        return expr;              \
    } catch (const SimnetsStatus &e) { \
        rethrow_status(e);        \
    }

at::Tensor op_similarity(const at::Tensor &input, const at::Tensor &templates, const at::Tensor &weights,
                         std::string function, at::IntArrayRef blocks, at::IntArrayRef strides, at::IntArrayRef padding,
                         bool norm, double fudge, bool ignore_nan, double oob)
{
    SIMNETS_OP_TRY(similarity_call(sim_attrs(function, blocks, strides, padding, norm, fudge, ignore_nan, oob), input,
                                   templates, weights, c10::nullopt))
}
at::Tensor op_similarity_input_grad(const at::Tensor &input, const at::Tensor &templates, const at::Tensor &weights,
                                    const at::Tensor &grad, std::string function, at::IntArrayRef blocks,
                                    at::IntArrayRef strides, at::IntArrayRef padding, bool norm, double fudge,
                                    bool ignore_nan, double oob)
{
    SIMNETS_OP_TRY(similarity_input_grad_call(sim_attrs(function, blocks, strides, padding, norm, fudge, ignore_nan, oob),
                                              input, templates, weights, grad))
}
std::tuple<at::Tensor, at::Tensor> op_similarity_parameters_grad(const at::Tensor &input, const at::Tensor &templates,
                                                                 const at::Tensor &weights, const at::Tensor &grad,
                                                                 std::string function, at::IntArrayRef blocks,
                                                                 at::IntArrayRef strides, at::IntArrayRef padding,
                                                                 bool norm, double fudge, bool ignore_nan, double oob)
{
    SIMNETS_OP_TRY(similarity_params_grad_call(sim_attrs(function, blocks, strides, padding, norm, fudge, ignore_nan, oob),
                                               input, templates, weights, grad))
}
at::Tensor op_mex(const at::Tensor &input, const at::Tensor &offsets, int64_t num_instances, bool softmax,
                  at::IntArrayRef padding, at::IntArrayRef strides, at::IntArrayRef blocks, double epsilon, double oob,
                  bool round_down, bool unshared, at::IntArrayRef shared_region, at::IntArrayRef unshared_region,
                  bool normalize)
{
    SIMNETS_OP_TRY(mex_call(mex_attrs(num_instances, softmax, padding, strides, blocks, epsilon, oob, round_down, unshared,
                                      shared_region, unshared_region, normalize),
                            input, offsets, c10::nullopt))
}
at::Tensor op_mex_input_grad(const at::Tensor &input, const at::Tensor &offsets, const at::Tensor &output,
                             const at::Tensor &grad, int64_t num_instances, bool softmax, at::IntArrayRef padding,
                             at::IntArrayRef strides, at::IntArrayRef blocks, double epsilon, double oob, bool round_down,
                             bool unshared, at::IntArrayRef shared_region, at::IntArrayRef unshared_region, bool normalize)
{
    SIMNETS_OP_TRY(mex_input_grad_call(mex_attrs(num_instances, softmax, padding, strides, blocks, epsilon, oob, round_down,
                                                 unshared, shared_region, unshared_region, normalize),
                                       input, offsets, output, grad))
}
at::Tensor op_mex_offsets_grad(const at::Tensor &input, const at::Tensor &offsets, const at::Tensor &output,
                               const at::Tensor &grad, int64_t num_instances, bool softmax, at::IntArrayRef padding,
                               at::IntArrayRef strides, at::IntArrayRef blocks, double epsilon, double oob,
                               bool round_down, bool unshared, at::IntArrayRef shared_region,
                               at::IntArrayRef unshared_region, bool normalize)
{
    SIMNETS_OP_TRY(mex_offsets_grad_call(mex_attrs(num_instances, softmax, padding, strides, blocks, epsilon, oob,
                                                   round_down, unshared, shared_region, unshared_region, normalize),
                                         input, offsets, output, grad))
}

}  // namespace

#define SIMNETS_SIM_SCHEMA                                                                                       \
    "str similarity_function, int[] blocks, int[] strides, int[] padding, bool normalization_term, "            \
    "float normalization_term_fudge, bool ignore_nan_input, float out_of_bounds_value"
#define SIMNETS_MEX_SCHEMA                                                                                       \
    "int num_instances, bool softmax_mode, int[] padding, int[] strides, int[] blocks, float epsilon, "         \
    "float blocks_out_of_bounds_value, bool blocks_round_down, bool use_unshared_regions, "                     \
    "int[] shared_offset_region, int[] unshared_offset_region, bool normalize_offsets"

TORCH_LIBRARY(simnets, m)
{
    m.def("similarity(Tensor input, Tensor templates, Tensor weights, " SIMNETS_SIM_SCHEMA ") -> Tensor");
    m.def("similarity_input_grad(Tensor input, Tensor templates, Tensor weights, Tensor output_grad, " SIMNETS_SIM_SCHEMA
          ") -> Tensor");
    m.def("similarity_parameters_grad(Tensor input, Tensor templates, Tensor weights, Tensor output_grad, "
          SIMNETS_SIM_SCHEMA ") -> (Tensor, Tensor)");
    m.def("mex(Tensor input, Tensor offsets, " SIMNETS_MEX_SCHEMA ") -> Tensor");
    m.def("mex_input_grad(Tensor input, Tensor offsets, Tensor orig_output, Tensor output_grad, " SIMNETS_MEX_SCHEMA
          ") -> Tensor");
    m.def("mex_offsets_grad(Tensor input, Tensor offsets, Tensor orig_output, Tensor output_grad, " SIMNETS_MEX_SCHEMA
          ") -> Tensor");
}

TORCH_LIBRARY_IMPL(simnets, CUDA, m)
{
    m.impl("similarity", &op_similarity);
    m.impl("similarity_input_grad", &op_similarity_input_grad);
    m.impl("similarity_parameters_grad", &op_similarity_parameters_grad);
    m.impl("mex", &op_mex);
    m.impl("mex_input_grad", &op_mex_input_grad);
    m.impl("mex_offsets_grad", &op_mex_offsets_grad);
}

PYBIND11_MODULE(_simnets_native, m)
{
    m.doc() = "compiled operator layer of simnets_tf_amd over the C ABI of libsimnets_hip.so";
    py::register_exception_translator([](std::exception_ptr p) {
        try {
            if (p)
                std::rethrow_exception(p);
        } catch (const SimnetsStatus &e) {
            if (g_error_class) {
                py::object exc = g_error_class(e.code);
                PyErr_SetObject(g_error_class.ptr(), exc.ptr());
            } else {
                PyErr_SetString(PyExc_ValueError, e.what());
            }
        }
    });
    m.def("set_error_class", [](py::object cls) { g_error_class = std::move(cls); });
    m.def("clear_workspaces", [] {
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        g_workspaces.clear();
    });

    using OptT = c10::optional<at::Tensor>;
    m.def("similarity",
          [](const at::Tensor &x, const at::Tensor &t, const at::Tensor &w, py::object function, py::object blocks,
             py::object strides, py::object padding, py::object norm, py::object fudge, py::object ignore_nan,
             py::object oob, py::object algo, bool every, OptT out) {
              return similarity_call(sim_attrs_py(function, blocks, strides, padding, norm, fudge, ignore_nan, oob, algo, every),
                                     x, t, w, out);
          });
    m.def("similarity_input_grad",
          [](const at::Tensor &x, const at::Tensor &t, const at::Tensor &w, const at::Tensor &g, py::object function,
             py::object blocks, py::object strides, py::object padding, py::object norm, py::object fudge,
             py::object ignore_nan, py::object oob, py::object algo) {
              return similarity_input_grad_call(
                  sim_attrs_py(function, blocks, strides, padding, norm, fudge, ignore_nan, oob, algo, false), x, t, w, g);
          });
    m.def("similarity_parameters_grad",
          [](const at::Tensor &x, const at::Tensor &t, const at::Tensor &w, const at::Tensor &g, py::object function,
             py::object blocks, py::object strides, py::object padding, py::object norm, py::object fudge,
             py::object ignore_nan, py::object oob, py::object algo) {
              return similarity_params_grad_call(
                  sim_attrs_py(function, blocks, strides, padding, norm, fudge, ignore_nan, oob, algo, false), x, t, w, g);
          });
    m.def("mex",
          [](const at::Tensor &x, const at::Tensor &off, int n, py::object softmax, py::object padding, py::object strides,
             py::object blocks, py::object epsilon, py::object oob, py::object round_down, py::object unshared,
             py::object shared_region, py::object unshared_region, bool normalize, OptT out) {
              return mex_call(mex_attrs_py(n, softmax, padding, strides, blocks, epsilon, oob, round_down, unshared,
                                           shared_region, unshared_region, normalize),
                              x, off, out);
          });
#define SIMNETS_MEX_GRAD(name, call)                                                                                    \
    m.def(name, [](const at::Tensor &x, const at::Tensor &off, const at::Tensor &y, const at::Tensor &g, int n,           \
                   py::object softmax, py::object padding, py::object strides, py::object blocks, py::object epsilon,     \
                   py::object oob, py::object round_down, py::object unshared, py::object shared_region,                  \
                   py::object unshared_region, bool normalize) {                                                          \
        return call(mex_attrs_py(n, softmax, padding, strides, blocks, epsilon, oob, round_down, unshared, shared_region, \
                                 unshared_region, normalize),                                                             \
                    x, off, y, g);                                                                                        \
    });
    SIMNETS_MEX_GRAD("mex_input_grad", mex_input_grad_call)
    SIMNETS_MEX_GRAD("mex_offsets_grad", mex_offsets_grad_call)
#undef SIMNETS_MEX_GRAD
    m.def("mex_grads", [](const at::Tensor &x, const at::Tensor &off, const at::Tensor &y, const at::Tensor &g, int n,
                          py::object softmax, py::object padding, py::object strides, py::object blocks,
                          py::object epsilon, py::object oob, py::object round_down, py::object unshared,
                          py::object shared_region, py::object unshared_region, bool normalize, OptT saved) {
        return mex_grads_call(mex_attrs_py(n, softmax, padding, strides, blocks, epsilon, oob, round_down, unshared,
                                           shared_region, unshared_region, normalize),
                              x, off, y, g, saved);
    });
    m.def("mex_saving",
          [](const at::Tensor &x, const at::Tensor &off, int n, py::object softmax, py::object padding, py::object strides,
             py::object blocks, py::object epsilon, py::object oob, py::object round_down, py::object unshared,
             py::object shared_region, py::object unshared_region, bool normalize) {
              return mex_saving_call(mex_attrs_py(n, softmax, padding, strides, blocks, epsilon, oob, round_down, unshared,
                                                  shared_region, unshared_region, normalize),
                                     x, off);
          });
    m.def("mex_sum_pool_saving",
          [](const at::Tensor &x, const at::Tensor &off, int n, int ph, int pw, py::object softmax, py::object padding,
             py::object strides, py::object blocks, py::object epsilon, py::object oob, py::object round_down,
             py::object unshared, py::object shared_region, py::object unshared_region, bool normalize) {
              return mex_sum_pool_saving_call(mex_attrs_py(n, softmax, padding, strides, blocks, epsilon, oob, round_down,
                                                           unshared, shared_region, unshared_region, normalize),
                                              x, off, ph, pw);
          });
    m.def("mex_sum_pool",
          [](const at::Tensor &x, const at::Tensor &off, int n, int ph, int pw, py::object softmax, py::object padding,
             py::object strides, py::object blocks, py::object epsilon, py::object oob, py::object round_down,
             py::object unshared, py::object shared_region, py::object unshared_region, bool normalize, OptT out) {
              return mex_sum_pool_call(mex_attrs_py(n, softmax, padding, strides, blocks, epsilon, oob, round_down, unshared,
                                                    shared_region, unshared_region, normalize),
                                       x, off, ph, pw, out);
          });
    m.def("mex_sum_pool_both",
          [](const at::Tensor &x, const at::Tensor &off, int n, int ph, int pw, py::object softmax, py::object padding,
             py::object strides, py::object blocks, py::object epsilon, py::object oob, py::object round_down,
             py::object unshared, py::object shared_region, py::object unshared_region, bool normalize) {
              return mex_sum_pool_both_call(mex_attrs_py(n, softmax, padding, strides, blocks, epsilon, oob, round_down,
                                                         unshared, shared_region, unshared_region, normalize),
                                            x, off, ph, pw);
          });
    m.def("mex_sum_pool_grads",
          [](const at::Tensor &x, const at::Tensor &off, const at::Tensor &full, const at::Tensor &g, int n, int ph, int pw,
             bool want_input, bool want_offsets, py::object softmax, py::object padding, py::object strides,
             py::object blocks, py::object epsilon, py::object oob, py::object round_down, py::object unshared,
             py::object shared_region, py::object unshared_region, bool normalize, OptT saved) {
              return mex_sum_pool_grads_call(mex_attrs_py(n, softmax, padding, strides, blocks, epsilon, oob, round_down,
                                                          unshared, shared_region, unshared_region, normalize),
                                             x, off, full, g, ph, pw, want_input, want_offsets, saved);
          });
    // the attribute structs of the two-operator calls come from Python as dicts of keyword arguments
    auto sim_from_dict = [](const py::dict &d) {
        auto get = [&](const char *k) -> py::object { return d.contains(k) ? py::object(d[k]) : py::none(); };
        const py::object every = get("norm_const_every_iteration");
        return sim_attrs_py(get("similarity_function"), get("blocks"), get("strides"), get("padding"),
                            get("normalization_term"), get("normalization_term_fudge"), get("ignore_nan_input"),
                            get("out_of_bounds_value"), get("algo"), !every.is_none() && py::bool_(every));
    };
    auto mex_from_dict = [](int n, const py::dict &d) {
        auto get = [&](const char *k) -> py::object { return d.contains(k) ? py::object(d[k]) : py::none(); };
        const py::object normalize = get("normalize_offsets");
        return mex_attrs_py(n, get("softmax_mode"), get("padding"), get("strides"), get("blocks"), get("epsilon"),
                            get("blocks_out_of_bounds_value"), get("blocks_round_down"), get("use_unshared_regions"),
                            get("shared_offset_region"), get("unshared_offset_region"),
                            !normalize.is_none() && py::bool_(normalize));
    };
    m.def("similarity_mex_sum_pool",
          [sim_from_dict, mex_from_dict](const at::Tensor &x, const at::Tensor &t, const at::Tensor &w, const at::Tensor &off,
                                         int n, int ph, int pw, py::dict similarity, py::dict mex, OptT out) {
              return similarity_mex_sum_pool_call(sim_from_dict(similarity), mex_from_dict(n, mex), x, t, w, off, ph, pw, out);
          });
    m.def("sum_pooling", &sum_pooling_call);
    m.def("sum_pooling_input_grad", &sum_pooling_input_grad_call);

    py::class_<Prepared, std::shared_ptr<Prepared>>(
        m, "Prepared",
        "A forward operator bound to packed parameters and one input shape; call it with the input\n"
        "(`prepared(input, out=None)`).\n\n"
        "Made by `similarity_prepare`, `mex_prepare`, `mex_sum_pool_prepare` or `similarity_mex_sum_pool_prepare`.  The\n"
        "results are those of the plain call, bit for bit.  The buffer (`.buffer`) also serves as the per-call scratch of\n"
        "the kernels, so calls of one object must not overlap (keep them on one stream).  Later changes of the parameter\n"
        "tensors are not seen: prepare again.")
        .def("__call__", &Prepared::run, py::arg("input"), py::arg("out") = py::none())
        .def_property_readonly("buffer", [](const Prepared &p) { return p.buffer; })
        .def_property_readonly("input_shape", [](const Prepared &p) { return py::make_tuple(p.xs[0], p.xs[1], p.xs[2], p.xs[3]); })
        .def_property_readonly("output_shape", [](const Prepared &p) { return py::make_tuple(p.os[0], p.os[1], p.os[2], p.os[3]); });
    m.def("similarity_prepare", [sim_from_dict](std::vector<int64_t> input_shape, const at::Tensor &t, const at::Tensor &w,
                                                py::dict attrs) {
        return similarity_prepare(sim_from_dict(attrs), input_shape, t, w);
    });
    m.def("mex_prepare", [mex_from_dict](std::vector<int64_t> input_shape, const at::Tensor &off, int n, py::dict attrs) {
        return mex_prepare(mex_from_dict(n, attrs), input_shape, off, 1, 1, false);
    });
    m.def("mex_sum_pool_prepare",
          [mex_from_dict](std::vector<int64_t> input_shape, const at::Tensor &off, int n, int ph, int pw, py::dict attrs) {
              return mex_prepare(mex_from_dict(n, attrs), input_shape, off, ph, pw, true);
          });
    m.def("similarity_mex_sum_pool_prepare",
          [sim_from_dict, mex_from_dict](std::vector<int64_t> input_shape, const at::Tensor &t, const at::Tensor &w,
                                         const at::Tensor &off, int n, int ph, int pw, py::dict similarity, py::dict mex) {
              return similarity_mex_sum_pool_prepare(sim_from_dict(similarity), mex_from_dict(n, mex), input_shape, t, w, off,
                                                     ph, pw);
          });
}
