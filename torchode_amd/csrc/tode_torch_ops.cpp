// torch.ops.torchode_amd.*: the whole-solve entry point of the C ABI as an operator of PyTorch's dispatcher, so that a
// program captured by torch.compile holds the solve as one node (the reference's loop, adjoints.py:42-311, is a
// data-dependent Python while loop that a tracing compiler cannot capture).  This file holds no kernel and no solver
// logic: it turns tensors into the pointers of tode_solve_args, allocates the outputs and the workspace with PyTorch's
// allocator, and calls tode_solve_builtin_auto on PyTorch's current stream.
#include <ATen/ATen.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/library.h>

#include <tuple>

#include "../../include/torchode_amd.h"

namespace {

using at::Tensor;
using OptTensor = std::optional<Tensor>;

const void *data_or_null(const OptTensor &t) { return t.has_value() && t->defined() && t->numel() > 0 ? t->data_ptr() : nullptr; }

void same_device(const Tensor &like, const OptTensor &t, const char *name) {
    TORCH_CHECK(!t.has_value() || !t->defined() || t->device() == like.device(), "torchode_amd::solve_builtin: ", name, " is on ", t->device(),
                ", y0 on ", like.device());
}

// Returns (ys [B, max(E, 1), F], n_steps, n_accepted, n_initialized, status [B] int64, iterations: int64 scalar on the
// CPU).  `control` = (atol, rtol, pcoeff, icoeff, dcoeff, safety, factor_min, factor_max, dt_min, dt_max) with NaN for
// a limit that is not set, in the order of struct tode_controller.
std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor, Tensor> solve_builtin(const Tensor &y0, const Tensor &t_start, const Tensor &t_end,
                                                                         const OptTensor &t_eval, const OptTensor &dt0, const OptTensor &params,
                                                                         const OptTensor &shared_params, int64_t method, int64_t term,
                                                                         c10::ArrayRef<double> term_scalars, int64_t controller_kind,
                                                                         c10::ArrayRef<double> control, int64_t max_steps, bool allow_one_kernel) {
    TORCH_CHECK(y0.is_cuda(), "torchode_amd::solve_builtin runs on the GPU only (y0 is on ", y0.device(), ")");
    TORCH_CHECK(y0.dim() == 2, "y0 must be [batch, features]");
    TORCH_CHECK(y0.scalar_type() == at::kFloat || y0.scalar_type() == at::kDouble, "y0 must be float32 or float64");
    TORCH_CHECK(control.size() == 10, "control holds 10 values, got ", control.size());
    TORCH_CHECK(term_scalars.size() <= 4, "at most 4 term scalars");
    const auto dtype = y0.scalar_type(), time_dtype = t_start.scalar_type();  // (they may differ: reference problems.py:44-56)
    TORCH_CHECK(time_dtype == at::kFloat || time_dtype == at::kDouble, "times must be float32 or float64");
    const int64_t B = y0.size(0), F = y0.size(1);
    const bool has_eval = t_eval.has_value() && t_eval->defined();
    const int64_t E = has_eval ? t_eval->size(1) : 0;
    for (const Tensor *t : {&t_start, &t_end}) {
        TORCH_CHECK(t->dim() == 1 && t->size(0) == B && t->scalar_type() == time_dtype && t->device() == y0.device(),
                    "t_start / t_end must be [batch], of one dtype, on y0's device");
        TORCH_CHECK(B == 0 || t->stride(0) >= 1, "t_start / t_end must not be expanded views");
    }
    same_device(y0, t_eval, "t_eval"), same_device(y0, dt0, "dt0"), same_device(y0, params, "params"), same_device(y0, shared_params, "shared_params");
    TORCH_CHECK(!has_eval || (t_eval->dim() == 2 && t_eval->size(0) == B && t_eval->scalar_type() == time_dtype), "t_eval must be [batch, points] in t_start's dtype");

    const Tensor y0_c = y0.contiguous();
    const OptTensor t_eval_c = has_eval ? OptTensor(t_eval->contiguous()) : OptTensor();
    const OptTensor dt0_c = dt0.has_value() && dt0->defined() ? OptTensor(dt0->to(time_dtype).contiguous()) : OptTensor();
    const OptTensor params_c = params.has_value() && params->defined() ? OptTensor(params->to(dtype).contiguous()) : OptTensor();
    const OptTensor shared_c = shared_params.has_value() && shared_params->defined() ? OptTensor(shared_params->contiguous()) : OptTensor();
    TORCH_CHECK(!dt0_c.has_value() || (dt0_c->dim() == 1 && dt0_c->size(0) == B), "dt0 must be [batch]");
    TORCH_CHECK(!params_c.has_value() || (params_c->dim() == 2 && params_c->size(0) == B), "params must be [batch, parameters per sample]");
    TORCH_CHECK(!shared_c.has_value() || shared_c->scalar_type() == dtype, "shared_params must be in y0's dtype");

    tode_solve_args a = {};
    const int data_code = dtype == at::kFloat ? TODE_F32 : TODE_F64, time_code = time_dtype == at::kFloat ? TODE_F32 : TODE_F64;
    a.dtype = data_code == time_code ? data_code : TODE_DTYPES(data_code, time_code);
    a.method = (int32_t)method, a.term = (int32_t)term;
    a.n_features = (int32_t)F, a.n_eval = (int32_t)E, a.n_params = params_c.has_value() ? (int32_t)params_c->size(1) : 0;
    a.batch = B, a.max_steps = max_steps, a.iteration_cap = -1;
    for (size_t i = 0; i < term_scalars.size(); ++i) a.term_scalars[i] = term_scalars[i];
    a.y0 = y0_c.data_ptr();
    a.t_start = t_start.data_ptr(), a.t_end = t_end.data_ptr();
    a.t_start_stride = B > 0 ? t_start.stride(0) : 1, a.t_end_stride = B > 0 ? t_end.stride(0) : 1;
    a.t_eval = data_or_null(t_eval_c), a.dt0 = dt0_c.has_value() ? dt0_c->data_ptr() : nullptr;
    a.params = data_or_null(params_c);
    a.shared_params = data_or_null(shared_c), a.n_shared_params = shared_c.has_value() ? shared_c->numel() : 0;

    tode_controller c = {};
    c.kind = (int32_t)controller_kind;
    c.atol = control[0], c.rtol = control[1], c.pcoeff = control[2], c.icoeff = control[3], c.dcoeff = control[4];
    c.safety = control[5], c.factor_min = control[6], c.factor_max = control[7];
    c.has_dt_min = control[8] == control[8], c.has_dt_max = control[9] == control[9];
    c.dt_min = c.has_dt_min ? control[8] : 0.0, c.dt_max = c.has_dt_max ? control[9] : 0.0;

    const c10::DeviceGuard guard(y0.device());  // (the generic guard: this build of PyTorch names the GPU's device type "cuda")
    Tensor ys = at::empty({B, E > 0 ? E : 1, F}, y0.options());
    // (four tensors, not four rows of one: an operator's results must not share memory unless its schema says so)
    Tensor n_steps = at::empty({B}, y0.options().dtype(at::kLong)), n_accepted = at::empty_like(n_steps), n_initialized = at::empty_like(n_steps),
           status = at::empty_like(n_steps);
    a.ys = ys.data_ptr();
    const int64_t need = tode_solve_workspace_bytes(&a);
    TORCH_CHECK(need >= 0, "torchode_amd::solve_builtin: bad problem sizes");
    Tensor workspace = at::empty({need}, y0.options().dtype(at::kByte));
    int64_t iterations = 0;
    const int rc = tode_solve_builtin_auto(&a, &c, n_steps.data_ptr<int64_t>(), n_accepted.data_ptr<int64_t>(), n_initialized.data_ptr<int64_t>(),
                                           status.data_ptr<int64_t>(), workspace.data_ptr(), need, allow_one_kernel ? 1 : 0,
                                           (void *)c10::hip::getCurrentHIPStream(y0.device().index()).stream(), &iterations);
    TORCH_CHECK(rc == TODE_OK, "torchode_amd::solve_builtin: ", tode_last_error(), " (code ", rc, ")");
    return {ys, n_steps, n_accepted, n_initialized, status, at::scalar_tensor(iterations, at::TensorOptions().dtype(at::kLong))};
}

// tode_mlp_pack_weights_for: W1 | b1 | W2 | b2 concatenated -> the order the MLP kernel loads them in.
Tensor mlp_pack_weights(const Tensor &raw, int64_t matrix_inputs, int64_t n_features) {
    TORCH_CHECK(raw.is_cuda() && raw.scalar_type() == at::kFloat && raw.dim() == 1, "torchode_amd::mlp_pack_weights takes a float32 vector on the GPU");
    TORCH_CHECK(matrix_inputs == TODE_MLP_INPUTS_F32 || matrix_inputs == TODE_MLP_INPUTS_BF16, "unknown matrix input kind ", matrix_inputs);
    const Tensor raw_c = raw.contiguous();
    const c10::DeviceGuard guard(raw.device());
    Tensor packed = at::empty({matrix_inputs == TODE_MLP_INPUTS_BF16 ? TODE_MLP_PACKED_SIZE_BF16 : TODE_MLP_PACKED_SIZE}, raw.options());
    const int rc = tode_mlp_pack_weights_for(raw_c.data_ptr(), raw_c.numel(), (int32_t)n_features, (int32_t)matrix_inputs, packed.data_ptr(),
                                             (void *)c10::hip::getCurrentHIPStream(raw.device().index()).stream());
    TORCH_CHECK(rc == TODE_OK, "torchode_amd::mlp_pack_weights: ", tode_last_error(), " (code ", rc, ")");
    return packed;
}

}  // namespace

TORCH_LIBRARY(torchode_amd, m) {
    m.def("mlp_pack_weights(Tensor raw, int matrix_inputs, int n_features=64) -> Tensor");
    m.def(
        "solve_builtin(Tensor y0, Tensor t_start, Tensor t_end, Tensor? t_eval, Tensor? dt0, Tensor? params, Tensor? shared_params, int method, int term, "
        "float[] term_scalars, int controller_kind, float[] control, int max_steps, bool allow_one_kernel) -> (Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)");
}

TORCH_LIBRARY_IMPL(torchode_amd, CUDA, m) {
    m.impl("solve_builtin", &solve_builtin);
    m.impl("mlp_pack_weights", &mlp_pack_weights);
}
