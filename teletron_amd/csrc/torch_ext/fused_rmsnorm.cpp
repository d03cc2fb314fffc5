// Python module `fused_rmsnorm`: the two functions TeleTron's glue exports
// (teletron_op/fused_rmsnorm/rms_ops.cpp:6-13,25-33,47-61), same names, argument order and
// in-place output convention, backed by the C ABI of libteletron_op.so.
#include "glue.hpp"

using namespace tt_glue;

void torch_launch_rms_forward(torch::Tensor& output, const torch::Tensor& input, const torch::Tensor& weight,
                              int64_t rows, int64_t cols, double epsilon, torch::Tensor& inv_variance) {
  check_shape(rows, cols);
  check_act(input, "input", rows, cols);
  check_act(output, "output", rows, cols);
  check_param(weight, "weight", cols, input);
  check_rowstat(inv_variance, "inv_variance", rows, input);
  c10::hip::HIPGuard guard(input.device().index());
  check_status(tt_launch_rms_forward(output.data_ptr(), input.data_ptr(), weight.data_ptr(), rows, cols, epsilon,
                                     static_cast<float*>(inv_variance.data_ptr()), current_stream(input)),
               "torch_launch_rms_forward");
}

void torch_launch_rms_backward(torch::Tensor& dinp, torch::Tensor& dweight, const torch::Tensor& dout,
                               const torch::Tensor& x_norm, const torch::Tensor& weight,
                               const torch::Tensor& inv_variance, int64_t rows, int64_t cols) {
  check_shape(rows, cols);
  check_act(dout, "dout", rows, cols);
  check_act(x_norm, "x_norm", rows, cols);
  check_act(dinp, "dinp", rows, cols);
  check_param(weight, "weight", cols, dout);
  check_param(dweight, "dweight", cols, dout);
  check_rowstat(inv_variance, "inv_variance", rows, dout);
  c10::hip::HIPGuard guard(dout.device().index());
  const size_t ws_bytes = tt_rmsnorm_backward_workspace_bytes(rows, cols);
  torch::Tensor ws = workspace(ws_bytes, dout);
  check_status(tt_launch_rms_backward(dinp.data_ptr(), dweight.data_ptr(), dout.data_ptr(), x_norm.data_ptr(),
                                      weight.data_ptr(), static_cast<const float*>(inv_variance.data_ptr()),
                                      rows, cols, ws.data_ptr(), ws_bytes, current_stream(dout)),
               "torch_launch_rms_backward");
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("torch_launch_rms_forward", &torch_launch_rms_forward, "RMSNorm forward kernel");
  m.def("torch_launch_rms_backward", &torch_launch_rms_backward, "RMSNorm backward kernel");
}

TORCH_LIBRARY(Fused_RMSNorm, m) {
  m.def("torch_launch_rms_forward", torch_launch_rms_forward);
  m.def("torch_launch_rms_backward", torch_launch_rms_backward);
}
