// Python module `fused_adaln`: the two functions TeleTron's glue exports
// (teletron_op/fused_adaln/adaln_ops.cpp:6-15,29-38,52-65), same names, argument order and
// in-place output convention, backed by the C ABI of libteletron_op.so.  Unlike the
// reference glue, arguments are validated, the launch goes to the current stream of the
// input's device and a failing launch raises.
#include "glue.hpp"

using namespace tt_glue;

void torch_launch_adaln_forward(torch::Tensor& output, torch::Tensor& x_norm, const torch::Tensor& input,
                                const torch::Tensor& scale, const torch::Tensor& shift,
                                int64_t rows, int64_t cols, double epsilon, torch::Tensor& inv_variance) {
  check_shape(rows, cols);
  check_act(input, "input", rows, cols);
  check_act(output, "output", rows, cols);
  check_act(x_norm, "x_norm", rows, cols);
  check_param(scale, "scale", cols, input);
  check_param(shift, "shift", cols, input);
  check_rowstat(inv_variance, "inv_variance", rows, input);
  c10::hip::HIPGuard guard(input.device().index());
  check_status(tt_launch_adaln_forward(output.data_ptr(), x_norm.data_ptr(), input.data_ptr(), scale.data_ptr(),
                                       shift.data_ptr(), rows, cols, epsilon,
                                       static_cast<float*>(inv_variance.data_ptr()), current_stream(input)),
               "torch_launch_adaln_forward");
}

void torch_launch_adaln_backward(torch::Tensor& dinp, torch::Tensor& dscale, torch::Tensor& dshift,
                                 const torch::Tensor& dout, const torch::Tensor& x_norm, const torch::Tensor& scale,
                                 const torch::Tensor& inv_variance, int64_t rows, int64_t cols) {
  check_shape(rows, cols);
  check_act(dout, "dout", rows, cols);
  check_act(x_norm, "x_norm", rows, cols);
  check_act(dinp, "dinp", rows, cols);
  check_param(scale, "scale", cols, dout);
  check_param(dscale, "dscale", cols, dout);
  check_param(dshift, "dshift", cols, dout);
  check_rowstat(inv_variance, "inv_variance", rows, dout);
  c10::hip::HIPGuard guard(dout.device().index());
  const size_t ws_bytes = tt_adaln_backward_workspace_bytes(rows, cols, rows);
  torch::Tensor ws = workspace(ws_bytes, dout);
  check_status(tt_launch_adaln_backward(dinp.data_ptr(), dscale.data_ptr(), dshift.data_ptr(), dout.data_ptr(),
                                        x_norm.data_ptr(), scale.data_ptr(),
                                        static_cast<const float*>(inv_variance.data_ptr()), rows, cols,
                                        ws.data_ptr(), ws_bytes, current_stream(dout)),
               "torch_launch_adaln_backward");
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("torch_launch_adaln_forward", &torch_launch_adaln_forward, "AdaLN forward kernel");
  m.def("torch_launch_adaln_backward", &torch_launch_adaln_backward, "AdaLN backward kernel");
}

TORCH_LIBRARY(layernorm_block_smem, m) {
  m.def("torch_launch_adaln_forward", torch_launch_adaln_forward);
  m.def("torch_launch_adaln_backward", torch_launch_adaln_backward);
}
