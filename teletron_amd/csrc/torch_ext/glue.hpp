// Shared host glue of the torch-facing modules: tensor checks, current stream,
// device guard, workspace from the caching allocator, status -> exception.
#pragma once
#include <torch/extension.h>
#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <map>
#include <mutex>
#include <utility>

#include "teletron_op.h"

namespace tt_glue {

inline void check_act(const torch::Tensor& t, const char* name, int64_t rows, int64_t cols) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  TORCH_CHECK(t.scalar_type() == at::kBFloat16, name, " must be bfloat16, got ", t.scalar_type());
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
  TORCH_CHECK(t.numel() == rows * cols, name, " has ", t.numel(), " elements, expected rows*cols = ", rows * cols);
}
inline void check_param(const torch::Tensor& t, const char* name, int64_t cols, const torch::Tensor& ref) {
  TORCH_CHECK(t.is_cuda() && t.device() == ref.device(), name, " must be on the input's device");
  TORCH_CHECK(t.scalar_type() == at::kBFloat16, name, " must be bfloat16, got ", t.scalar_type());
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
  TORCH_CHECK(t.numel() == cols, name, " has ", t.numel(), " elements, expected cols = ", cols);
}
inline void check_rowstat(const torch::Tensor& t, const char* name, int64_t rows, const torch::Tensor& ref) {
  TORCH_CHECK(t.is_cuda() && t.device() == ref.device(), name, " must be on the input's device");
  TORCH_CHECK(t.scalar_type() == at::kFloat, name, " must be float32, got ", t.scalar_type());
  TORCH_CHECK(t.is_contiguous() && t.numel() == rows, name, " must be contiguous with rows = ", rows, " elements");
}
inline void check_shape(int64_t rows, int64_t cols) {
  TORCH_CHECK(rows >= 0 && cols > 0, "rows must be >= 0 and cols > 0");
}
inline void* current_stream(const torch::Tensor& t) {
  return static_cast<void*>(c10::hip::getCurrentHIPStream(t.device().index()).stream());
}
// Backward workspace (per-workgroup partial sums): one tensor per (device, stream), grown on demand
// and reused from call to call, so a backward call does not go to the allocator (the reference
// allocates its fp32 [32, C] scratch on every call, teletron_op/fused_rmsnorm/weight_backward.cu:229).
// Launches on one stream run in order, so consecutive calls never overlap in it.  A stream under
// graph capture gets memory of its own from the capture's pool: the graph keeps the pointer.
// The cache is never destroyed (the HIP runtime may be gone by the time static destructors run).
inline torch::Tensor workspace(size_t bytes, const torch::Tensor& ref) {
  const auto opts = at::TensorOptions().dtype(at::kByte).device(ref.device());
  const int64_t need = static_cast<int64_t>(bytes < 16 ? 16 : bytes);
  hipStream_t stream = c10::hip::getCurrentHIPStream(ref.device().index()).stream();
  hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) (void)hipGetLastError();
  if (capturing != hipStreamCaptureStatusNone) return at::empty({need}, opts);
  static std::mutex mu;
  static auto* cache = new std::map<std::pair<int, hipStream_t>, torch::Tensor>();
  std::lock_guard<std::mutex> lock(mu);
  torch::Tensor& ws = (*cache)[{static_cast<int>(ref.device().index()), stream}];
  if (!ws.defined() || ws.numel() < need) ws = at::empty({need}, opts);
  return ws;
}
inline void check_status(int rc, const char* what) {
  TORCH_CHECK(rc == TT_OK, what, " failed: ", tt_error_string(rc),
              rc == TT_ERR_HIP ? " (hipError_t " + std::to_string(tt_last_hip_error()) + ")" : std::string());
}

}  // namespace tt_glue
