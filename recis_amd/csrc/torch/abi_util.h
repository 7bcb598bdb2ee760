// Helpers shared by the torch-facing translation units: everything between a torch::Tensor and
// the plain pointers + sizes that librecis_hip.so takes (include/recis_hip.h).
#pragma once

#include <ATen/ATen.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <c10/util/Exception.h>

#include <string>
#include <vector>

#include "recis_hip.h"

namespace recis {
namespace hipabi {

// A failed call of the C ABI becomes a c10::Error (a Python RuntimeError), like the reference's
// TORCH_CHECKs (csrc/embedding/hashtable.cc:84-85).
inline void check(int rc) {
  TORCH_CHECK(rc == RECIS_OK, "librecis_hip: ", recis_hip_last_error(), " (code ", rc, ")");
}

// The stream the reference's kernels use: the current one of the tensor's device
// (at::cuda::getCurrentCUDAStream in csrc/ops/*_kernel.cu).
inline void* stream_of(const at::Device& device) {
  return c10::hip::getCurrentHIPStream(device.index()).stream();
}

inline void require_gpu(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor in this build (there is no CPU path), got ",
              t.device());
}

inline void require_gpu(const std::vector<at::Tensor>& ts, const char* name) {
  for (const auto& t : ts) require_gpu(t, name);
}

inline int dtype_code(at::ScalarType t) {
  switch (t) {
    case at::kFloat: return RECIS_F32;
    case at::kBFloat16: return RECIS_BF16;
    case at::kHalf: return RECIS_F16;
    default: TORCH_CHECK(false, "unsupported row dtype ", t, " (float32, bfloat16, float16)");
  }
}

// 1 for int64, 0 for int32.
inline int index_kind(const at::Tensor& t, const char* name) {
  if (t.scalar_type() == at::kLong) return 1;
  TORCH_CHECK(t.scalar_type() == at::kInt, name, " must be int32 or int64, got ", t.scalar_type());
  return 0;
}

inline at::Tensor flat_i64(const at::Tensor& t, const char* name) {
  require_gpu(t, name);
  TORCH_CHECK(t.scalar_type() == at::kLong, name, " must be int64, got ", t.scalar_type());
  return t.contiguous().view({-1});
}

inline int64_t row_bytes(const at::Tensor& block) {
  int64_t n = block.element_size();
  for (int64_t d = 1; d < block.dim(); ++d) n *= block.size(d);
  return n;
}

// Every row of the block is contiguous and rows do not overlap; rows may lie a pitch apart (a slot
// that shares its allocation with the optimizer state of the same keys).
inline bool rows_dense(const at::Tensor& block) {
  if (block.is_contiguous()) return true;
  if (block.dim() < 1) return false;
  int64_t row = 1;
  for (int64_t d = block.dim() - 1; d >= 1; --d) {
    if (block.size(d) != 1 && block.stride(d) != row) return false;
    row *= block.size(d);
  }
  return block.stride(0) >= row;
}

// Checks a block list (one dtype, one row shape, contiguous rows at one pitch, at least block_size
// rows each) and returns its first block.
const at::Tensor& check_blocks(const std::vector<at::Tensor>& blocks, int64_t block_size);

// The row_pitch_bytes argument of the C header for a block: 0 when its rows lie back to back.
int64_t row_pitch_bytes(const at::Tensor& block);
// The same for slots that go into one call (their first blocks): they must agree.
int64_t shared_row_pitch_bytes(std::initializer_list<const at::Tensor*> first_blocks);

// Device array holding the base pointer of every block, as the row kernels take it. Cached on the
// pointer values, so a slot that does not grow pays the host-to-device copy once, not per launch
// (the reference builds and uploads the table on every launch, csrc/cuda/cuda_param.cuh:20-60).
at::Tensor block_ptr_table(const std::vector<at::Tensor>& blocks);

template <typename T>
std::vector<const T*> host_ptrs(const std::vector<at::Tensor>& ts) {
  std::vector<const T*> out(ts.size());
  for (size_t i = 0; i < ts.size(); ++i) out[i] = static_cast<const T*>(ts[i].data_ptr());
  return out;
}

template <typename T>
std::vector<T*> host_mut_ptrs(const std::vector<at::Tensor>& ts) {
  std::vector<T*> out(ts.size());
  for (size_t i = 0; i < ts.size(); ++i) out[i] = static_cast<T*>(ts[i].data_ptr());
  return out;
}

inline std::vector<int64_t> numels(const std::vector<at::Tensor>& ts) {
  std::vector<int64_t> out(ts.size());
  for (size_t i = 0; i < ts.size(); ++i) out[i] = ts[i].numel();
  return out;
}

// A 1-D integer tensor on any device as host values.
std::vector<int64_t> host_values(const at::Tensor& t);

inline const void* opt_ptr(const c10::optional<at::Tensor>& t) {
  return t.has_value() && t->defined() ? t->data_ptr() : nullptr;
}

}  // namespace hipabi
}  // namespace recis
