// Parts whose kind the caller registered through the C boundary: every call goes out through a
// table of callbacks with tensors as pointers and shapes.
#pragma once
#include "parts.h"
#include "step.h"

namespace tq {

void register_plugin_kind(const std::string& category, const std::string& kind, const tqe_part_callbacks_t& callbacks, void* user);
tqe_tensor_t to_c(const Tensor& t, int64_t row_stride = 0);
Tensor from_c(const tqe_tensor_t& t);
void fill_step_view(const StepContext& c, tqe_step_view_t& v);

}  // namespace tq
