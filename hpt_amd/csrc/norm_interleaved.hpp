// Softmax over rows that are contiguous [cols / L, L] slabs (NormPlan::interleave): the instantiations of
// row_reg_kernel for them are many and are compiled in a translation unit of their own, once per kind.
#pragma once
#include <hip/hip_runtime.h>

#include "common.hpp"

namespace hpt {

struct NormArgs;

// Launch the plan `p` (kind RowReg, interleave != 1) for element type T. KIND is NORM_SOFTMAX or NORM_LOGSOFTMAX.
template <int KIND, class T>
void launch_interleaved_rows(const NormPlan& p, const NormArgs& a, dim3 grid, dim3 block, hipStream_t st);

}  // namespace hpt
