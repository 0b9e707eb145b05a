// Launchers of the elementwise kernels (strided copy, fill, binary operators).
#pragma once

#include <hip/hip_runtime.h>

#include "common.hpp"

namespace hpt {

enum { EW_COPY = -1, EW_ADD = HPT_BIN_ADD, EW_SUB = HPT_BIN_SUB, EW_MUL = HPT_BIN_MUL, EW_DIV = HPT_BIN_DIV };

void launch_strided_copy(int dtype, const EwPlan& p, void* out, const void* in, hipStream_t st);
void launch_binary(int op, int dtype, const EwPlan& p, void* out, const void* a, const void* b, hipStream_t st);
// Cast to a float dtype (`p` planned for the wider of the two element sizes).
void launch_cast(int in_dtype, int out_dtype, const EwPlan& p, void* out, const void* in, hipStream_t st);
// `value` points at one element of `dtype` in host memory.
void launch_fill(int dtype, void* out, int64_t n, const void* value, hipStream_t st);

}  // namespace hpt
