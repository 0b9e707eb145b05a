// Launch table of the normalisation kernels: one object file per kind
// (softmax, log_softmax, layernorm), one launcher per float dtype.
#pragma once

#include <hip/hip_runtime.h>

#include "common.hpp"

namespace hpt {

enum { NORM_SOFTMAX = 0, NORM_LOGSOFTMAX = 1, NORM_LAYERNORM = 2 };

struct NormArgs {
    const void* in;
    void* out;
    const void* gamma;
    const void* beta;
    Dims kept_in;   // row index -> input offset
    Dims kept_out;  // row index -> output offset
    Dims norm_in;   // position in the row -> input offset
    int64_t rows, cols;
    int64_t sa;               // input stride along the row when norm_in.n == 1
    int64_t out_axis_stride;  // output stride along the row
    double eps;
    double inv_cols;  // 1 / cols
    void* scratch;    // library-owned scratch (partial row statistics of the transposed form)
    int tpr, tpr_log2, rpb;
};

using NormLaunchFn = void (*)(const NormPlan&, NormArgs, hipStream_t);

// Launcher for `dtype` (a float dtype) or nullptr. Defined in norm_op.hip,
// compiled once per KIND.
template <int KIND> NormLaunchFn norm_launcher(int dtype);

NormLaunchFn norm_launcher_for(int kind, int dtype);

}  // namespace hpt
