// Launch table of the normalisation kernels: one object file per kind
// (softmax, log_softmax, layernorm and their fused forms), one launcher per float dtype.
#pragma once

#include <hip/hip_runtime.h>

#include "common.hpp"

namespace hpt {

enum {
    NORM_SOFTMAX = 0,
    NORM_LOGSOFTMAX = 1,
    NORM_LAYERNORM = 2,
    NORM_ADD_LAYERNORM = 3,       // layernorm(in + residual)
    NORM_SOFTMAX_CAUSAL = 4,      // softmax(scale * in) with the causal mask as a parameter
    NORM_LOGSOFTMAX_CAUSAL = 5,
    NORM_KIND_COUNT = 6
};
constexpr bool norm_is_layer(int k) { return k == NORM_LAYERNORM || k == NORM_ADD_LAYERNORM; }
constexpr bool norm_is_log(int k) { return k == NORM_LOGSOFTMAX || k == NORM_LOGSOFTMAX_CAUSAL; }
constexpr bool norm_is_causal(int k) { return k == NORM_SOFTMAX_CAUSAL || k == NORM_LOGSOFTMAX_CAUSAL; }

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
    const void* residual;  // NORM_ADD_LAYERNORM: contiguous tensor of out's shape, added to `in` first
    double scale;          // causal kinds: the input is multiplied by this (and rounded to its dtype) first
    int64_t q_rows;        // causal kinds: rows per attention matrix (size of the dim before the axis)
    int64_t causal_offset; // causal kinds: row q keeps columns 0 .. q + causal_offset
    int tpr, tpr_log2, rpb;
};

using NormLaunchFn = void (*)(const NormPlan&, NormArgs, hipStream_t);

// Launcher for `dtype` (a float dtype) or nullptr. Defined in norm_op.hip,
// compiled once per KIND.
template <int KIND> NormLaunchFn norm_launcher(int dtype);

NormLaunchFn norm_launcher_for(int kind, int dtype);

// Launcher for an INTEGER (or bool) input dtype whose result has the dtype's FloatBinaryType: the
// promotion is fused into the load of the streaming row kernel. Plain kinds only (softmax,
// log_softmax, layernorm); the plan must have been passed through restrict_to_row_stream.
template <int KIND> NormLaunchFn norm_promoting_launcher(int in_dtype);

NormLaunchFn norm_promoting_launcher_for(int kind, int in_dtype);

}  // namespace hpt
