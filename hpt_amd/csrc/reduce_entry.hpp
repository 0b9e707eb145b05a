// Table of reduction launchers: one entry per op, one slot per dtype. Each
// entry is defined in its own object file (reduce_op.hip compiled once per op)
// so that the ops build in parallel.
#pragma once

#include <hip/hip_runtime.h>

#include "common.hpp"

namespace hpt {

// Library-owned scratch of the reductions that are split over workgroups: the
// partial accumulators the first stage writes and the second stage folds.
struct ReduceScratch {
    void* partial = nullptr;
};

// Bytes of partial-accumulator scratch a plan needs (0: a single stage).
size_t scratch_need(const ReducePlan& p, size_t acc_size);

using ReduceLaunchFn = void (*)(const ReducePlan&, const void* in, void* out,
                                const ReduceScratch&, hipStream_t, int init_out);

struct ReduceEntry {
    ReduceLaunchFn launch[HPT_DTYPE_COUNT];
    size_t acc_size[HPT_DTYPE_COUNT];
};

// OP in [0, HPT_REDUCE_OP_COUNT) are the hpt_reduce_op values; HPT_REDUCE_OP_COUNT
// is argmin and HPT_REDUCE_OP_COUNT + 1 is argmax.
constexpr int kArgMinEntry = HPT_REDUCE_OP_COUNT;
constexpr int kArgMaxEntry = HPT_REDUCE_OP_COUNT + 1;
constexpr int kReduceEntryCount = HPT_REDUCE_OP_COUNT + 2;

template <int OP> const ReduceEntry& reduce_entry();

const ReduceEntry& reduce_entry_for(int op);

}  // namespace hpt
