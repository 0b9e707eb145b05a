// Shared host-side declarations of libhpt_hip: error transport, coalesced
// dimension lists, and the plans the host logic hands to the kernel launchers.
#pragma once

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "hpt_hip.h"

namespace hpt {

constexpr int kMaxDims = 8;   // coalesced dims per group (kept / reduced) a kernel can walk
constexpr int kMaxRank = 32;  // rank of a view accepted at the ABI

// Thrown by host logic and launchers; the C ABI wrappers turn it into a status
// code plus the thread-local message.
struct Error {
    int code;
    std::string msg;
};

[[noreturn]] inline void fail(int code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    throw Error{code, buf};
}

// A list of (size, stride) pairs, outermost first. Strides are in elements of
// the view they came from and may be negative (reversed slices) or zero.
struct Dims {
    int n = 0;
    int64_t size[kMaxDims] = {};
    int64_t stride[kMaxDims] = {};
    int64_t count() const {
        int64_t c = 1;
        for (int i = 0; i < n; ++i) c *= size[i];
        return c;
    }
};

inline size_t dtype_size(int dt) {
    switch (dt) {
        case HPT_BOOL: case HPT_I8: case HPT_U8: return 1;
        case HPT_I16: case HPT_U16: case HPT_F16: case HPT_BF16: return 2;
        case HPT_I32: case HPT_U32: case HPT_F32: return 4;
        case HPT_I64: case HPT_U64: case HPT_F64: return 8;
        default: return 0;
    }
}

inline const char* dtype_name(int dt) {
    static const char* names[] = {"bool", "i8", "i16", "i32", "i64", "u8", "u16",
                                  "u32", "u64", "f16", "bf16", "f32", "f64"};
    return (dt >= 0 && dt < HPT_DTYPE_COUNT) ? names[dt] : "?";
}

inline bool is_float_dtype(int dt) {
    return dt == HPT_F16 || dt == HPT_BF16 || dt == HPT_F32 || dt == HPT_F64;
}

// ---- host shape logic (layout.cpp) ---------------------------------------

// process_axes of the reference: wrap negatives, reject out-of-range and
// duplicates. Returns normalised axes in the caller's order.
void process_axes(const int64_t* axes, int naxes, int ndim, int64_t* out);

// Output dtype of reduce op `op` on input dtype `in`.
int reduce_out_dtype(int op, int in);

enum class ReduceKind {
    Empty,     // no output elements: nothing to launch
    Identity,  // outputs exist but nothing is reduced into them (a reduced dim has size 0)
    Row,       // lanes walk the reduced index space (the reduced group owns the smallest stride)
    Col        // lanes walk the outputs (a kept dim owns the smallest stride)
};

struct ReducePlan {
    ReduceKind kind = ReduceKind::Empty;
    int64_t K = 0;  // number of outputs
    int64_t R = 0;  // number of elements reduced into each output
    Dims kept;      // kept dims, logical order, coalesced
    Dims red;       // reduced dims, sorted by |stride| descending, coalesced
    // launch shape
    int vec = 1;     // elements per vector load
    int tpr = 1;     // Row: threads cooperating on one output (power of two)
    int rpb = 1;     // Row: outputs per block
    int bx = 1;      // Col: lanes along the outputs
    int by = 1;      // Col: thread rows that split the reduced range inside a block
    int split = 1;   // blocks that share one output (second stage combines them)
    int split_q = 1; // Row: how `split` divides the outer reduced dims ...
    int split_i = 1; // ... and the innermost reduced dim (split = split_q * split_i)
    int64_t chunk = 0;  // Col: reduced indices per split
    int sstride = 1;    // lean kernels: 2 = elements along the lane dim sit at every second position
    bool lean = false;  // the layout fits the lean kernels (one reduced dim, <= 2 kept dims, 32-bit extents)
    bool ragged = false;        // Row (lean): rows of any length and alignment; aligned 128-bit loads over the body, the two ends element-wise
    bool unaligned = false;     // Col (lean): rows are not whole / aligned vectors; lanes still take VEC neighbours with unaligned 128-bit loads. Row: runs off the 16-byte grid read with unaligned 128-bit loads
    bool kept_swapped = false;  // Col (lean): the two kept dims are listed inner-most-in-memory last, not in output order
    int mod_rows = 0;   // Row, > 0: a row is a contiguous [R, mod_rows] slab with mod_rows = 3, 5, 6 or 7 (no divisor of the vector) reduced over its first dim: threads in multiples of mod_rows keep an accumulator per vector place, rotated into outputs at the end
    int interleave = 1; // Row (lean), > 1: a row is a contiguous [R, interleave] slab reduced over its first dim (K counts the outputs, rows x interleave)
    int group_tile = 0; // Col, > 0: small contiguous [R, kin] groups staged through LDS, this many groups per workgroup
    int row_tile = 0;   // Row, > 0: short contiguous rows staged through LDS, this many rows per workgroup
    int flat_t = 0;     // Col, > 0: contiguous [R, kin] slab walked as a flat array by this many threads
    int flat_xb = 0;    // > 0: a period of the flat walk is wider than a workgroup and spans this many of them;
                        // `split` then counts the partials per output (slices x row phases)
    int flat_phases = 1;  // rows per period in that case
};

// Build the plan for reducing `axes` (already normalised) of a view.
// `elem_size` and `data` decide whether 128-bit loads are legal; `acc_size` is
// the size of one accumulator (bounds the LDS a column kernel may use). `heavy`: the op spends many
// instructions per element (an exponential, f64 arithmetic on f32 data), which wants more wavefronts
// per compute unit than a plain sum.
ReducePlan plan_reduce(const void* data, const int64_t* shape, const int64_t* strides, int ndim,
                       const int64_t* axes, int naxes, size_t elem_size, size_t acc_size, bool heavy = false);

std::string describe(const ReducePlan& p);

enum class NormKind {
    Empty,
    RowReg,     // a row sits in the registers of `tpr` threads; one HBM read, one write
    RowStream,  // rows too long for registers: statistics pass, then a second read
    RowSplit,   // few, very long rows: several workgroups per row (statistics, finalize, apply)
    Col,        // the normalised axis is strided in input and output alike; lanes walk the inner dim
    ColSplit,   // same layout, vectorisable inner dim: statistics over workgroups, finalize, apply in place
    Transposed, // input contiguous along the rows, output along the axis: statistics, then a register-tile transpose
    TransposedTile,  // same layout, a block of rows fits one compute unit's registers: one read, one write
    ColReg,     // softmax over a SHORT strided axis (channels): each thread keeps the whole axis of its inner positions in registers
    Generic     // anything else: one block per row, per-element offset arithmetic
};

struct NormPlan {
    NormKind kind = NormKind::Empty;
    int64_t rows = 0, cols = 0;
    Dims kept_in;        // input strides of the row dims (logical order, coalesced with the output)
    Dims kept_out;       // output strides of the same dims
    Dims norm_in;        // input (size, stride) of the normalised dims, logical order, coalesced
    int64_t out_axis_stride = 1;  // output stride between consecutive elements of a row
    int vec = 1;
    int tpr = 1;      // threads per row (RowReg / RowStream / Generic); TransposedTile: lanes along the rows (rgN)
    int rpb = 1;      // rows per block; TransposedTile: wavefronts per workgroup
    int nchunk = 1;   // RowReg: vectors held per thread
    int max_blocks = 1024;  // RowReg layernorm: workgroups launched at most (they walk the rows)
    int64_t inner = 1;  // Col: size of the contiguous inner dim the lanes walk
    int sstride = 1;    // RowReg: 2 = the row's elements sit at every second position of full vectors
    int flat_t = 0;     // ColSplit, > 0: a narrow inner dim; the slab is walked as a flat array by this many threads
    int interleave = 1;  // RowReg softmax whose rows are contiguous [cols / |interleave|, |interleave|] slabs normalised over their first dim: > 1, a divisor of the vector or two vectors; < 0, minus an inner dim of 3, 5, 6 or 7 (the largest multiple of it of a row's lanes take part)
    int slab_tile = 0;  // Col softmax over the middle axis of mid-sized contiguous [cols, L] slabs with a narrow L: one workgroup per slab through LDS (the value: lanes per column)
    int group_tile = 0; // Col softmax over a short middle axis of small contiguous [cols, L] groups: this many groups per workgroup through LDS
    int lds_rows = 0;   // RowReg softmax of 2- and 4-byte types: long rows held in the registers and the LDS of tpr = 256 or 512 threads (nchunk: vectors per thread in both together)
    int raw_rows = 0;   // RowReg softmax of 2-byte types, 98305 ... 131072 elements per row: only the raw row stays in registers
    int gb_lds = 0;     // RowReg layernorm: 1 = gamma / beta in LDS (2-byte types, three or four vectors of the row per
                        // thread), 2 = gamma / beta read from L2 for every row (rows too long for either)
    int tile_rows = 0;  // RowReg, > 0: short back-to-back rows; the plain kinds stage this many rows per workgroup in LDS
    int shift = 0;      // RowStream: rows start off 16-byte boundaries; aligned vectors, masked at both ends
    int tsplit = 1;     // Transposed: workgroups sharing the axis in the statistics pass
    size_t scratch_bytes = 0;  // Transposed: partial statistics (rows * tsplit * 24 bytes at most)
};

// axis >= 0: softmax-style single axis; n_norm_dims > 0: trailing dims (layernorm).
// fused: the plan is for a fused kind: layernorm(x + residual), whose rows are held twice, or the
// causal softmax, which the plain softmax's register + LDS kernels do not implement.
NormPlan plan_normalize(const void* in_data, const void* out_data, const int64_t* shape,
                        const int64_t* strides, int ndim, int64_t axis, int n_norm_dims,
                        size_t elem_size, bool fused = false);

std::string describe(const NormPlan& p);

// Turn a plan into the generic row form (one group of lanes per row, per-element offsets):
// what the caller falls back to when an operand rules the specialised kernels out.
void demote_to_generic(NormPlan& p);

// Keep of a plan what the streaming row kernel can run: rows that are contiguous along the axis and
// on the vector grid keep their vector width, everything else becomes the generic row form.
void restrict_to_row_stream(NormPlan& p);

// ---- elementwise: strided copy (contiguous()), fill, binary ops with broadcasting ----

enum class EwKind {
    Empty,
    Inner,      // lanes walk the innermost coalesced dim (vectors where every operand allows them)
    Transpose   // some other dim is the contiguous one in the input (a binary op: in one or both): tiles transposed in registers / LDS
};

// The output is contiguous over `size[0..n)`; `stride[k][i]` is operand k's stride (in
// elements, 0 = broadcast) along dim i. Dims are coalesced across all operands at once.
struct EwPlan {
    EwKind kind = EwKind::Empty;
    int n = 0;     // coalesced dims
    int nin = 0;   // input operands (1 or 2)
    int64_t size[kMaxDims] = {};
    int64_t stride[2][kMaxDims] = {};
    int64_t total = 0;
    int vec = 1;   // output elements per thread along the innermost dim
    int sstride = 1;  // 2: (copy) the innermost input stride is 2: full vectors in, every second element kept
    // Transpose: dim `tdim` has input stride 1; the innermost dim is strided in the input
    int tdim = -1;
    bool tile_lds = false;  // Transpose: both dims hold a whole (16 vec)^2 tile: staged through LDS
    int tmask = 0;          // Transpose: bit k set = operand k is the one contiguous along `tdim` (a binary op may have one such operand or two)
};

EwPlan plan_elementwise(const void* out_data, const int64_t* shape, int ndim, int nin, const void* const* in_data,
                        const int64_t* const* in_strides, size_t elem_size, bool allow_transpose);

std::string describe(const EwPlan& p);

}  // namespace hpt
