// The interleaved and modular rows of row_reg_kernel (softmax over the middle axis of a contiguous [B, C, L] with a
// narrow L) for one softmax kind and the four float dtypes. Compiled with -DHPT_NORM_KIND=<0 or 1>.
#include "norm_interleaved.hpp"
#include "norm_kernels.hpp"

#ifndef HPT_NORM_KIND
#error "compile with -DHPT_NORM_KIND=<kind>"
#endif

namespace hpt {

namespace {

constexpr int KIND = HPT_NORM_KIND;
static_assert(KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX, "interleaved rows are a softmax plan");

// Rows that are [cols / IL, IL] slabs, softmax over the first dim (whole aligned vectors, IL a divisor of the vector).
template <class T, int VEC, int IL, bool PF = false>
void launch_row_reg_interleaved(const NormPlan& p, const NormArgs& a, dim3 grid, dim3 block, hipStream_t st) {
    if constexpr ((KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX) && VEC > 1 &&
                  ((IL > 1 && (VEC % IL == 0 || IL == 2 * VEC)) || (IL <= -3 && IL >= -7 && VEC % (-IL) != 0))) {
        switch (p.nchunk) {
            case 3: row_reg_kernel<KIND, T, VEC, 3, 1, false, PF, 0, IL><<<grid, block, 0, st>>>(a); return;
            case 4: row_reg_kernel<KIND, T, VEC, 4, 1, false, PF, 0, IL><<<grid, block, 0, st>>>(a); return;
            case 5: row_reg_kernel<KIND, T, VEC, 5, 1, false, PF, 0, IL><<<grid, block, 0, st>>>(a); return;
            case 6: row_reg_kernel<KIND, T, VEC, 6, 1, false, PF, 0, IL><<<grid, block, 0, st>>>(a); return;
            case 7: row_reg_kernel<KIND, T, VEC, 7, 1, false, PF, 0, IL><<<grid, block, 0, st>>>(a); return;
            case 8: row_reg_kernel<KIND, T, VEC, 8, 1, false, PF, 0, IL><<<grid, block, 0, st>>>(a); return;
            default: break;
        }
        // (rows of 512 and 1024 threads hold at least three vectors per thread)
        if constexpr (!PF) {
            switch (p.nchunk) {
                case 1: row_reg_kernel<KIND, T, VEC, 1, 1, false, false, 0, IL><<<grid, block, 0, st>>>(a); return;
                case 2: row_reg_kernel<KIND, T, VEC, 2, 1, false, false, 0, IL><<<grid, block, 0, st>>>(a); return;
                default: break;
            }
        }
    }
    fail(HPT_ERR_KERNEL, "interleaved rows: no kernel for %d vectors per thread of %d interleaved softmaxes", p.nchunk, IL);
}

}  // namespace

template <class T> static void launch_interleaved_t(const NormPlan& p, const NormArgs& a, dim3 grid, dim3 block, hipStream_t st) {
    constexpr int FULL = 16 / sizeof(T);
    if (p.vec != FULL || p.sstride != 1 || p.shift || p.tile_rows || p.gb_lds || p.cols % FULL != 0 ||
        (p.interleave > 1 && FULL % p.interleave != 0 && (p.interleave != 2 * FULL || p.tpr < 2)) ||
        (p.interleave < 0 && (int64_t)(p.tpr / -p.interleave * -p.interleave) * p.nchunk * FULL < p.cols))
        fail(HPT_ERR_KERNEL, "interleaved rows need whole aligned vectors");
    // (the longest slabs: 512 workgroups walk the rows and prefetch the next one - f32 [1000, 16384, 2] 59.7 -> 54.7 us,
    // f16 [2000, 4096, 8] 98.3 -> 89.3; rows of 512 threads lose by it, f32 [2000, 1280, 8] 35.8 -> 41.5)
    if (p.tpr == 1024 && p.nchunk >= 3) {
        if (grid.x > 512u) grid.x = 512u;
        switch (p.interleave) {
            case 2: launch_row_reg_interleaved<T, FULL, 2, true>(p, a, grid, block, st); return;
            case 4: launch_row_reg_interleaved<T, FULL, 4, true>(p, a, grid, block, st); return;
            case 8: launch_row_reg_interleaved<T, FULL, 8, true>(p, a, grid, block, st); return;
            case 16: launch_row_reg_interleaved<T, FULL, 16, true>(p, a, grid, block, st); return;
            case -3: launch_row_reg_interleaved<T, FULL, -3, true>(p, a, grid, block, st); return;
            case -5: launch_row_reg_interleaved<T, FULL, -5, true>(p, a, grid, block, st); return;
            case -6: launch_row_reg_interleaved<T, FULL, -6, true>(p, a, grid, block, st); return;
            case -7: launch_row_reg_interleaved<T, FULL, -7, true>(p, a, grid, block, st); return;
            default: break;
        }
    }
    switch (p.interleave) {
        case 2: launch_row_reg_interleaved<T, FULL, 2>(p, a, grid, block, st); return;
        case 4: launch_row_reg_interleaved<T, FULL, 4>(p, a, grid, block, st); return;
        case 8: launch_row_reg_interleaved<T, FULL, 8>(p, a, grid, block, st); return;
        case 16: launch_row_reg_interleaved<T, FULL, 16>(p, a, grid, block, st); return;
        case -3: launch_row_reg_interleaved<T, FULL, -3>(p, a, grid, block, st); return;
        case -5: launch_row_reg_interleaved<T, FULL, -5>(p, a, grid, block, st); return;
        case -6: launch_row_reg_interleaved<T, FULL, -6>(p, a, grid, block, st); return;
        case -7: launch_row_reg_interleaved<T, FULL, -7>(p, a, grid, block, st); return;
        default: fail(HPT_ERR_KERNEL, "interleaved rows: %d softmaxes per row", p.interleave);
    }
}

template <> void launch_interleaved_rows<HPT_NORM_KIND, f16_t>(const NormPlan& p, const NormArgs& a, dim3 grid, dim3 block, hipStream_t st) {
    launch_interleaved_t<f16_t>(p, a, grid, block, st);
}
template <> void launch_interleaved_rows<HPT_NORM_KIND, bf16_t>(const NormPlan& p, const NormArgs& a, dim3 grid, dim3 block, hipStream_t st) {
    launch_interleaved_t<bf16_t>(p, a, grid, block, st);
}
template <> void launch_interleaved_rows<HPT_NORM_KIND, float>(const NormPlan& p, const NormArgs& a, dim3 grid, dim3 block, hipStream_t st) {
    launch_interleaved_t<float>(p, a, grid, block, st);
}
template <> void launch_interleaved_rows<HPT_NORM_KIND, double>(const NormPlan& p, const NormArgs& a, dim3 grid, dim3 block, hipStream_t st) {
    launch_interleaved_t<double>(p, a, grid, block, st);
}

}  // namespace hpt
