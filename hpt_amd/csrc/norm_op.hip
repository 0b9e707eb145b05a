// One normalisation kind (softmax, log_softmax or layernorm) for the four
// float dtypes. Compiled once per kind with -DHPT_NORM_KIND=<0...5>.
#include <algorithm>

#include "norm_interleaved.hpp"
#include "transpose_norm.hpp"

#ifndef HPT_NORM_KIND
#error "compile with -DHPT_NORM_KIND=<kind>"
#endif

namespace hpt {

namespace {

constexpr int KIND = HPT_NORM_KIND;

inline int ilog2(int v) {
    int l = 0;
    while ((1 << l) < v) ++l;
    return l;
}

template <class T, int VEC, int SS = 1, bool SHIFT = false, bool PF = false>
void launch_row_reg(const NormPlan& p, const NormArgs& a, dim3 grid, dim3 block, hipStream_t st) {
    // (3, 5, 6 and 7 vectors per thread: rows of whole vectors whose length is 3, 5, 6 or 7 times a power of
    // two - 768, 1536, 2560, 3072, 3584, 5120, 6144 ... - without idle lanes; full-vector rows only)
    if constexpr (VEC > 1 && SS == 1) {
        switch (p.nchunk) {
            case 3: row_reg_kernel<KIND, T, VEC, 3, SS, SHIFT, PF><<<grid, block, 0, st>>>(a); return;
            case 5: row_reg_kernel<KIND, T, VEC, 5, SS, SHIFT, PF><<<grid, block, 0, st>>>(a); return;
            case 6: row_reg_kernel<KIND, T, VEC, 6, SS, SHIFT, PF><<<grid, block, 0, st>>>(a); return;
            case 7: row_reg_kernel<KIND, T, VEC, 7, SS, SHIFT, PF><<<grid, block, 0, st>>>(a); return;
            default: break;
        }
    }
    switch (p.nchunk) {
        case 1: row_reg_kernel<KIND, T, VEC, 1, SS, SHIFT, PF><<<grid, block, 0, st>>>(a); break;
        case 2: row_reg_kernel<KIND, T, VEC, 2, SS, SHIFT, PF><<<grid, block, 0, st>>>(a); break;
        case 4: row_reg_kernel<KIND, T, VEC, 4, SS, SHIFT, PF><<<grid, block, 0, st>>>(a); break;
        case 8: row_reg_kernel<KIND, T, VEC, 8, SS, SHIFT, PF><<<grid, block, 0, st>>>(a); break;
        default: fail(HPT_ERR_KERNEL, "row_reg: unsupported chunk count %d", p.nchunk);
    }
}

// Few, very long rows: several workgroups per row.
template <class T, int VEC, bool UA> void launch_row_split(const NormPlan& p, const NormArgs& a, hipStream_t st) {
    RowSplitArgs r{};
    r.in = a.in;
    r.out = a.out;
    r.gamma = a.gamma;
    r.beta = a.beta;
    r.residual = a.residual;
    r.kept_in = a.kept_in;
    r.rows = a.rows;
    r.cols = a.cols;
    r.eps = a.eps;
    r.inv_cols = a.inv_cols;
    r.S = p.tsplit;
    const int64_t nv = UA ? (a.cols + VEC - 1) / VEC : a.cols / VEC;
    r.chunk_v = (nv + r.S - 1) / r.S;
    r.part = a.scratch;
    const dim3 grid((unsigned)r.S, (unsigned)a.rows);
    row_split_stats_kernel<KIND, T, VEC, UA><<<grid, dim3(256), 0, st>>>(r);
    row_split_apply_kernel<KIND, T, VEC, UA><<<grid, dim3(256), 0, st>>>(r);
}

// Softmax / log_softmax over an axis that is strided in the output too: three passes.
template <class T, int VEC> void launch_col_split(const NormPlan& p, const NormArgs& a, hipStream_t st) {
    TransposedArgs t{};
    t.in = a.in;
    t.out = a.out;
    const int nk = p.kept_in.n;
    const unsigned batch = nk > 1 ? (unsigned)p.kept_in.size[0] : 1u;
    t.R = (int)p.kept_in.size[nk - 1];
    t.cols = (int)p.cols;
    t.S = p.tsplit;
    t.stats = a.scratch;
    t.params = (char*)a.scratch + (size_t)batch * t.S * t.R * 16;
    t.sa = a.sa;
    t.bi = nk > 1 ? p.kept_in.stride[0] : 0;
    t.inv_cols = a.inv_cols;
    using Part = typename RowPartial<KIND, T>::type;
    if constexpr (VEC > 1) {
        if (p.flat_t > 0) {  // narrow inner dim: flat walk (statistics, the shared finalize, apply)
            const unsigned block = (unsigned)((p.flat_t + 63) / 64 * 64);
            const size_t smem = (size_t)p.flat_t * VEC * sizeof(Part);
            const dim3 grid((unsigned)t.S, 1, batch);
            if (p.shift) {  // batch slabs off 16-byte boundaries: unaligned vectors
                col_flat_stats_kernel<KIND, T, VEC, true><<<grid, dim3(block), smem, st>>>(t, p.flat_t);
                transposed_finalize_kernel<KIND, T><<<dim3((unsigned)((t.R + 15) / 16), 1, batch), dim3(16, 16), 0, st>>>(t);
                col_flat_apply_kernel<KIND, T, VEC, true><<<grid, dim3(block), 0, st>>>(t, p.flat_t, t.S);
            } else {
                col_flat_stats_kernel<KIND, T, VEC><<<grid, dim3(block), smem, st>>>(t, p.flat_t);
                transposed_finalize_kernel<KIND, T><<<dim3((unsigned)((t.R + 15) / 16), 1, batch), dim3(16, 16), 0, st>>>(t);
                col_flat_apply_kernel<KIND, T, VEC><<<grid, dim3(block), 0, st>>>(t, p.flat_t, t.S);
            }
            return;
        }
    }
    const unsigned nw = (unsigned)p.tpr;
    const unsigned rg = (unsigned)((t.R + 64 * VEC - 1) / (64 * VEC));
    const bool ua = VEC > 1 && p.shift;  // inner rows off the vector grid: unaligned vectors
    if (ua && t.R < VEC) fail(HPT_ERR_KERNEL, "col-split: an inner row of %d elements holds no vector of %d", t.R, VEC);
    if constexpr (VEC > 1) {
        if (ua)
            transposed_stats_kernel<KIND, T, VEC, true>
                <<<dim3(rg, (unsigned)t.S, batch), dim3(64 * nw), (size_t)nw * VEC * 64 * sizeof(Part), st>>>(t);
    }
    if (!ua)
        transposed_stats_kernel<KIND, T, VEC>
            <<<dim3(rg, (unsigned)t.S, batch), dim3(64 * nw), (size_t)nw * VEC * 64 * sizeof(Part), st>>>(t);
    transposed_finalize_kernel<KIND, T><<<dim3((unsigned)((t.R + 15) / 16), 1, batch), dim3(16, 16), 0, st>>>(t);
    // apply: enough axis chunks for ~2048 workgroups, at least 16 positions each
    int64_t want = (2048 + (int64_t)rg * batch - 1) / ((int64_t)rg * batch);
    int64_t chunks = std::max<int64_t>(1, std::min<int64_t>(want, (t.cols + 15) / 16));
    chunks = std::min<int64_t>(chunks, 65535);
    const int chunk = (int)((t.cols + chunks - 1) / chunks);
    chunks = (t.cols + chunk - 1) / chunk;
    if constexpr (VEC > 1) {
        if (ua) {
            col_apply_kernel<KIND, T, VEC, true><<<dim3(rg, (unsigned)chunks, batch), dim3(256), 0, st>>>(t, chunk);
            return;
        }
    }
    col_apply_kernel<KIND, T, VEC><<<dim3(rg, (unsigned)chunks, batch), dim3(256), 0, st>>>(t, chunk);
}

// A short strided axis held in registers (softmax kinds).
// WIDE: twice the vectors per thread (128 registers of raw values instead of 64).
template <class T, int EV, bool WIDE = false> void launch_col_reg(const NormPlan& p, const NormArgs& a, hipStream_t st) {
    constexpr int REGS = (EV * (int)sizeof(T) + 3) / 4;
    constexpr int NC = (64 / REGS > 64 ? 64 : 64 / REGS) * (WIDE ? 2 : 1);
    ColRegArgs c{};
    const int nk = p.kept_in.n;
    c.in = a.in;
    c.out = a.out;
    c.sa = a.sa;
    c.bi = nk > 1 ? p.kept_in.stride[0] : 0;
    c.L = p.kept_in.size[nk - 1];
    c.nvec = p.shift ? (c.L + EV - 1) / EV : c.L / EV;
    c.total = (nk > 1 ? p.kept_in.size[0] : 1) * c.nvec;
    c.cols = (int)p.cols;
    c.ty_log2 = ilog2(p.tpr);  // thread rows per inner position
    if (p.tpr > 16 || c.cols > NC * p.tpr)
        fail(HPT_ERR_KERNEL, "col-reg: axis of %d does not fit %d thread rows of %d vectors", c.cols, p.tpr, NC);
    const int64_t tx = 256 / p.tpr;
    const dim3 grid((unsigned)((c.total + tx - 1) / tx));
    if constexpr (EV > 1) {
        if (p.shift) {
            col_reg_kernel<KIND, T, EV, NC, true><<<grid, dim3(256), 0, st>>>(c);
            return;
        }
    }
    col_reg_kernel<KIND, T, EV, NC><<<grid, dim3(256), 0, st>>>(c);
}

// The transposed forms (kinds 0..2 only).
template <class T> void launch_transposed(const NormPlan& p, const NormArgs& a, hipStream_t st) {
    constexpr int FULL = 16 / sizeof(T);
    if (p.kind == NormKind::TransposedTile) {
        TileArgs t{};
        t.in = a.in;
        t.out = a.out;
        t.gamma = a.gamma;
        t.beta = a.beta;
        const int nk = p.kept_in.n;
        const unsigned batch = nk > 1 ? (unsigned)p.kept_in.size[0] : 1u;
        t.R = (int)p.kept_in.size[nk - 1];
        t.cols = (int)p.cols;
        t.sa = a.sa;
        t.bi = nk > 1 ? p.kept_in.stride[0] : 0;
        t.eps = a.eps;
        t.inv_cols = a.inv_cols;
        t.rg_log2 = ilog2(p.tpr);
        t.share_log2 = p.tpr >= 8 ? 0 : (p.tpr == 4 ? 1 : 2);
        const unsigned blocks = (unsigned)((t.R + p.tpr * FULL - 1) / (p.tpr * FULL));
        transposed_tile_kernel<KIND, T><<<dim3(blocks, batch), dim3(64u * (unsigned)p.rpb), 0, st>>>(t);
        return;
    }
    if (p.kind == NormKind::Transposed) {
        constexpr int TILE = 8 * FULL;
        TransposedArgs t{};
        t.in = a.in;
        t.out = a.out;
        t.gamma = a.gamma;
        t.beta = a.beta;
        const int nk = p.kept_in.n;
        const unsigned batch = nk > 1 ? (unsigned)p.kept_in.size[0] : 1u;
        t.R = (int)p.kept_in.size[nk - 1];
        t.cols = (int)p.cols;
        t.S = p.tsplit;
        // scratch: [batch][S][R] partial statistics (16 bytes each at most), then [batch][3][R] numbers
        t.stats = a.scratch;
        t.params = (char*)a.scratch + (size_t)batch * t.S * t.R * 16;
        t.sa = a.sa;
        t.bi = nk > 1 ? p.kept_in.stride[0] : 0;
        t.eps = a.eps;
        t.inv_cols = a.inv_cols;
        t.cols_per_split = (t.cols + t.S - 1) / t.S;
        const int tiles = (t.cols + TILE - 1) / TILE;
        const unsigned rt = (unsigned)((t.R + TILE - 1) / TILE);
        const unsigned rg = (unsigned)((t.R + 64 * FULL - 1) / (64 * FULL));
        using Part = typename RowPartial<KIND, T>::type;
        const unsigned nw = (unsigned)p.tpr;  // wavefronts per workgroup of the statistics pass
        transposed_stats_kernel<KIND, T>
            <<<dim3(rg, (unsigned)t.S, batch), dim3(64 * nw), (size_t)nw * FULL * 64 * sizeof(Part), st>>>(t);
        transposed_finalize_kernel<KIND, T><<<dim3((unsigned)((t.R + 15) / 16), 1, batch), dim3(16, 16), 0, st>>>(t);
        transposed_apply_kernel<KIND, T><<<dim3((rt + 3) / 4, (unsigned)((tiles + 1) / 2), batch), dim3(256), 0, st>>>(t);
        return;
    }
}

template <class T> void launch_t(const NormPlan& p, NormArgs a, hipStream_t st) {
    constexpr int FULL = 16 / sizeof(T);
    if (p.kind == NormKind::Empty) return;
    a.tpr = p.tpr;
    a.tpr_log2 = ilog2(p.tpr);
    a.rpb = p.rpb;
    a.inv_cols = 1.0 / (double)p.cols;
    dim3 grid((unsigned)((p.rows + p.rpb - 1) / p.rpb));
    dim3 block((unsigned)(p.tpr * p.rpb));
    if (p.kind == NormKind::Col && p.slab_tile > 0) {
        if constexpr (FULL > 1 && (KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX)) {
            const int L = (int)p.kept_in.size[1];
            const size_t bytes = ((size_t)p.cols * L * sizeof(T) + 15) / 16 * 16;
            norm_slab_kernel<KIND, T, FULL><<<dim3((unsigned)p.kept_in.size[0]), dim3(256), bytes, st>>>(a, L, ilog2(p.slab_tile));
        } else {
            fail(HPT_ERR_KERNEL, "slab tiles are a softmax plan");
        }
        return;
    }
    if (p.kind == NormKind::Col && p.group_tile > 0) {
        if constexpr (FULL > 1 && (KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX)) {
            const int64_t batch = p.kept_in.size[0];
            a.rpb = p.group_tile;
            // a very narrow inner dim with groups of a multiple of 128 bytes: the lanes' group starts collide in LDS
            const bool padded = p.kept_in.size[1] * (int64_t)sizeof(T) <= 16 && (p.cols * p.kept_in.size[1] * (int64_t)sizeof(T)) % 128 == 0;
            const dim3 ggrid((unsigned)((batch + p.group_tile - 1) / p.group_tile));
            if (padded) norm_group_tile_kernel<KIND, T, FULL, true><<<ggrid, dim3(256), 0, st>>>(a, (int)p.kept_in.size[1], batch);
            else norm_group_tile_kernel<KIND, T, FULL, false><<<ggrid, dim3(256), 0, st>>>(a, (int)p.kept_in.size[1], batch);
        } else {
            fail(HPT_ERR_KERNEL, "group tiles are a softmax plan");
        }
        return;
    }
    if (p.kind == NormKind::RowSplit) {
        if constexpr (norm_is_causal(KIND)) {
            fail(HPT_ERR_KERNEL, "row-split has no causal form");
        } else {
            if (p.vec == FULL && FULL > 1 && p.shift) launch_row_split<T, FULL, true>(p, a, st);
            else if (p.vec == FULL && FULL > 1) launch_row_split<T, FULL, false>(p, a, st);
            else launch_row_split<T, 1, false>(p, a, st);
        }
        return;
    }
    if (p.kind == NormKind::ColReg) {
        if constexpr (KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX) {
            switch (p.vec) {
                case 1: launch_col_reg<T, 1>(p, a, st); break;
                case 2: if constexpr (FULL >= 2) launch_col_reg<T, 2>(p, a, st); break;
                case 4:
                    if constexpr (FULL == 4) {
                        if (p.nchunk == 32) launch_col_reg<T, 4, true>(p, a, st);
                        else launch_col_reg<T, 4>(p, a, st);
                    } else if constexpr (FULL > 4) {
                        launch_col_reg<T, 4>(p, a, st);
                    }
                    break;
                case 8: if constexpr (FULL >= 8) launch_col_reg<T, 8>(p, a, st); break;
                default: fail(HPT_ERR_KERNEL, "col-reg: unsupported vector width %d", p.vec);
            }
        } else {
            fail(HPT_ERR_KERNEL, "col-reg is a softmax plan");
        }
        return;
    }
    if (p.kind == NormKind::ColSplit) {
        if constexpr (KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX) {
            if (p.vec == FULL && FULL > 1) launch_col_split<T, FULL>(p, a, st);
            else launch_col_split<T, 1>(p, a, st);
        } else {
            fail(HPT_ERR_KERNEL, "col-split is a softmax plan");
        }
        return;
    }
    if (p.kind == NormKind::TransposedTile || p.kind == NormKind::Transposed) {
        // the fused kinds run on the row kernels only (the caller demotes transposed plans)
        if constexpr (KIND > NORM_LAYERNORM) fail(HPT_ERR_KERNEL, "fused normalisation: no transposed kernel for this kind");
        else launch_transposed<T>(p, a, st);
        return;
    }
    if (p.kind == NormKind::RowReg && p.lds_rows) {
        // long rows that stay on chip: registers + LDS; the fused kinds stream
        if constexpr (FULL > 1 && sizeof(T) <= 4 && (KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX)) {
            // 24 + 8 vectors of a four-byte type (16 + 8 of a two-byte type) per thread and 128 registers:
            // 256 or 512 threads; 48 + 16 (32 + 16) and 256 registers: 512 threads. Shifted four-byte rows:
            // 20 + 8 and 44 + 16.
            constexpr int kRegs = sizeof(T) == 4 ? 24 : 16;
            constexpr int kRegsShift = sizeof(T) == 4 ? 20 : 16;
            constexpr int kBigShift = sizeof(T) == 4 ? 44 : 32;
            if (!p.shift) {
                if (p.nchunk == kRegs + 8 && p.tpr == 256) {
                    row_lds_kernel<KIND, T, kRegs, 8, false, 256, 4><<<grid, dim3(256), 0, st>>>(a);
                    return;
                }
                if (p.nchunk == kRegs + 8 && p.tpr == 512) {
                    row_lds_kernel<KIND, T, kRegs, 8, false, 512, 4><<<grid, dim3(512), 0, st>>>(a);
                    return;
                }
                if (p.nchunk == kRegs + 8 && p.tpr == 1024) {
                    row_lds_kernel<KIND, T, kRegs, 8, false, 1024, 1><<<grid, dim3(1024), 0, st>>>(a);
                    return;
                }
                if (p.nchunk == 2 * kRegs + 16 && p.tpr == 512) {
                    row_lds_kernel<KIND, T, 2 * kRegs, 16, false, 512, 1><<<grid, dim3(512), 0, st>>>(a);
                    return;
                }
            } else {
                if (p.nchunk == kRegsShift + 8 && p.tpr == 256) {
                    row_lds_kernel<KIND, T, kRegsShift, 8, true, 256, 4><<<grid, dim3(256), 0, st>>>(a);
                    return;
                }
                if (p.nchunk == kRegsShift + 8 && p.tpr == 512) {
                    row_lds_kernel<KIND, T, kRegsShift, 8, true, 512, 4><<<grid, dim3(512), 0, st>>>(a);
                    return;
                }
                if (p.nchunk == kRegsShift + 8 && p.tpr == 1024) {
                    row_lds_kernel<KIND, T, kRegsShift, 8, true, 1024, 1><<<grid, dim3(1024), 0, st>>>(a);
                    return;
                }
                if (p.nchunk == kBigShift + 16 && p.tpr == 512) {
                    row_lds_kernel<KIND, T, kBigShift, 16, true, 512, 1><<<grid, dim3(512), 0, st>>>(a);
                    return;
                }
            }
            fail(HPT_ERR_KERNEL, "row_lds: no kernel for %d threads x %d vectors", p.tpr, p.nchunk);
        }
        if constexpr (FULL > 1) {
            // (the fused kinds stream such rows, a full workgroup per row)
            a.tpr = 1024;
            a.tpr_log2 = 10;
            if (p.shift) row_stream_kernel<KIND, T, FULL, true><<<grid, dim3(1024), 0, st>>>(a);
            else row_stream_kernel<KIND, T, FULL><<<grid, dim3(1024), 0, st>>>(a);
        }
        return;
    }
    if (p.kind == NormKind::RowReg && p.raw_rows) {
        // two-byte softmax rows of 98305 ... 131072 elements: the raw row in registers, sixteen vectors per
        // thread; the fused kinds stream
        if constexpr (sizeof(T) == 2 && (KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX)) {
            if (grid.x > 512u) grid.x = 512u;
            row_raw_kernel<KIND, T, 16><<<grid, dim3(1024), 0, st>>>(a);
        } else {
            if (p.vec == FULL) row_stream_kernel<KIND, T, FULL><<<grid, block, 0, st>>>(a);
            else row_stream_kernel<KIND, T, 1><<<grid, block, 0, st>>>(a);
        }
        return;
    }
    if (p.kind == NormKind::RowReg && p.interleave != 1) {
        // (these kernels are compiled in a translation unit of their own)
        if constexpr (KIND == NORM_SOFTMAX || KIND == NORM_LOGSOFTMAX) launch_interleaved_rows<KIND, T>(p, a, grid, block, st);
        else fail(HPT_ERR_KERNEL, "interleaved rows are a softmax plan");
        return;
    }
    if (p.kind == NormKind::RowReg) {
        // Layernorm workgroups walk the rows (gamma / beta stay in registers);
        // softmax has nothing to reuse across rows and runs one row per group.
        if constexpr (FULL > 1 && KIND <= NORM_LAYERNORM) {
            if (p.tile_rows > 0) {
                a.rpb = p.tile_rows;
                a.tpr = 1;
                while (a.tpr < 64 && a.tpr * 8 < p.cols) a.tpr <<= 1;
                a.tpr_log2 = ilog2(a.tpr);
                // (the lanes' sweeps are unrolled to exactly the elements a lane of this row length has: rows of 257 take
                // 5 per lane of 64, and three more steps with every lane masked off cost a fifth of the launch)
                const dim3 tgrid((unsigned)((p.rows + p.tile_rows - 1) / p.tile_rows));
                switch ((int)((p.cols + a.tpr - 1) / a.tpr)) {
                    case 1: norm_tile_kernel<KIND, T, FULL, 1><<<tgrid, dim3(256), 0, st>>>(a); break;
                    case 2: norm_tile_kernel<KIND, T, FULL, 2><<<tgrid, dim3(256), 0, st>>>(a); break;
                    case 3: norm_tile_kernel<KIND, T, FULL, 3><<<tgrid, dim3(256), 0, st>>>(a); break;
                    case 4: norm_tile_kernel<KIND, T, FULL, 4><<<tgrid, dim3(256), 0, st>>>(a); break;
                    case 5: norm_tile_kernel<KIND, T, FULL, 5><<<tgrid, dim3(256), 0, st>>>(a); break;
                    case 6: norm_tile_kernel<KIND, T, FULL, 6><<<tgrid, dim3(256), 0, st>>>(a); break;
                    case 7: norm_tile_kernel<KIND, T, FULL, 7><<<tgrid, dim3(256), 0, st>>>(a); break;
                    case 8: norm_tile_kernel<KIND, T, FULL, 8><<<tgrid, dim3(256), 0, st>>>(a); break;
                    default: fail(HPT_ERR_KERNEL, "norm_tile: %d elements per lane", (int)((p.cols + a.tpr - 1) / a.tpr));
                }
                return;
            }
        }
        if (norm_is_layer(KIND) && grid.x > (unsigned)p.max_blocks) grid.x = (unsigned)p.max_blocks;
        if constexpr (FULL > 1) {
            if (p.vec == FULL && p.shift) {
                // shifted rows: a thread's gamma / beta fit every row it walks only if those rows share
                // their misalignment, i.e. the row step is a whole number of vectors
                if (norm_is_layer(KIND) && (int64_t)grid.x * p.rpb < p.rows) {
                    if (grid.x >= (unsigned)FULL) grid.x -= grid.x % FULL;
                    else fail(HPT_ERR_KERNEL, "row_reg: shifted rows need a row step of whole vectors");
                }
                launch_row_reg<T, FULL, 1, true>(p, a, grid, block, st);
                return;
            }
        }
        if constexpr (FULL > 1 && norm_is_layer(KIND)) {
            if (p.gb_lds == 2 && p.vec == FULL && p.sstride == 1 && !p.shift) {
                // gamma / beta from L2 in the last sweep: one row per group of threads, nothing carried between rows
                // (rows of 512 or 1024 threads: 512 workgroups walk the rows and prefetch)
                const bool pf = p.tpr >= 512 && KIND != NORM_ADD_LAYERNORM;
                if (pf && grid.x > 512u) grid.x = 512u;
#define HPT_L2GB_CASE(N)                                                                                  \
    case 2 * N: row_reg_kernel<KIND, T, FULL, N, 1, false, false, 2><<<grid, block, 0, st>>>(a); return; \
    case 2 * N + 1: row_reg_kernel<KIND, T, FULL, N, 1, false, true, 2><<<grid, block, 0, st>>>(a); return;
                if constexpr (sizeof(T) >= 4) {  // (two-byte rows of seven or eight vectors per thread spill: not planned)
                    switch (p.nchunk * 2 + (pf ? 1 : 0)) {
                        HPT_L2GB_CASE(7) HPT_L2GB_CASE(8)
                        default: break;
                    }
                }
                switch (p.nchunk * 2 + (pf ? 1 : 0)) {
                    HPT_L2GB_CASE(3) HPT_L2GB_CASE(4) HPT_L2GB_CASE(5) HPT_L2GB_CASE(6)
                    default: fail(HPT_ERR_KERNEL, "row_reg: unsupported chunk count %d with gamma / beta from L2", p.nchunk);
                }
#undef HPT_L2GB_CASE
            }
        }
        if constexpr (FULL > 1 && sizeof(T) == 2 && norm_is_layer(KIND)) {
            if (p.gb_lds == 1 && p.vec == FULL && p.sstride == 1 && !p.shift && p.nchunk >= 3 && p.nchunk <= 4) {
                const size_t smem = 2 * (size_t)p.cols * sizeof(T);
                if (p.tpr >= 512 && KIND != NORM_ADD_LAYERNORM) {
                    if (grid.x > 512u) grid.x = 512u;
                    if (p.nchunk == 3) row_reg_kernel<KIND, T, FULL, 3, 1, false, true, 1><<<grid, block, smem, st>>>(a);
                    else row_reg_kernel<KIND, T, FULL, 4, 1, false, true, 1><<<grid, block, smem, st>>>(a);
                } else {
                    if (p.nchunk == 3) row_reg_kernel<KIND, T, FULL, 3, 1, false, false, 1><<<grid, block, smem, st>>>(a);
                    else row_reg_kernel<KIND, T, FULL, 4, 1, false, false, 1><<<grid, block, smem, st>>>(a);
                }
                return;
            }
        }
        if constexpr (FULL > 1 && KIND != NORM_ADD_LAYERNORM) {
            // Long rows: 512 large workgroups that walk the rows and prefetch the next one. Measured
            // (TB/s, without -> with): f32 [3355, 10000] layernorm 3.6 -> 5.1, softmax 3.2 -> 4.2;
            // f32 [2048, 16384] 4.4 -> 5.2 / 4.1 -> 4.8; f16 [1024, 32768] softmax 3.9 -> 4.3. Two-byte
            // softmax rows of 512 threads are the exception (4.6 -> 4.2): they fit three to a compute
            // unit and do better one row per workgroup.
            if (p.vec == FULL && p.sstride == 1 && p.tpr >= 512 &&
                (sizeof(T) >= 4 || p.tpr == 1024 || norm_is_layer(KIND))) {
                if (grid.x > 512u) grid.x = 512u;
                launch_row_reg<T, FULL, 1, false, true>(p, a, grid, block, st);
                return;
            }
        }
        if (p.vec == FULL && p.sstride == 2 && FULL > 1) launch_row_reg<T, FULL, 2>(p, a, grid, block, st);
        else if (p.vec == FULL) launch_row_reg<T, FULL>(p, a, grid, block, st);
        else launch_row_reg<T, 1>(p, a, grid, block, st);
        return;
    }
    if constexpr (FULL > 1) {
        if (p.vec == FULL && p.shift) {
            row_stream_kernel<KIND, T, FULL, true><<<grid, block, 0, st>>>(a);
            return;
        }
    }
    if (p.vec == FULL) row_stream_kernel<KIND, T, FULL><<<grid, block, 0, st>>>(a);
    else row_stream_kernel<KIND, T, 1><<<grid, block, 0, st>>>(a);
}

// FloatBinaryType<TI> of the integer types (hpt-types/src/type_promote.rs)
template <class TI> struct PromotedOf { using type = f16_t; };  // bool, i8, i16, u8, u16
template <> struct PromotedOf<int32_t> { using type = float; };
template <> struct PromotedOf<uint32_t> { using type = float; };
template <> struct PromotedOf<int64_t> { using type = double; };
template <> struct PromotedOf<uint64_t> { using type = double; };

template <class TI> void launch_promoting_t(const NormPlan& p, NormArgs a, hipStream_t st) {
    using T = typename PromotedOf<TI>::type;
    constexpr int FULL = 16 / sizeof(T);
    if (p.kind == NormKind::Empty) return;
    if constexpr (KIND > NORM_LAYERNORM) {
        fail(HPT_ERR_DTYPE, "fused normalisation: the input must have a float dtype");
    } else {
        if (p.kind != NormKind::RowStream && p.kind != NormKind::Generic)
            fail(HPT_ERR_KERNEL, "promoted input: the plan was not restricted to the streaming row kernel");
        a.tpr = p.tpr;
        a.tpr_log2 = ilog2(p.tpr);
        a.rpb = p.rpb;
        a.inv_cols = 1.0 / (double)p.cols;
        const dim3 grid((unsigned)((p.rows + p.rpb - 1) / p.rpb));
        const dim3 block((unsigned)(p.tpr * p.rpb));
        if (p.vec == FULL && FULL > 1) row_stream_kernel<KIND, T, FULL, false, TI><<<grid, block, 0, st>>>(a);
        else row_stream_kernel<KIND, T, 1, false, TI><<<grid, block, 0, st>>>(a);
    }
}

}  // namespace

template <> NormLaunchFn norm_promoting_launcher<HPT_NORM_KIND>(int in_dtype) {
    switch (in_dtype) {
        case HPT_BOOL: return &launch_promoting_t<bool8>;
        case HPT_I8: return &launch_promoting_t<int8_t>;
        case HPT_I16: return &launch_promoting_t<int16_t>;
        case HPT_I32: return &launch_promoting_t<int32_t>;
        case HPT_I64: return &launch_promoting_t<int64_t>;
        case HPT_U8: return &launch_promoting_t<uint8_t>;
        case HPT_U16: return &launch_promoting_t<uint16_t>;
        case HPT_U32: return &launch_promoting_t<uint32_t>;
        case HPT_U64: return &launch_promoting_t<uint64_t>;
        default: return nullptr;
    }
}

template <> NormLaunchFn norm_launcher<HPT_NORM_KIND>(int dtype) {
    switch (dtype) {
        case HPT_F16: return &launch_t<f16_t>;
        case HPT_BF16: return &launch_t<bf16_t>;
        case HPT_F32: return &launch_t<float>;
        case HPT_F64: return &launch_t<double>;
        default: return nullptr;
    }
}

}  // namespace hpt
