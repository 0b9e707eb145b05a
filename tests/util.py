"""Helpers shared by the parity tests: the same view (permute / slice) applied to a numpy
array and to a device tensor, dtype tables and tolerances."""
import numpy as np

F32_RTOL, F32_ATOL = 1e-5, 1e-6     # f32 against the f64-accumulating oracle
HALF_RTOL = 1e-2                    # f16 / bf16 against the f32-accumulating oracle


LONG_ROW = 65536


def half_acc(orc, n_reduced):
    """Which oracle mode is the truth for an f16 / bf16 row of `n_reduced` elements. The sequential f32
    sum (ACC_F32) restates "accumulated in f32" literally, but its own error grows with the row: beyond
    2^24 a running sum of squares moves in steps of 2 and comes out low by about a percent on millions
    of elements (see test_sequential_f32_accumulation_is_no_truth_for_long_half_rows). From 65536 elements
    on the truth is the f64 accumulation rounded once, which any f32 scheme with bounded error (the
    kernels' trees, pairwise sums) agrees with to half-precision rounding."""
    return orc.ACC_F64 if n_reduced > LONG_ROW else orc.ACC_F32


def half_atol(want, bits):
    """Absolute floor for half types: half an ulp (2^-bits relative) of the output's scale."""
    w = np.asarray(want, np.float64)
    w = w[np.isfinite(w)]
    scale = float(np.sqrt(np.mean(w * w))) if w.size else 0.0
    return scale * 2.0 ** (-bits)


def apply_view_np(a, ops):
    for kind, arg in ops:
        if kind == "permute":
            a = a.transpose(arg)
        elif kind == "slice":
            a = a[tuple(slice(*s) for s in arg)]
        else:
            raise ValueError(kind)
    return a


def apply_view_t(t, ops):
    for kind, arg in ops:
        if kind == "permute":
            t = t.permute(list(arg))
        elif kind == "slice":
            t = t[tuple(slice(*s) for s in arg)]
        else:
            raise ValueError(kind)
    return t


def upload(hpt, base, ops=(), dtype=None, dev=0):
    """Upload the contiguous `base` array and return (device view, numpy view) of the same layout."""
    t = hpt.Tensor.from_numpy(base, dtype).to_hip(dev)
    return apply_view_t(t, ops), apply_view_np(base, ops)


# the four layouts the reference's test rules demand (docs/dev_guide/test_rules.md:3-7):
# contiguous, permuted, sliced, sliced with a step
def layouts_for(shape, rng):
    nd = len(shape)
    out = [("contiguous", ())]
    if nd >= 2:
        perm = list(rng.permutation(nd))
        if perm == list(range(nd)):
            perm = perm[::-1]
        out.append(("permuted", (("permute", tuple(int(p) for p in perm)),)))
    sl = tuple((1 if s > 2 else 0, s - 1 if s > 3 else s, 1) for s in shape)
    out.append(("sliced", (("slice", sl),)))
    st = tuple((0, s, 2 if s > 1 else 1) for s in shape)
    out.append(("stepped", (("slice", st),)))
    return out
