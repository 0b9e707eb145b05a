"""Writes tests/golden/*.npz: inputs and expected outputs for the oracle and the GPU path.

The expected values come from PyTorch's CPU operators in float64 (torch.softmax,
torch.log_softmax, torch.nn.functional.layer_norm, sum/mean/amax/argmax): the library the
reference's own tests compare against (hpt-tests/src/hpt/cpu/reduce.rs:22-34,
hpt-tests/src/hpt/cpu/softmax.rs:12-23). PyTorch is a third-party library, not reference code.
Shapes follow the reference's tests: one per softmax kernel size class
(hpt-tests/src/hpt/cuda/normalization.rs:39-53), the [2,5,10] arange cases of
hpt-tests/src/hpt/cpu/reduce.rs:293-650, plus permuted / sliced / stepped views.

    python tests/golden/make_golden.py        # rewrites the fixtures (deterministic seeds)
"""
from pathlib import Path

import numpy as np
import torch

HERE = Path(__file__).resolve().parent


def views(a):
    """name -> (list of view ops, numpy view)"""
    out = {"contiguous": ([], a)}
    if a.ndim >= 2:
        perm = list(range(a.ndim))[::-1]
        out["permuted"] = ([("permute", perm)], a.transpose(perm))
    sl = [(1 if s > 2 else 0, s - 1 if s > 3 else s, 1) for s in a.shape]
    out["sliced"] = ([("slice", sl)], a[tuple(slice(*s) for s in sl)])
    st = [(0, s, 2 if s > 1 else 1) for s in a.shape]
    out["stepped"] = ([("slice", st)], a[tuple(slice(*s) for s in st)])
    return out


def main():
    rng = np.random.default_rng(12345)
    data = {}
    cases = []

    bases = {}

    def add(name, base, **arrays):
        # every distinct base array is stored once and referred to by number
        key = (base.ctypes.data, base.shape, str(base.dtype))
        if key not in bases:
            bases[key] = len(bases)
            data[f"base/{bases[key]}"] = np.ascontiguousarray(base)
        data[f"{name}/base_ref"] = np.array(bases[key])
        for k, v in arrays.items():
            data[f"{name}/{k}"] = np.array(v, order="C")
        cases.append(name)

    # ---- softmax / log_softmax: size classes and layouts ----
    for shape in ([1, 13], [2, 1024], [3, 1123], [3, 4096], [3, 5551], [6, 7, 5]):
        base = rng.uniform(-10, 10, shape).astype(np.float32)
        for lname, (ops, v) in views(base).items():
            if lname != "contiguous" and shape[-1] > 1200:
                continue
            tv = torch.from_numpy(np.ascontiguousarray(v)).double()
            for axis in range(v.ndim):
                add(f"softmax/{'x'.join(map(str, shape))}/{lname}/axis{axis}", base=base,
                    ops=np.array(repr(ops)), axis=np.array(axis),
                    softmax=torch.softmax(tv, axis).numpy(), log_softmax=torch.log_softmax(tv, axis).numpy())

    # ---- layernorm ----
    for shape, nn in (([5, 9], 1), ([4, 1024], 1), ([2, 4097], 1), ([3, 4, 6], 2), ([7, 1], 1)):
        base = (rng.standard_normal(shape) + rng.uniform(-5, 5, (shape[0],) + (1,) * (len(shape) - 1))).astype(np.float32)
        for lname, (ops, v) in views(base).items():
            if lname == "permuted":
                continue
            ns = list(v.shape[v.ndim - nn:])
            g = rng.normal(1, 0.1, ns).astype(np.float32)
            b = rng.normal(0, 0.1, ns).astype(np.float32)
            tv = torch.from_numpy(np.ascontiguousarray(v)).double()
            want = torch.nn.functional.layer_norm(tv, ns, torch.from_numpy(g).double(), torch.from_numpy(b).double(), 1e-5)
            want_plain = torch.nn.functional.layer_norm(tv, ns, None, None, 1e-5)
            add(f"layernorm/{'x'.join(map(str, shape))}/{lname}", base=base, ops=np.array(repr(ops)),
                n_norm=np.array(nn), gamma=g, beta=b, out=want.numpy(), out_plain=want_plain.numpy())

    # ---- reductions: the reference's [2,5,10] arange cases and random f32 / i32 ----
    ar = np.arange(100, dtype=np.float32).reshape(2, 5, 10)
    rnd = rng.standard_normal((6, 33, 10)).astype(np.float32)
    for tag, base in (("arange2x5x10", ar), ("randn6x33x10", rnd)):
        for lname, (ops, v) in views(base).items():
            tv = torch.from_numpy(np.ascontiguousarray(v)).double()
            for axes in ([0], [1], [2], [0, 1], [0, 2], [1, 2], [0, 1, 2]):
                add(f"reduce/{tag}/{lname}/axes{''.join(map(str, axes))}", base=base, ops=np.array(repr(ops)),
                    axes=np.array(axes), sum=tv.sum(axes).numpy(), mean=tv.mean(axes).numpy(),
                    max=tv.amax(axes).numpy(), min=tv.amin(axes).numpy(),
                    sum_square=(tv * tv).sum(axes).numpy(), reducel1=tv.abs().sum(axes).numpy(),
                    reducel2=(tv * tv).sum(axes).sqrt().numpy(),
                    reducel3=(tv.abs() ** 3).sum(axes).pow(1.0 / 3.0).numpy())
            for axis in range(3):
                add(f"argreduce/{tag}/{lname}/axis{axis}", base=base, ops=np.array(repr(ops)), axis=np.array(axis),
                    argmax=tv.argmax(axis).numpy(), argmin=tv.argmin(axis).numpy())
    # integer sums and tie-heavy arg-reductions (hpt-tests/src/hpt/cuda/reduce.rs:17-37, 1421-1612)
    ib = rng.integers(-1000, 1001, (5, 64, 12)).astype(np.int32)
    ties = rng.integers(-2, 3, (5, 64, 12)).astype(np.int32)
    for lname, (ops, v) in views(ib).items():
        tv = torch.from_numpy(np.ascontiguousarray(v))
        for axes in ([0], [1], [2], [0, 1, 2]):
            add(f"reduce_i32/{lname}/axes{''.join(map(str, axes))}", base=ib, ops=np.array(repr(ops)),
                axes=np.array(axes), sum=tv.sum(axes, dtype=torch.int32).numpy(), max=tv.amax(axes).numpy())
    for lname, (ops, v) in views(ties).items():
        for axis in range(3):
            # first extremum along the axis (numpy's rule, the reference's strict-compare scan)
            add(f"argreduce_i32_ties/{lname}/axis{axis}", base=ties, ops=np.array(repr(ops)), axis=np.array(axis),
                argmax=np.argmax(v, axis), argmin=np.argmin(v, axis))

    np.savez_compressed(HERE / "golden.npz", **data)
    (HERE / "cases.txt").write_text("\n".join(cases) + "\n")
    print(f"{len(cases)} cases, {sum(v.nbytes for v in data.values()) / 1e6:.1f} MB uncompressed")


if __name__ == "__main__":
    main()
