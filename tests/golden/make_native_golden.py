"""Writes tests/golden/native_golden.npz from the reference's own host code.

Run in the build container only (needs oracle/_ref/tmq_native.so, built by `make -C oracle ref`
from the reference's tmq/tmq_native.cpp where it lies). The fixture holds data only: seeded ternary
tensors, the compact words and the range-coded streams the reference produces for them, and its
expansion back to fp32. The GPU box has no reference tree; tests there read this file.

    python3 tests/golden/make_native_golden.py
"""
import importlib.util
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))


def load_ref():
    path = os.path.join(ROOT, "oracle", "_ref", "tmq_native.so")
    spec = importlib.util.spec_from_file_location("tmq_native", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def ternary(gen, shape, p0):
    u = torch.rand(shape, generator=gen)
    return torch.where(u < (1 - p0) / 2, 1.0, torch.where(u < 1 - p0, -1.0, 0.0))


def main():
    ref = load_ref()
    gen = torch.Generator().manual_seed(1234)
    out = {}
    cases = [((16, 1), .5), ((6, 5), .5), ((17, 3), .3), ((102, 64), .5), ((64, 147), .5), ((33, 65), .9),
             ((48, 20), 0.0), ((20, 5, 3, 2), .5), ((64, 3, 7, 7), .5), ((10, 16, 1, 1), .7)]
    for i, (shape, p0) in enumerate(cases):
        w = ternary(gen, shape, p0)
        compact = ref.compactify_ternary(w)
        stream = ref.compress_ternary(w, list(shape), False)
        stream2 = ref.compress_ternary(compact, list(shape), True)
        assert torch.equal(stream, stream2)
        back = ref.decompress_ternary(stream, list(shape))
        assert torch.equal(back, compact)
        out[f"w{i}"] = w.numpy()
        out[f"compact{i}"] = compact.numpy()
        out[f"stream{i}"] = stream.numpy()
        # The reference's 2-D expander reads rows*ceil(cols/16) words of a buffer that holds
        # cols*ceil(rows/16); only keep its output where that stays inside the buffer.
        in_bounds = len(shape) == 4 or shape[0] * ((shape[1] + 15) // 16) <= compact.numel()
        if in_bounds:
            out[f"expand{i}"] = ref.expand_ternary(compact, list(shape), False).numpy()
    # float rounding / clamping and integer inputs
    v = torch.tensor([0.5, -0.5, 0.49999997, -0.49999997, 1.5, -1.5, 2.5, -2.5, 0.0, -0.0, 1e-30, 7.0, -7.0, 3e9, -3e9,
                      float("inf"), float("-inf"), float("nan"), 2147483520.0, 2147483648.0, 0.50000006, 1e38])
    wf = torch.zeros(32, 3)
    wf[:v.numel(), 1] = v
    out["round_in"] = wf.numpy()
    out["round_compact"] = ref.compactify_ternary(wf).numpy()
    wi8 = torch.zeros(16, 2, dtype=torch.int8)
    wi8[:9, 0] = torch.tensor([0, 1, -1, 2, -2, 127, -128, 5, -5], dtype=torch.int8)
    out["i8_in"] = wi8.numpy()
    out["i8_compact"] = ref.compactify_ternary(wi8).numpy()
    wi32 = torch.zeros(16, 2, dtype=torch.int32)
    wi32[:7, 1] = torch.tensor([0, 1, -1, 2 ** 31 - 1, -2 ** 31, 70000, -70000], dtype=torch.int32)
    out["i32_in"] = wi32.numpy()
    out["i32_compact"] = ref.compactify_ternary(wi32).numpy()
    out["ncases"] = np.array(len(cases))
    np.savez_compressed(os.path.join(HERE, "native_golden.npz"), **out)
    print("wrote native_golden.npz with", len(out), "arrays")


if __name__ == "__main__":
    main()
