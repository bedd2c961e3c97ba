"""Two to sixteen fp32 rows over whole weight blocks (the reference's kernels take fp32 activations,
tmq/tmq_cuda.cu:242-427, tmq/tmq.py:680-683): tmq_ternary_linear_ws splits them once into fp16 row pairs -- hi =
fp16(s x), lo = fp16(s x - hi), s the row's own power of two -- and runs the fp16 weight stream once over twice the
rows, adding each pair in the epilogue (nine to sixteen rows: two such passes over about half the rows each).

Bar: 1e-5 of each row's largest output against an fp64 product of the expanded weights (22 significant bits per
value; a single fp16 rounding of the row is ~100 times worse), rows of any magnitude side by side, 22-bit integers
through identity weights exactly, every epilogue, and the plain entry point when the workspace is missing.
"""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _layer(cuda, oracle, rng, N, K):
    from tmq_amd import ops
    W = rng.integers(-1, 2, size=(N, K)).astype(np.float32)
    return W, ops.NativeWeights(torch.from_numpy(oracle.pack(W).view(np.int32)).to(cuda), N)


def _row_err(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float(np.max(np.max(np.abs(got - want), axis=1) / np.maximum(1e-300, np.max(np.abs(want), axis=1))))


@pytest.mark.parametrize("K,N", [(2048, 1000), (2304, 16), (4096, 4100), (6912, 520), (8192, 8200), (16384, 2064)])
@pytest.mark.parametrize("M", [2, 3, 4, 5, 7, 8, 9, 11, 16])
def test_rows_against_fp64(cuda, oracle, M, K, N):
    from tmq_amd import ops, _capi
    print("fp32 row pairs", M, K, N, flush=True)
    rng = np.random.default_rng(M * 100000 + K + N)
    W, nw = _layer(cuda, oracle, rng, N, K)
    assert _capi.load().tmq_ternary_linear_workspace_bytes(_capi.F32, M, K, N) == 256 + 4 * M * K
    x = rng.standard_normal((M, K)).astype(np.float32)
    ref = x.astype(np.float64) @ W.astype(np.float64).T
    t = lambda a: torch.from_numpy(a).to(cuda)
    y = ops.ternary_linear(t(x), nw)
    assert y.shape == (M, N) and y.dtype == torch.float32
    err = _row_err(y.cpu().numpy(), ref)
    assert err <= 1e-5, err
    y16 = ops.ternary_linear(t(x).half(), nw)
    assert err < 0.1 * _row_err(y16.cpu().numpy(), ref)
    assert torch.equal(ops.ternary_linear(t(x), nw), y)          # run to run identical
    # every epilogue
    scale = (0.5 + rng.random(N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    res = rng.standard_normal((M, N)).astype(np.float32)
    full = ref * scale + bias
    y2 = ops.ternary_linear(t(x), nw, t(scale), t(bias), residual=t(res), relu=True)
    assert _row_err(y2.cpu().numpy(), np.maximum(full + res, 0)) <= 1e-5
    y3 = ops.ternary_linear(t(x), nw, t(scale), t(bias), residual=t(res.astype(np.float16)), relu=False, out_dtype=torch.float16)
    assert _row_err(y3.float().cpu().numpy(), full + res.astype(np.float16)) <= 1e-3


def test_rows_of_any_magnitude_side_by_side(cuda, oracle):
    """Each row is scaled by its own power of two: a row of 1e-30s loses nothing next to a row of 1e30s; zeros,
    a row of zeros and the sign of zero survive."""
    from tmq_amd import ops
    K, N, M = 4096, 1000, 6
    rng = np.random.default_rng(77)
    W, nw = _layer(cuda, oracle, rng, N, K)
    x = rng.standard_normal((M, K)).astype(np.float32)
    for m, s in enumerate((1e-30, 1e30, 1.0, 3e-12, 7e18)):
        x[m] *= np.float32(s)
    x[5] = 0.0
    x[2, :100] = 0.0
    ref = x.astype(np.float64) @ W.astype(np.float64).T
    y = ops.ternary_linear(torch.from_numpy(x).to(cuda), nw).cpu().numpy()
    assert np.all(np.isfinite(y))
    assert _row_err(y[:5], ref[:5]) <= 1e-5
    assert np.array_equal(y[5], np.zeros(N, np.float32))


@pytest.mark.parametrize("M", [2, 5, 8, 13])
def test_22_bit_values_pass_through_exactly(cuda, oracle, M):
    from tmq_amd import ops
    K = N = 2048
    nw = ops.NativeWeights(torch.from_numpy(oracle.pack(np.eye(N, dtype=np.float32)).view(np.int32)).to(cuda), N)
    rng = np.random.default_rng(M)
    x = rng.integers(-(1 << 21), 1 << 21, size=(M, K)).astype(np.float32)
    x[:, :4] = [0.0, -0.0, 1.0, -1.0]
    x *= (2.0 ** rng.integers(-60, 60, size=(M, 1))).astype(np.float32)      # every row its own magnitude
    y = ops.ternary_linear(torch.from_numpy(x).to(cuda), nw).cpu().numpy()
    assert np.array_equal(y, x)


def test_c_abi_workspace_rules_and_graph_replay(cuda, oracle):
    """Shapes outside the path report no workspace; a missing or short workspace gives tmq_ternary_linear's result;
    replays of a captured call equal the eager one."""
    from tmq_amd import ops, _capi
    lib = _capi.load()
    K, N, M = 4096, 520, 12
    for m, k in ((1, 4096), (17, 4096), (4, 4096 + 128), (4, 1024)):
        assert lib.tmq_ternary_linear_workspace_bytes(_capi.F32, m, k, N) == 0
    rng = np.random.default_rng(3)
    W, nw = _layer(cuda, oracle, rng, N, K)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(cuda)
    ref = x.double() @ torch.from_numpy(W).to(cuda).double().t()
    ep = _capi.Epilogue(None, None, None, 0, _capi.F32)
    need = lib.tmq_ternary_linear_workspace_bytes(_capi.F32, M, K, N)
    ws = torch.empty(need, dtype=torch.uint8, device=cuda)
    outs = []
    for wptr, wbytes in ((ops.ptr(ws), need), (None, 0), (ops.ptr(ws), need - 1)):
        y = torch.empty((M, N), dtype=torch.float32, device=cuda)
        assert lib.tmq_ternary_linear_ws(ops.ptr(x), _capi.F32, M, K, ops.ptr(nw.buf), N, ctypes.byref(ep), ops.ptr(y),
                                         wptr, wbytes, None) == 0
        torch.cuda.synchronize()
        assert ((y.double() - ref).abs().max() / ref.abs().max()).item() <= 1e-5
        outs.append(y)
    assert torch.equal(outs[1], outs[2])
    eager = ops.ternary_linear(x, nw)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        ops.ternary_linear(x, nw)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            out = ops.ternary_linear(x, nw)
    for _ in range(3):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
