"""Seventeen fp16 rows or more whose reduction length is no multiple of 64 (the reference's kernels take any K,
tmq/tmq_cuda.cu:289-427, host 478-549): with a workspace tmq_ternary_linear_ws copies the rows once to rows of the
next multiple of 64, zeros behind, and runs the kernels that want whole tiles; without one the guarded kernel runs.

fp32 rows of such lengths (seventeen or more) are split into fp16 row pairs that are written padded the same way.

Bar: both routes against an fp64 product of the expanded weights (fp16 inputs, fp32 accumulation: 2e-5 of the largest
output), exact on small integers, every epilogue, rows that are not 16-byte aligned, and the workspace rules of the ABI.
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


@pytest.mark.parametrize("K", [65, 100, 520, 784, 1000, 4000, 4100])
@pytest.mark.parametrize("M,N", [(17, 1000), (128, 520), (300, 4100), (1030, 64)])
def test_ragged_lengths_against_fp64(cuda, oracle, M, N, K):
    from tmq_amd import ops, _capi
    rng = np.random.default_rng(M + N + K)
    W, nw = _layer(cuda, oracle, rng, N, K)
    Kp = (K + 63) // 64 * 64
    assert _capi.load().tmq_ternary_linear_workspace_bytes(_capi.F16, M, K, N) == 2 * M * Kp
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float16)).to(cuda)
    Wd = torch.from_numpy(W).to(cuda).double()
    ref = x.double() @ Wd.t()
    y = ops.ternary_linear(x, nw)
    assert ((y.double() - ref).abs().max() / ref.abs().max()).item() <= 2e-5
    assert torch.equal(ops.ternary_linear(x, nw), y)
    scale = torch.from_numpy((0.5 + rng.random(N)).astype(np.float32)).to(cuda)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(cuda)
    res = torch.from_numpy(rng.standard_normal((M, N)).astype(np.float16)).to(cuda)
    y2 = ops.ternary_linear(x, nw, scale, bias, residual=res, relu=True, out_dtype=torch.float16)
    ref2 = torch.clamp_min(ref * scale.double() + bias.double() + res.double(), 0)
    assert ((y2.double() - ref2).abs().max() / ref2.abs().max()).item() <= 1e-3
    xi = torch.from_numpy(rng.integers(-8, 9, size=(M, K)).astype(np.float16)).to(cuda)
    assert torch.equal(ops.ternary_linear(xi, nw).double(), xi.double() @ Wd.t())      # integers: exact whatever the order


@pytest.mark.parametrize("K", [7, 64, 100, 257, 520, 784, 1000, 4000, 4100])
@pytest.mark.parametrize("M,N", [(17, 1000), (128, 520), (300, 4100), (1030, 64)])
def test_ragged_fp32_rows_against_fp64(cuda, oracle, M, N, K):
    """fp32 rows (the reference's convention) of such lengths: split into fp16 row pairs in groups of eight, written as
    zero-padded rows of whole tiles; 22 significant bits, groups of any magnitude side by side."""
    from tmq_amd import ops, _capi
    rng = np.random.default_rng(M + N + K + 1)
    W, nw = _layer(cuda, oracle, rng, N, K)
    Kp = (K + 63) // 64 * 64
    groups = (M + 7) // 8
    assert _capi.load().tmq_ternary_linear_workspace_bytes(_capi.F32, M, K, N) == (4 * groups + 255) // 256 * 256 + 32 * groups * Kp
    x = rng.standard_normal((M, K)).astype(np.float32)
    x[:8] *= np.float32(1e-25)
    x[8:16] *= np.float32(1e25)
    x = torch.from_numpy(x).to(cuda)
    Wd = torch.from_numpy(W).to(cuda).double()
    ref = x.double() @ Wd.t()
    y = ops.ternary_linear(x, nw)
    err = ((y.double() - ref).abs().amax(1) / ref.abs().amax(1)).max().item()
    assert err <= 1e-5, err
    assert torch.isfinite(y).all()
    xi = torch.from_numpy(rng.integers(-(1 << 20), 1 << 20, size=(M, K)).astype(np.float32)).to(cuda)
    scale = torch.from_numpy((0.5 + rng.random(N)).astype(np.float32)).to(cuda)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(cuda)
    res = torch.from_numpy(rng.standard_normal((M, N)).astype(np.float32)).to(cuda)
    y2 = ops.ternary_linear(xi, nw, scale, bias, residual=res, relu=True)
    ref2 = torch.clamp_min((xi.double() @ Wd.t()) * scale.double() + bias.double() + res.double(), 0)
    assert ((y2.double() - ref2).abs().max() / ref2.abs().max()).item() <= 1e-5
    # rows that do not start on 16 bytes (the C ABI; the bindings only take the route for aligned tensors)
    lib = _capi.load()
    flat = torch.zeros(M * K + 4, dtype=torch.float32, device=cuda)
    flat[1:1 + M * K] = x.reshape(-1)
    xs = flat[1:1 + M * K].view(M, K)
    need = lib.tmq_ternary_linear_workspace_bytes(_capi.F32, M, K, N)
    ws = torch.empty(need, dtype=torch.uint8, device=cuda)
    ep = _capi.Epilogue(None, None, None, 0, _capi.F32)
    y3 = torch.empty((M, N), dtype=torch.float32, device=cuda)
    assert lib.tmq_ternary_linear_ws(ops.ptr(xs), _capi.F32, M, K, ops.ptr(nw.buf), N, ctypes.byref(ep), ops.ptr(y3),
                                     ops.ptr(ws), need, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(y3, y)


def test_workspace_rules_unaligned_rows_and_graph_replay(cuda, oracle):
    """A missing or short workspace gives tmq_ternary_linear's values; rows that start at an odd element take the
    element-wise copy; shapes outside the route ask for nothing; replays of a captured call equal the eager one."""
    from tmq_amd import ops, _capi
    lib = _capi.load()
    for m, k in ((16, 1000), (17, 1024), (1, 100), (64, 4096)):
        assert lib.tmq_ternary_linear_workspace_bytes(_capi.F16, m, k, 1000) == 0
    rng = np.random.default_rng(21)
    M, K, N = 70, 1000, 520
    W, nw = _layer(cuda, oracle, rng, N, K)
    Wd = torch.from_numpy(W).to(cuda).double()
    flat = torch.from_numpy(rng.integers(-8, 9, size=(M * K + 8,)).astype(np.float16)).to(cuda)
    ep = _capi.Epilogue(None, None, None, 0, _capi.F32)
    need = lib.tmq_ternary_linear_workspace_bytes(_capi.F16, M, K, N)
    ws = torch.empty(need, dtype=torch.uint8, device=cuda)
    for shift in (0, 1, 3):                                         # 16-byte aligned rows, then rows at odd elements
        x = flat[shift:shift + M * K].view(M, K)
        ref = x.double() @ Wd.t()
        for wptr, wbytes in ((ops.ptr(ws), need), (None, 0), (ops.ptr(ws), need - 1)):
            y = torch.full((M, N), float("nan"), dtype=torch.float32, device=cuda)
            assert lib.tmq_ternary_linear_ws(ops.ptr(x), _capi.F16, M, K, ops.ptr(nw.buf), N, ctypes.byref(ep), ops.ptr(y),
                                             wptr, wbytes, None) == 0
            torch.cuda.synchronize()
            assert torch.equal(y.double(), ref), (shift, wbytes)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float16)).to(cuda)
    eager = ops.ternary_linear(x, nw).clone()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        out = torch.empty_like(eager)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=s):
            out.copy_(ops.ternary_linear(x, nw))
    for rep in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), rep
        ops.ternary_linear(torch.randn_like(x), nw)                 # eager work on the same weights in between
        torch.cuda.synchronize()


def test_reference_binding_takes_the_route(cuda, oracle):
    """ternary_mmm_cuda (the reference's binding name, through the extension when it is built) on a ragged length."""
    import tmq_amd
    from tmq_amd import ops
    rng = np.random.default_rng(5)
    M, K, N = 96, 784, 300
    W = rng.integers(-1, 2, size=(N, K)).astype(np.float32)
    words = torch.from_numpy(oracle.pack(W).view(np.int32)).to(cuda)
    x = torch.from_numpy(rng.integers(-8, 9, size=(M, K)).astype(np.float16)).to(cuda)
    y = ops.ternary_mmm_cuda(x, words, N)
    assert torch.equal(y.double(), x.double() @ torch.from_numpy(W).to(cuda).double().t())
