"""17 .. 32 activation rows over a very large layer with a workspace: the reduction cut across workgroups
(rows_split_kernel + the ordered sum of the slices), against an fp64 product of the same operands
(a11: tmq/tmq_cuda.cu:478-549 computes these sums in fp32), through every epilogue, ragged rows / channels /
block counts, and the C ABI's contract for the workspace (absent or too small: the plain call's result).
"""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _case(cuda, M, K, N, seed):
    g = torch.Generator(device=cuda).manual_seed(seed)
    W = torch.randint(-1, 2, (N, K), device=cuda, generator=g, dtype=torch.int8)
    x = torch.randn((M, K), device=cuda, generator=g).half()
    return W, x


@pytest.mark.parametrize("M,K,N", [(17, 16384, 16384), (32, 16384, 16384), (24, 16640, 16400), (32, 8192, 32768), (20, 34048, 8208),
                                   (31, 4096, 65536)])
def test_rows_over_a_large_layer(cuda, M, K, N):
    from tmq_amd import ops, _capi
    lib = _capi.load()
    assert lib.tmq_ternary_linear_workspace_bytes(_capi.F16, M, K, N) > 0       # these shapes take the split kernel
    W, x = _case(cuda, M, K, N, M + K + N)
    nw = ops.NativeWeights(ops.compactify_ternary(W), N)
    ref = x.double() @ W.double().t()
    y = ops.ternary_linear(x, nw)
    err = ((y.double() - ref).abs().max() / ref.abs().max()).item()
    assert y.shape == (M, N) and err <= 2e-5, err
    assert torch.equal(ops.ternary_linear(x, nw), y)                            # run to run identical
    scale = 0.5 + torch.rand(N, device=cuda)
    bias = torch.randn(N, device=cuda)
    res = torch.randn(M, N, device=cuda)
    y2 = ops.ternary_linear(x, nw, scale, bias, residual=res, relu=True)
    ref2 = (ref * scale.double() + bias.double() + res.double()).clamp_min(0)
    assert ((y2.double() - ref2).abs().max() / ref2.abs().max()).item() <= 2e-5
    y3 = ops.ternary_linear(x, nw, scale, None, residual=res.half(), relu=False, out_dtype=torch.float16)
    ref3 = ref * scale.double() + res.half().double()
    assert ((y3.double() - ref3).abs().max() / ref3.abs().max()).item() <= 2e-3
    # small integers: exact whatever the order of the slices
    xi = torch.randint(-4, 5, (M, K), device=cuda).half()
    yi = ops.ternary_linear(xi, nw)
    assert torch.equal(yi.double(), xi.double() @ W.double().t())


def test_workspace_contract(cuda):
    """A missing or short workspace gives the plain call's values; shapes outside the kernel's range ask for none."""
    from tmq_amd import ops, _capi
    lib = _capi.load()
    M, K, N = 28, 16384, 16384
    W, x = _case(cuda, M, K, N, 5)
    nw = ops.NativeWeights(ops.compactify_ternary(W), N)
    need = lib.tmq_ternary_linear_workspace_bytes(_capi.F16, M, K, N)
    assert need >= 2 * M * N * 4
    for Mx, Kx, Nx in ((16, 16384, 16384), (33, 16384, 16384), (28, 2048, 131072), (28, 16384, 16392), (28, 8192, 8192)):
        assert lib.tmq_ternary_linear_workspace_bytes(_capi.F16, Mx, Kx, Nx) == 0, (Mx, Kx, Nx)
    # a ragged length asks for the rows' padded copy instead (test_ragged_rows_gpu.py)
    assert lib.tmq_ternary_linear_workspace_bytes(_capi.F16, 28, 16392, 16384) == 2 * 28 * 16448
    # fp32 rows use the workspace for their fp16 row pairs, not for partial sums (test_fp32_row_pairs_gpu.py)
    assert lib.tmq_ternary_linear_workspace_bytes(_capi.F32, M, K, N) == 256 + 32 * ((M + 7) // 8) * K
    ep = _capi.Epilogue()
    ep.y_dtype = _capi.F32
    outs = []
    for ws_bytes in (need, need - 16, 0):
        y = torch.full((M, N), float("nan"), device=cuda)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=cuda)
        _capi.check(lib.tmq_ternary_linear_ws(_capi.ptr(x), _capi.F16, M, K, _capi.ptr(nw.buf), N, ctypes.byref(ep), _capi.ptr(y),
                                              _capi.ptr(ws) if ws_bytes else None, ws_bytes, _capi.stream_of(x)), "linear_ws")
        torch.cuda.synchronize()
        outs.append(y)
    ref = x.double() @ W.double().t()
    for y in outs:
        assert ((y.double() - ref).abs().max() / ref.abs().max()).item() <= 2e-5
    assert torch.equal(outs[1], outs[2])                                        # both took the single-launch kernel


def test_graph_replays_equal_eager(cuda):
    from tmq_amd import ops
    M, K, N = 32, 16384, 16384
    W, x = _case(cuda, M, K, N, 9)
    nw = ops.NativeWeights(ops.compactify_ternary(W), N)
    eager = ops.ternary_linear(x, nw).clone()
    torch.cuda.synchronize()
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        y = torch.empty(M, N, device=cuda)
        with torch.cuda.graph(graph, stream=side):
            y.copy_(ops.ternary_linear(x, nw))
    for rep in range(3):
        y.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), rep
        ops.ternary_linear(torch.randn_like(x), nw)
        torch.cuda.synchronize()
