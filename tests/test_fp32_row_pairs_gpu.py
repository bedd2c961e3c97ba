"""Two to sixteen fp32 rows over whole weight blocks (the reference's kernels take fp32 activations,
tmq/tmq_cuda.cu:242-427, tmq/tmq.py:680-683): tmq_ternary_linear_ws splits them once into fp16 row pairs -- hi =
fp16(s x), lo = fp16(s x - hi), s the row's own power of two -- and runs the fp16 weight stream once over twice the
rows, adding each pair in the epilogue (nine to sixteen rows: two such passes over about half the rows each).

Seventeen rows or more take groups of eight rows, each group with a power of two of its own, laid out so that a row's
two terms sit in one 16-row MFMA fragment of whatever fp16 kernel the shape reaches; the epilogues add them.

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


@pytest.mark.parametrize("K,N", [(7, 100), (100, 520), (1000, 8200), (4100, 1000), (256, 520), (1024, 8200), (2048, 1000), (2304, 16), (4096, 4100), (6912, 520),
                                 (8192, 8200), (16384, 2064)])
@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 7, 8, 9, 11, 16])
def test_rows_against_fp64(cuda, oracle, M, K, N):
    from tmq_amd import ops, _capi
    print("fp32 row pairs", M, K, N, flush=True)
    rng = np.random.default_rng(M * 100000 + K + N)
    W, nw = _layer(cuda, oracle, rng, N, K)
    # one row over whole weight blocks, two over a small layer: the 8-bit GEMV splits them itself
    one_launch = K % 256 == 0 and ((M == 1 and K <= 16384) or (M == 2 and K <= 6144 and N <= 6144))
    Kp = (K + 255) // 256 * 256                                   # ragged lengths: written zero-padded to whole weight blocks
    assert _capi.load().tmq_ternary_linear_workspace_bytes(_capi.F32, M, K, N) == (0 if one_launch else 256 + 4 * M * Kp)
    x = rng.standard_normal((M, K)).astype(np.float32)
    ref = x.astype(np.float64) @ W.astype(np.float64).T
    t = lambda a: torch.from_numpy(a).to(cuda)
    y = ops.ternary_linear(t(x), nw)
    assert y.shape == (M, N) and y.dtype == torch.float32
    err = _row_err(y.cpu().numpy(), ref)
    assert err <= 1e-5, err
    y16 = ops.ternary_linear(t(x).half(), nw)
    assert K < 64 or err < 0.1 * _row_err(y16.cpu().numpy(), ref)
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


@pytest.mark.parametrize("K", [256, 1024, 2048, 2304, 4096, 5120, 6144])
def test_two_rows_over_small_layers_in_one_launch(cuda, oracle, K):
    """Two fp32 rows, K <= 6144, N <= 6144: sixteen term planes in the 8-bit GEMV, each row scaled by its own power of
    two inside the launch. Rows 60 orders of magnitude apart, a row of zeros, the C ABI without any workspace, and the
    neighbouring shape (N = 6160: fp16 row pairs) agree."""
    from tmq_amd import ops, _capi
    lib = _capi.load()
    rng = np.random.default_rng(K)
    for N in (16, 1000, 4100, 6144):
        W, nw = _layer(cuda, oracle, rng, N, K)
        x = rng.standard_normal((2, K)).astype(np.float32)
        x[0] *= np.float32(1e-30)
        x[1] *= np.float32(1e30)
        tx = torch.from_numpy(x).to(cuda)
        assert lib.tmq_fp32_rows_self_scaled_for(ops.ptr(tx), 2, K, N) == 1
        assert lib.tmq_fp32_rows_self_scaled(ops.ptr(tx), 2, K) == 0
        ref = x.astype(np.float64) @ W.astype(np.float64).T
        y = ops.ternary_linear(tx, nw)
        assert np.all(np.isfinite(y.cpu().numpy()))
        assert _row_err(y.cpu().numpy(), ref) <= 1e-5, (K, N)
        for m in range(2):                                       # each row is the single-row launch of that row
            assert torch.equal(ops.ternary_linear(tx[m:m + 1], nw)[0], y[m]), (K, N, m)
        ep = _capi.Epilogue(None, None, None, 0, _capi.F32)
        y2 = torch.empty_like(y)
        assert lib.tmq_ternary_linear(ops.ptr(tx), _capi.F32, 2, K, ops.ptr(nw.buf), N, ctypes.byref(ep), ops.ptr(y2), None) == 0
        torch.cuda.synchronize()
        assert torch.equal(y2, y)
        x[0] = 0.0
        y0 = ops.ternary_linear(torch.from_numpy(x).to(cuda), nw).cpu().numpy()
        assert np.array_equal(y0[0], np.zeros(N, np.float32)) and np.array_equal(y0[1], y[1].cpu().numpy())
    W, nw = _layer(cuda, oracle, rng, 6160, K)
    x = torch.from_numpy(rng.standard_normal((2, K)).astype(np.float32)).to(cuda)
    assert lib.tmq_fp32_rows_self_scaled_for(ops.ptr(x), 2, K, 6160) == 0
    small = ops.NativeWeights(torch.from_numpy(oracle.pack(W[:6144]).view(np.int32)).to(cuda), 6144)
    ya, yb = ops.ternary_linear(x, nw)[:, :6144], ops.ternary_linear(x, small)
    assert ((ya - yb).abs().max() / ya.abs().max()).item() <= 1e-5


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
    assert lib.tmq_ternary_linear_workspace_bytes(_capi.F32, 1, 4096, N) == 0         # a single row scales itself
    # a length that is no multiple of 256: the pairs are written zero-padded to whole weight blocks
    assert lib.tmq_ternary_linear_workspace_bytes(_capi.F32, 4, 4096 + 128, N) == 256 + 4 * 4 * 4352
    assert lib.tmq_ternary_linear_workspace_bytes(_capi.F32, 4, 100, N) == 256 + 4 * 4 * 256
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


# ---- seventeen rows or more: groups of eight rows, pairs inside one 16-row MFMA fragment -------------------------------
# (M, K, N): which fp16 kernel the 16 ceil(M / 8) rows reach
MANY = [
    (17, 4096, 4096),      # split reduction, 32 x 32 tiles
    (23, 1024, 1000),      # ragged N (a multiple of 4 and 8), M not a multiple of 8
    (64, 256, 72),         # the shortest reduction the path takes
    (100, 2304, 4100),     # N a multiple of 4 only
    (128, 576, 67),        # scalar stores (N odd)
    (256, 4096, 4096),     # split reduction, 64 x 64 tiles, eight wavefronts
    (300, 8192, 520),      # long reduction, narrow layer
    (1000, 1024, 1024),    # direct-to-LDS tiles
    (1024, 4096, 4096),    # 64 x 512 tiles, eight wavefronts
    (2048, 4096, 2048),    # 128 x 512 tiles
    (4096, 1024, 11008),   # 128 x 256 tiles, two workgroups per CU
]


@pytest.mark.parametrize("M,K,N", MANY)
def test_many_rows_against_fp64(cuda, oracle, M, K, N):
    from tmq_amd import ops, _capi
    print("fp32 row groups", M, K, N, flush=True)
    g = torch.Generator(device=cuda).manual_seed(M + K + N)
    W = torch.randint(-1, 2, (N, K), device=cuda, generator=g).to(torch.int8)
    words = torch.from_numpy(oracle.pack(W.float().cpu().numpy()).view(np.int32)).to(cuda)
    nw = ops.NativeWeights(words, N)
    groups = (M + 7) // 8
    assert _capi.load().tmq_ternary_linear_workspace_bytes(_capi.F32, M, K, N) == (4 * groups + 255) // 256 * 256 + 32 * groups * K
    x = torch.randn((M, K), device=cuda, generator=g)
    # every group of eight rows its own magnitude: the groups are scaled separately
    x *= (2.0 ** torch.randint(-40, 40, (groups, 1), device=cuda, generator=g).float()).repeat_interleave(8, 0)[:M]
    Wd = W.double()
    ref = x.double() @ Wd.t()
    rows = lambda got, want: float(((got.double() - want).abs().amax(1) / want.abs().amax(1).clamp_min(1e-300)).max())
    y = ops.ternary_linear(x, nw)
    assert y.shape == (M, N) and y.dtype == torch.float32
    err = rows(y, ref)
    assert err <= 1e-5, err
    assert torch.equal(ops.ternary_linear(x, nw), y)
    scale = torch.rand(N, device=cuda, generator=g) + 0.5
    bias = torch.randn(N, device=cuda, generator=g)
    res = torch.randn((M, N), device=cuda, generator=g) * ref.abs().amax(1, keepdim=True).float()
    full = ref * scale.double() + bias.double()
    y2 = ops.ternary_linear(x, nw, scale, bias, residual=res, relu=True)
    assert rows(y2, torch.relu(full + res.double())) <= 1e-5
    # fp16 output (the wide-row epilogue where N is a multiple of 8): rows of order one
    x1 = torch.randn((M, K), device=cuda, generator=g)
    ref1 = (x1.double() @ Wd.t()) * (scale.double() / K ** 0.5) + bias.double()
    res16 = torch.randn((M, N), device=cuda, generator=g).half()
    y3 = ops.ternary_linear(x1, nw, scale / K ** 0.5, bias, residual=res16, out_dtype=torch.float16)
    assert y3.dtype == torch.float16 and rows(y3, ref1 + res16.double()) <= 1e-3


def test_many_rows_22_bit_values_pass_through_exactly(cuda, oracle):
    from tmq_amd import ops
    K = N = 1024
    nw = ops.NativeWeights(torch.from_numpy(oracle.pack(np.eye(N, dtype=np.float32)).view(np.int32)).to(cuda), N)
    rng = np.random.default_rng(21)
    M = 77
    x = rng.integers(-(1 << 21), 1 << 21, size=(M, K)).astype(np.float32)
    x[:, :4] = [0.0, -0.0, 1.0, -1.0]
    x *= np.repeat((2.0 ** rng.integers(-60, 60, size=((M + 7) // 8, 1))).astype(np.float32), 8, axis=0)[:M]
    y = ops.ternary_linear(torch.from_numpy(x).to(cuda), nw).cpu().numpy()
    assert np.array_equal(y, x)


def test_many_rows_workspace_rules_and_graph_replay(cuda, oracle):
    from tmq_amd import ops, _capi
    lib = _capi.load()
    M, K, N = 200, 1024, 520
    assert lib.tmq_ternary_linear_workspace_bytes(_capi.F32, 200, 128, N) == 256 + 32 * 25 * 128   # short reductions as well
    # a length that is no multiple of 64: the pairs are written as zero-padded rows of the next multiple (test_ragged_rows_gpu.py)
    assert lib.tmq_ternary_linear_workspace_bytes(_capi.F32, 200, 1024 + 32, N) == 256 + 32 * 25 * 1088
    g = torch.Generator(device=cuda).manual_seed(8)
    W = torch.randint(-1, 2, (N, K), device=cuda, generator=g).to(torch.int8)
    nw = ops.NativeWeights(ops.compactify_ternary(W), N)
    x = torch.randn((M, K), device=cuda, generator=g)
    ref = x.double() @ W.double().t()
    ep = _capi.Epilogue(None, None, None, 0, _capi.F32)
    need = lib.tmq_ternary_linear_workspace_bytes(_capi.F32, M, K, N)
    ws = torch.empty(need, dtype=torch.uint8, device=cuda)
    for wptr, wbytes in ((ops.ptr(ws), need), (None, 0), (ops.ptr(ws), need - 1)):
        y = torch.empty((M, N), dtype=torch.float32, device=cuda)
        assert lib.tmq_ternary_linear_ws(ops.ptr(x), _capi.F32, M, K, ops.ptr(nw.buf), N, ctypes.byref(ep), ops.ptr(y),
                                         wptr, wbytes, None) == 0
        torch.cuda.synchronize()
        assert ((y.double() - ref).abs().max() / ref.abs().max()).item() <= 1e-5
    eager = ops.ternary_linear(x, nw)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        ops.ternary_linear(x, nw)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            out = ops.ternary_linear(x, nw)
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
