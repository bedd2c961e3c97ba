"""GPU parity of the MFMA tile kernel (large-M linear and implicit-GEMM convolution) vs the oracle."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _ternary(rng, shape, p0=0.5):
    u = rng.random(shape)
    return np.where(u < (1 - p0) / 2, 1.0, np.where(u < 1 - p0, -1.0, 0.0)).astype(np.float32)


def _rel_err(got, want):
    want = np.asarray(want, np.float64)
    got = np.asarray(got, np.float64)
    return np.max(np.abs(got - want)) / max(1e-30, np.max(np.abs(want)))


GEMM_SHAPES = [(65, 64, 16), (128, 512, 64), (256, 4096, 256), (300, 147, 64), (1000, 576, 128), (513, 1000, 130),
               (4096, 512, 512), (777, 2304, 256), (3136, 256, 102), (2048, 64, 64),
               # few rows over a long reduction: the weight-stream kernel with every epilogue
               (4, 2048, 520), (16, 2304, 1000), (1, 4096, 96),
               # 192 .. 1023 tiles of 64 x 256 over a long reduction: the kernel that issues its loads and weight
               # expansion between the MFMAs (three-pass ring, counted waits); K = 256 b + 64 r exercises the
               # partial last weight block with r = 1, 2, 3 tiles, ragged M and N the clamped rows / channels
               (1024, 4096, 4096), (800, 1088, 4000), (777, 1152, 3900), (1500, 1216, 2100), (3072, 1024, 1024),
               (13000, 1280, 130)]


@pytest.mark.parametrize("M,K,N", GEMM_SHAPES)
def test_large_m_linear(cuda, oracle, M, K, N):
    from tmq_amd import ops
    rng = np.random.default_rng(M + 3 * K + 5 * N)
    W = _ternary(rng, (N, K))
    words = oracle.pack(W)
    x = rng.standard_normal((M, K)).astype(np.float16)
    scale = (0.5 + rng.random(N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    nw = ops.NativeWeights(torch.from_numpy(words.view(np.int32)).to(cuda), N)
    tx = torch.from_numpy(x).to(cuda)
    ts, tb = torch.from_numpy(scale).to(cuda), torch.from_numpy(bias).to(cuda)
    y = ops.ternary_linear(tx, nw, ts, tb)
    ref = (x.astype(np.float64) @ W.astype(np.float64).T) * scale + bias
    assert _rel_err(y.cpu().numpy(), ref) <= 1e-3
    assert _rel_err(y.cpu().numpy(), ref) <= 3e-6
    # exact on small integers, whatever the summation order
    xi = rng.integers(-4, 5, (M, K)).astype(np.float16)
    yi = ops.ternary_linear(torch.from_numpy(xi).to(cuda), nw).cpu().numpy()
    assert np.array_equal(yi, (xi.astype(np.int64) @ W.astype(np.int64).T).astype(np.float32))
    # fused epilogue: residual + relu, fp32 and fp16 outputs
    res = torch.from_numpy(rng.standard_normal((M, N)).astype(np.float32)).to(cuda)
    y2 = ops.ternary_linear(tx, nw, ts, tb, residual=res, relu=True)
    assert _rel_err(y2.cpu().numpy(), np.maximum(ref + res.cpu().numpy(), 0)) <= 3e-6
    y3 = ops.ternary_linear(tx, nw, ts, tb, residual=res.half(), relu=True, out_dtype=torch.float16)
    want3 = np.maximum(ref + res.half().cpu().numpy().astype(np.float64), 0)
    assert _rel_err(y3.float().cpu().numpy(), want3) <= 1e-3


def test_mid_size_kernel_is_deterministic_and_replays_in_a_graph(cuda, oracle):
    """M = 1024, K = N = 2048 (256 tiles of 64 x 256: the kernel with hand-counted waits): the same bits on every
    run, eager and as replays of a HIP graph with eager work in between."""
    from tmq_amd import ops
    rng = np.random.default_rng(21)
    M, K, N = 1024, 2048, 2048
    W = _ternary(rng, (N, K))
    nw = ops.NativeWeights(torch.from_numpy(oracle.pack(W).view(np.int32)).to(cuda), N)
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float16)).to(cuda)
    eager = ops.ternary_linear(x, nw).clone()
    ref = x.cpu().numpy().astype(np.float64) @ W.astype(np.float64).T
    assert _rel_err(eager.cpu().numpy(), ref) <= 3e-6
    for _ in range(3):
        assert torch.equal(ops.ternary_linear(x, nw), eager)
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


# 128 x 512 tiles, one k-tile per pass: whole weight blocks, then a last block of 1 and of 3 tiles (the third is fetched
# in the tail); 64 x 512 tiles (2000 x 4096: 256 of them)
@pytest.mark.parametrize("M,K,N", [(4100, 2048, 4096), (4096, 2112, 4608), (4096, 2240, 4096), (2000, 1280, 4096)])
def test_full_chip_of_wide_tiles_against_fp64_on_the_gpu(cuda, oracle, M, K, N):
    """At least 256 tiles of 128 x 512 over a long reduction: eight-wavefront workgroups. Too large for a CPU
    reference in a unit test: checked against the GPU's fp64 matrix product of the expanded weights (a library
    routine that shares nothing with these kernels), with ragged rows and every epilogue."""
    from tmq_amd import ops
    g = torch.Generator(device="cpu").manual_seed(M + K)
    W = torch.randint(-1, 2, (N, K), generator=g, dtype=torch.int8)
    nw = ops.NativeWeights(torch.from_numpy(oracle.pack(W.numpy().astype(np.float32)).view(np.int32)).to(cuda), N)
    x = torch.randn(M, K, generator=g).half().to(cuda)
    scale = (0.5 + torch.rand(N, generator=g)).to(cuda)
    bias = torch.randn(N, generator=g).to(cuda)
    ref = (x.double() @ W.to(cuda).double().t()) * scale.double() + bias.double()
    y = ops.ternary_linear(x, nw, scale, bias)
    assert ((y.double() - ref).abs().max() / ref.abs().max()).item() <= 3e-6
    res = torch.randn(M, N, generator=g).half().to(cuda)
    y2 = ops.ternary_linear(x, nw, scale, bias, residual=res, relu=True, out_dtype=torch.float16)
    want = (ref + res.double()).clamp_min(0)
    assert ((y2.double() - want).abs().max() / want.abs().max()).item() <= 1e-3
    xi = torch.randint(-4, 5, (M, K), generator=g).half().to(cuda)
    yi = ops.ternary_linear(xi, nw)
    assert torch.equal(yi.double(), xi.double() @ W.to(cuda).double().t())        # integers: exact


def test_skinny_and_tile_kernels_agree(cuda, oracle):
    """M = 64 (skinny kernel) and M = 65 (tile kernel) must give the same rows for integer data."""
    from tmq_amd import ops
    rng = np.random.default_rng(0)
    K, N = 1024, 192
    W = _ternary(rng, (N, K))
    nw = ops.NativeWeights(torch.from_numpy(oracle.pack(W).view(np.int32)).to(cuda), N)
    x = torch.from_numpy(rng.integers(-6, 7, (65, K)).astype(np.float16)).to(cuda)
    assert torch.equal(ops.ternary_linear(x[:64], nw), ops.ternary_linear(x, nw)[:64])


CONV_CASES = [  # B, C, H, W, N, k, stride, pad, dil
    (2, 8, 9, 9, 16, 3, 1, 1, 1), (1, 16, 14, 14, 32, 3, 2, 1, 1), (2, 64, 8, 8, 64, 3, 1, 1, 1),
    (3, 3, 20, 20, 64, 7, 2, 3, 1), (2, 64, 7, 7, 128, 1, 2, 0, 1), (1, 24, 10, 11, 20, (3, 2), (2, 1), (1, 0), 1),
    (1, 8, 12, 12, 17, 3, 1, 2, 2), (2, 5, 9, 9, 10, 3, 1, 1, 1), (1, 128, 14, 14, 256, 3, 1, 1, 1),
    (4, 64, 16, 16, 64, 3, 1, 1, 1), (1, 8, 7, 7, 8, 3, 2, 0, 1),
    # channel counts that are multiples of 64 take the uniform-tap loader
    (2, 64, 13, 11, 48, 3, 2, 1, 1), (1, 128, 9, 10, 70, (3, 5), (1, 2), (2, 1), (2, 1)), (3, 192, 6, 6, 64, 1, 1, 0, 1),
    (2, 256, 7, 7, 512, 3, 1, 1, 1), (1, 64, 5, 5, 32, 5, 1, 4, 2), (2, 512, 7, 7, 512, 3, 1, 1, 1),
    # small batches of ResNet-sized layers: split-reduction kernel with 32 x 32 / 16 x 32 / 32 x 64 tiles
    (1, 64, 56, 56, 64, 3, 1, 1, 1), (1, 128, 28, 28, 128, 3, 1, 1, 1), (4, 64, 56, 56, 64, 3, 1, 1, 1),
    (2, 128, 28, 28, 256, 1, 2, 0, 1),
    # a short reduction with many tiles stays on the tile kernel
    (8, 64, 40, 40, 128, 1, 1, 0, 1),
    # padding wider than the window's reach, dilation and strides on the direct-to-LDS loaders (taps outside the
    # image are out-of-range buffer offsets there), last tile ragged in M; 64 / 8 / 16 / 32 channels
    (3, 64, 9, 7, 64, 3, 1, 4, 1), (2, 64, 10, 10, 96, 3, 2, 3, 3), (1, 8, 11, 9, 40, 3, 1, 5, 2),
    (5, 16, 7, 7, 64, (5, 3), (2, 1), (4, 3), (1, 2)), (2, 32, 6, 13, 24, 3, (1, 2), (3, 0), 1),
    # ... and on the split-reduction kernel (many channels, few output tiles)
    (1, 256, 5, 5, 128, 3, 1, 3, 1), (2, 512, 4, 6, 256, 3, 2, 2, 2),
    # 129 .. 256 output channels over at least 8192 output positions: 64 x 256 tiles, eight wavefronts, loads between
    # the MFMAs (18 k-tiles + none / 2 k-tiles only / ragged channels, stride 2 and a ragged last row tile)
    (8, 128, 32, 32, 256, 3, 1, 1, 1), (8, 128, 32, 32, 256, 1, 1, 0, 1), (9, 64, 61, 63, 200, 3, 2, 1, 1),
    # split reduction over 256 .. 512 tiles of 64 x 64 with K >= 1024: four wavefronts per tile, two workgroups per CU
    (16, 128, 32, 32, 64, 3, 1, 1, 1), (15, 192, 23, 25, 100, 3, 1, 1, 1),
]


@pytest.mark.parametrize("B,C,H,W,N,k,stride,pad,dil", CONV_CASES)
def test_conv2d_matches_oracle(cuda, oracle, B, C, H, W, N, k, stride, pad, dil):
    from tmq_amd import ops
    pair = lambda v: tuple(v) if isinstance(v, tuple) else (v, v)
    k, stride, pad, dil = pair(k), pair(stride), pair(pad), pair(dil)
    rng = np.random.default_rng(B + C + H + N)
    Wt = _ternary(rng, (N, C, k[0], k[1]))
    words = oracle.pack(Wt.reshape(N, -1))
    x = rng.standard_normal((B, C, H, W)).astype(np.float16)
    scale = (0.5 + rng.random(N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    packed = ops.compactify_ternary(torch.from_numpy(Wt).to(cuda))
    assert np.array_equal(packed.cpu().numpy().view(np.uint32).reshape(words.shape), words)
    nw = ops.NativeWeights(packed, N, conv_kernel=k)
    tx = torch.from_numpy(x).to(cuda)
    ts, tb = torch.from_numpy(scale).to(cuda), torch.from_numpy(bias).to(cuda)
    y = ops.ternary_conv2d(tx, nw, stride, pad, dil, ts, tb)
    want = oracle.conv2d(x.astype(np.float32), words, N, k, stride, pad, dil, scale, bias)
    assert tuple(y.shape) == want.shape
    assert y.is_contiguous(memory_format=torch.channels_last)
    assert _rel_err(y.cpu().numpy(), want) <= 1e-3
    assert _rel_err(y.cpu().numpy(), want) <= 3e-6
    # the library routine on expanded weights
    ref = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(Wt).double(), None, stride, pad, dil)
    ref = ref * torch.from_numpy(scale).double().view(1, -1, 1, 1) + torch.from_numpy(bias).double().view(1, -1, 1, 1)
    assert _rel_err(y.cpu().numpy(), ref.numpy()) <= 3e-6
    # fp16 output with fused residual + relu
    res = torch.from_numpy(rng.standard_normal(want.shape).astype(np.float16)).to(cuda).contiguous(
        memory_format=torch.channels_last)
    y16 = ops.ternary_conv2d(tx, nw, stride, pad, dil, ts, tb, residual=res, relu=True, out_dtype=torch.float16)
    want16 = np.maximum(want + res.float().cpu().numpy(), 0)
    assert _rel_err(y16.float().cpu().numpy(), want16) <= 1e-3


@pytest.mark.parametrize("C,H,W,N,k,stride,pad,dil", [
    (8, 20, 13, 24, (7, 4), (2, 1), ((3, 3), (2, 1)), (1, 1)),     # the super-pixel stem
    (8, 9, 9, 16, (3, 3), (1, 1), ((0, 2), (1, 0)), (1, 1)),
    (16, 11, 10, 40, (3, 5), (2, 2), ((2, 1), (0, 3)), (1, 2)),
    (32, 8, 8, 64, (3, 3), (1, 1), ((1, 1), (1, 1)), (2, 2)),
    (64, 9, 7, 32, (3, 3), (1, 2), ((1, 0), (2, 1)), (1, 1)),
    (128, 6, 6, 512, (3, 3), (1, 1), ((0, 1), (1, 0)), (1, 1)),
    (5, 7, 8, 10, (2, 3), (1, 1), ((1, 0), (0, 2)), (1, 1)),
])
def test_conv2d_asymmetric_padding(cuda, C, H, W, N, k, stride, pad, dil):
    """Padding given per side, checked against torch's convolution of the explicitly padded input
    on the expanded weights (small integers: every product and sum is exact, so bit for bit)."""
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(C + H + N)
    Wt = torch.randint(-1, 2, (N, C, k[0], k[1]), device=cuda, generator=g).float()
    x = torch.randint(-4, 5, (3, C, H, W), device=cuda, generator=g).float()
    nw = ops.NativeWeights(ops.compactify_ternary(Wt), N, conv_kernel=k)
    y = ops.ternary_conv2d(x.half(), nw, stride, pad, dil)
    (pt, pb), (pl, pr) = pad
    ref = torch.nn.functional.conv2d(torch.nn.functional.pad(x, (pl, pr, pt, pb)), Wt, None, stride, 0, dil)
    assert y.shape == ref.shape
    assert torch.equal(y, ref)


def test_residual_with_a_dimension_of_size_one(cuda):
    """One output channel (or one row, one column): the residual's stride along a dimension of size one says nothing
    about its layout, so a channels_last residual is accepted whichever value torch left there."""
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(5)
    for N, H, W in ((1, 9, 11), (8, 1, 12), (8, 7, 1)):
        Wt = torch.randint(-1, 2, (N, 16, 1, 1), device=cuda, generator=g).float()
        x = torch.randint(-4, 5, (2, 16, H, W), device=cuda, generator=g).float()
        nw = ops.NativeWeights(ops.compactify_ternary(Wt), N, conv_kernel=(1, 1))
        ref = torch.nn.functional.conv2d(x, Wt)
        for res in (torch.randint(-3, 4, ref.shape, device=cuda, generator=g).float(),
                    torch.randint(-3, 4, ref.shape, device=cuda, generator=g).float().contiguous(memory_format=torch.channels_last)):
            if not res.is_contiguous(memory_format=torch.channels_last):
                continue
            y = ops.ternary_conv2d(x.half(), nw, residual=res)
            assert torch.equal(y, ref + res), (N, H, W)


def test_resnet_layer_shapes_against_torch(cuda):
    """Full-size ResNet-18 layer shapes (batch 8): checked against torch's fp32 convolution on the
    expanded weights, which the small cases above tie to the oracle."""
    from tmq_amd import ops
    g = torch.Generator().manual_seed(20)
    shapes = [(3, 224, 64, 7, 2, 3), (64, 56, 64, 3, 1, 1), (64, 56, 128, 3, 2, 1), (64, 56, 128, 1, 2, 0),
              (128, 28, 128, 3, 1, 1), (128, 28, 256, 3, 2, 1), (256, 14, 256, 3, 1, 1), (256, 14, 512, 3, 2, 1),
              (512, 7, 512, 3, 1, 1)]
    for C, HW, N, k, s, p in shapes:
        u = torch.rand(N, C, k, k, generator=g)
        Wt = torch.where(u < .25, 1.0, torch.where(u < .5, -1.0, 0.0))
        x = torch.randn(8, C, HW, HW, generator=g).half()
        nw = ops.NativeWeights(ops.compactify_ternary(Wt.to(cuda)), N, conv_kernel=(k, k))
        y = ops.ternary_conv2d(x.to(cuda), nw, s, p)
        ref = torch.nn.functional.conv2d(x.to(cuda).float(), Wt.to(cuda), None, s, p)
        err = (y - ref).abs().max().item() / ref.abs().max().item()
        assert err <= 1e-5, (C, HW, N, k, err)


@pytest.mark.parametrize("B,C,HW,N,k,s,p", [(64, 128, 28, 128, 3, 1, 1), (64, 64, 54, 128, 3, 2, 1), (59, 64, 27, 128, 3, 1, 1)])
def test_conv_on_112_row_tiles(cuda, B, C, HW, N, k, s, p):
    """Between one and two 128 x 128 tiles per CU: the convolution runs on 112-row tiles that are loaded as 128 rows
    (whole, ragged in the last tile, and with rows that do not divide by 112). Against torch's fp64 convolution
    (a12: tmq/tmq.py:822-871), with residual, ReLU and fp16 output as the networks use it."""
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(B + HW)
    Wt = torch.randint(-1, 2, (N, C, k, k), device=cuda, generator=g).float()
    x = torch.randn((B, C, HW, HW), device=cuda, generator=g).half().contiguous(memory_format=torch.channels_last)
    nw = ops.NativeWeights(ops.compactify_ternary(Wt), N, conv_kernel=(k, k))
    scale = (torch.rand(N, device=cuda, generator=g) + 0.5) * 0.03
    bias = torch.randn(N, device=cuda, generator=g)
    ref = torch.nn.functional.conv2d(x.double(), Wt.double(), None, s, p) * scale.double().view(1, -1, 1, 1) + bias.double().view(1, -1, 1, 1)
    M = ref.shape[0] * ref.shape[2] * ref.shape[3]
    assert (M + 127) // 128 > 256 and (M + 111) // 112 <= 512           # the shape the rule is for
    y = ops.ternary_conv2d(x, nw, s, p, 1, scale, bias)
    assert ((y.double() - ref).abs().max() / ref.abs().max()).item() <= 2e-5
    res = torch.randn(ref.shape, device=cuda, generator=g).half().contiguous(memory_format=torch.channels_last)
    y16 = ops.ternary_conv2d(x, nw, s, p, 1, scale, bias, residual=res, relu=True, out_dtype=torch.float16)
    want = torch.relu(ref + res.double())
    assert ((y16.double() - want).abs().max() / want.abs().max()).item() <= 1e-3
