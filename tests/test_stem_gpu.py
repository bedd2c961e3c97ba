"""The fused network opening (ternary convolution -> scale / bias -> ReLU -> 3 x 3 / 2 max-pool in one kernel)
through the C ABI. The bar is bit equality with the two separate entry points, which the convolution and
pooling tests tie to the oracle and to PyTorch; on small integers also with PyTorch's own fp32 ops, and directly
against the oracle's convolution followed by a window maximum in numpy."""
import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


def _case(cuda, B, C, H, W, N, k, stride, pad, dil, seed, with_scale=True, with_bias=True):
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(seed)
    Wt = torch.randint(-1, 2, (N, C, k[0], k[1]), device=cuda, generator=g).float()
    x = torch.randn((B, C, H, W), device=cuda, generator=g).half().contiguous(memory_format=torch.channels_last)
    scale = ((0.5 + torch.rand(N, device=cuda, generator=g)) * 0.1 * torch.where(torch.rand(N, device=cuda, generator=g) < 0.3, -1.0, 1.0)
             if with_scale else None)
    bias = torch.randn(N, device=cuda, generator=g) if with_bias else None
    nw = ops.NativeWeights(ops.compactify_ternary(Wt), N, conv_kernel=k)
    return ops, x, nw, scale, bias, Wt


# B, C, H, W, N, kernel, stride, padding ((top, bottom), (left, right)) or int, dilation
SHAPES = [
    (2, 8, 20, 13, 24, (7, 4), (2, 1), ((3, 3), (2, 1)), (1, 1)),        # the super-pixel stem, small
    (5, 8, 224, 112, 64, (7, 4), (2, 1), ((3, 3), (2, 1)), (1, 1)),      # ... at ResNet's size: 8 x 7 patches per image
    (1, 8, 9, 9, 16, (3, 3), (1, 1), ((0, 2), (1, 0)), (1, 1)),          # reduction of 72: the last MFMA step is ragged
    (3, 16, 31, 37, 40, (3, 5), (2, 2), ((2, 1), (0, 3)), (1, 2)),       # 16 channels, dilation, 240-long reduction
    (2, 32, 21, 18, 64, (2, 4), (1, 2), 1, (1, 1)),                      # 32 channels, K = 256 exactly
    (1, 8, 3, 3, 8, (3, 3), (1, 1), 1, (1, 1)),                          # one patch, mostly padding
    (2, 8, 57, 59, 56, (5, 5), (1, 1), 2, (1, 1)),                       # odd extents: ragged last patch row and column
    (3, 8, 30, 34, 64, (1, 1), (1, 1), 0, (1, 1)),                       # 1 x 1: one piece per output
    (2, 8, 64, 64, 32, (4, 4), (4, 4), 0, (1, 1)),                       # patchify: stride = kernel
    (2, 8, 33, 29, 48, (3, 3), (2, 3), ((1, 0), (0, 2)), (2, 1)),
]


@pytest.mark.parametrize("B,C,H,W,N,k,stride,pad,dil", SHAPES)
def test_fused_opening_equals_the_two_calls(cuda, B, C, H, W, N, k, stride, pad, dil):
    ops, x, nw, scale, bias, _ = _case(cuda, B, C, H, W, N, k, stride, pad, dil, seed=B + C + H + N)
    full = ops.ternary_conv2d(x, nw, stride, pad, dil, scale, bias, relu=True, out_dtype=torch.float16)
    want = ops.maxpool2d_nhwc(full, 3, 2, 1)
    got = ops.ternary_conv2d_relu_maxpool(x, nw, stride, pad, dil, scale, bias)
    assert got.shape == want.shape and got.dtype == torch.float16
    assert got.is_contiguous(memory_format=torch.channels_last)
    assert torch.equal(got, want)
    assert torch.equal(want, F.max_pool2d(full.float(), 3, 2, 1).half())


@pytest.mark.parametrize("with_scale,with_bias", [(False, False), (True, False), (False, True)])
def test_optional_scale_and_bias(cuda, with_scale, with_bias):
    ops, x, nw, scale, bias, _ = _case(cuda, 2, 8, 40, 26, 64, (7, 4), (2, 1), ((3, 3), (2, 1)), (1, 1), 5, with_scale, with_bias)
    want = ops.maxpool2d_nhwc(ops.ternary_conv2d(x, nw, (2, 1), ((3, 3), (2, 1)), 1, scale, bias, relu=True, out_dtype=torch.float16), 3, 2, 1)
    assert torch.equal(ops.ternary_conv2d_relu_maxpool(x, nw, (2, 1), ((3, 3), (2, 1)), 1, scale, bias), want)


@pytest.mark.parametrize("B,C,H,W,N,k,stride,pad", [(2, 8, 37, 26, 64, (7, 4), (2, 1), ((3, 3), (2, 1))), (3, 16, 19, 23, 24, (3, 3), (1, 1), (1, 1))])
def test_fused_opening_against_the_oracle(cuda, oracle, B, C, H, W, N, k, stride, pad):
    """Against the CPU restatement: the oracle's convolution (fp32 accumulation over the reference's compact words),
    then ReLU and a window maximum in numpy. The fused kernel rounds the convolution's value to fp16 before the
    maximum, hence the fp16 tolerance; the maximum itself is exact."""
    import numpy as np
    from tmq_amd import ops
    rng = np.random.default_rng(B + C + H + N)
    Wt = rng.integers(-1, 2, (N, C, k[0], k[1])).astype(np.float32)
    words = oracle.pack(Wt.reshape(N, -1))
    x = rng.standard_normal((B, C, H, W)).astype(np.float16)
    scale = ((0.5 + rng.random(N)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    if isinstance(pad[0], tuple):
        # the oracle pads symmetrically: hand it the explicitly padded image
        xp = np.pad(x, ((0, 0), (0, 0), pad[0], pad[1]))
        conv = oracle.conv2d(xp.astype(np.float32), words, N, k, stride, (0, 0), (1, 1), scale, bias)
    else:
        conv = oracle.conv2d(x.astype(np.float32), words, N, k, stride, pad, (1, 1), scale, bias)
    act = np.maximum(conv, 0)
    Ho, Wo = act.shape[2:]
    padded = np.full((B, N, Ho + 2, Wo + 2), -np.inf, dtype=np.float32)
    padded[:, :, 1:-1, 1:-1] = act
    Po, Pwo = (Ho - 1) // 2 + 1, (Wo - 1) // 2 + 1
    want = np.stack([padded[:, :, i:i + 2 * Po:2, j:j + 2 * Pwo:2] for i in range(3) for j in range(3)]).max(axis=0)
    nw = ops.NativeWeights(ops.compactify_ternary(torch.from_numpy(Wt).to(cuda)), N, conv_kernel=k)
    got = ops.ternary_conv2d_relu_maxpool(torch.from_numpy(x).to(cuda), nw, stride, pad, 1, torch.from_numpy(scale).to(cuda),
                                          torch.from_numpy(bias).to(cuda))
    assert tuple(got.shape) == want.shape
    err = np.abs(got.float().cpu().numpy() - want).max() / np.abs(want).max()
    assert err <= 1e-3, err


def test_small_integers_against_torch(cuda):
    """Integer activations and weights: every product and sum is exact, so PyTorch's fp32 convolution, ReLU and
    max-pool give the same numbers."""
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(9)
    Wt = torch.randint(-1, 2, (64, 8, 7, 4), device=cuda, generator=g).float()
    x = torch.randint(-4, 5, (3, 8, 50, 41), device=cuda, generator=g).float()
    bias = torch.randint(-20, 21, (64,), device=cuda, generator=g).float()
    nw = ops.NativeWeights(ops.compactify_ternary(Wt), 64, conv_kernel=(7, 4))
    got = ops.ternary_conv2d_relu_maxpool(x.half(), nw, (2, 1), ((3, 3), (2, 1)), 1, None, bias)
    ref = F.max_pool2d(F.relu(F.conv2d(F.pad(x, (2, 1, 3, 3)), Wt, bias, (2, 1))), 3, 2, 1)
    assert torch.equal(got.float(), ref)


def test_fp32_input_is_prescaled_like_the_convolution(cuda):
    ops, x, nw, scale, bias, _ = _case(cuda, 2, 8, 30, 30, 64, (3, 3), (1, 1), 1, (1, 1), 11)
    x32 = (x.float() * 3e5).contiguous(memory_format=torch.channels_last)       # beyond fp16's range
    want = ops.maxpool2d_nhwc(ops.ternary_conv2d(x32, nw, 1, 1, 1, scale * 1e-5, bias, relu=True, out_dtype=torch.float16), 3, 2, 1)
    got = ops.ternary_conv2d_relu_maxpool(x32, nw, 1, 1, 1, scale * 1e-5, bias)
    assert torch.isfinite(got).all() and torch.equal(got, want)


@pytest.mark.parametrize("C,N,k", [(64, 64, (3, 3)), (32, 64, (3, 3)), (8, 128, (3, 3)), (8, 60, (3, 3)), (4, 16, (3, 3))])
def test_shapes_outside_the_kernel_take_the_two_calls(cuda, C, N, k):
    """More channels, a longer reduction, more or ragged output channels: the C entry point declines and the
    operator makes the two calls; same result."""
    import ctypes
    from tmq_amd import ops, _capi
    ops_, x, nw, scale, bias, _ = _case(cuda, 2, C, 19, 23, N, k, (1, 1), 1, (1, 1), 3)
    shp = _capi.ConvShape(2, C, 19, 23, N, k[0], k[1], 1, 1, 1, 1, 1, 1, 1, 1)
    y = torch.empty((2, 10, 12, N), dtype=torch.float16, device=cuda)
    status = _capi.load().tmq_ternary_conv2d_relu_maxpool(_capi.ptr(x), ctypes.byref(shp), _capi.ptr(nw.buf), None, None,
                                                          _capi.ptr(y), _capi.stream_of(x))
    assert status == _capi.ERR_UNSUPPORTED
    want = ops.maxpool2d_nhwc(ops.ternary_conv2d(x, nw, 1, 1, 1, scale, bias, relu=True, out_dtype=torch.float16), 3, 2, 1)
    assert torch.equal(ops.ternary_conv2d_relu_maxpool(x, nw, 1, 1, 1, scale, bias), want)


def test_argument_errors(cuda):
    import ctypes
    from tmq_amd import ops, _capi
    ops_, x, nw, scale, bias, _ = _case(cuda, 1, 8, 12, 12, 16, (3, 3), (1, 1), 1, (1, 1), 4)
    lib = _capi.load()
    shp = _capi.ConvShape(1, 8, 12, 12, 16, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1)
    y = torch.empty((1, 6, 6, 16), dtype=torch.float16, device=cuda)
    assert lib.tmq_ternary_conv2d_relu_maxpool(None, ctypes.byref(shp), _capi.ptr(nw.buf), None, None, _capi.ptr(y), None) == -1
    assert lib.tmq_ternary_conv2d_relu_maxpool(_capi.ptr(x), None, _capi.ptr(nw.buf), None, None, _capi.ptr(y), None) == -1
    with pytest.raises(RuntimeError):
        ops.ternary_conv2d_relu_maxpool(x[:, :4], nw, 1, 1)                    # channel mismatch
    with pytest.raises(RuntimeError):
        ops.ternary_conv2d_relu_maxpool(x, nw, 1, 1, 1, scale[:3], bias)      # scale of the wrong length
    empty = ops.ternary_conv2d_relu_maxpool(x[:0], nw, 1, 1, 1, scale, bias)
    assert tuple(empty.shape) == (0, 16, 6, 6)


def test_replays_in_a_graph(cuda):
    ops, x, nw, scale, bias, _ = _case(cuda, 4, 8, 224, 112, 64, (7, 4), (2, 1), ((3, 3), (2, 1)), (1, 1), 21)
    args = (x, nw, (2, 1), ((3, 3), (2, 1)), 1, scale, bias)
    eager = ops.ternary_conv2d_relu_maxpool(*args)
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        ops.ternary_conv2d_relu_maxpool(*args)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            out = ops.ternary_conv2d_relu_maxpool(*args)
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)


@pytest.mark.parametrize("B,C,H,W,N,k,pad", [(4, 3, 224, 224, 64, 7, 3), (2, 3, 33, 48, 64, 7, 3), (3, 1, 20, 24, 16, 5, 2), (2, 4, 17, 20, 40, 3, 1),
                                             (1, 2, 9, 12, 8, 7, 3), (2, 3, 64, 60, 32, 3, 0)])
def test_opening_from_nchw_planes_equals_the_repacked_form(cuda, B, C, H, W, N, k, pad):
    """tmq_ternary_conv2d_relu_maxpool_planar gathers the pixel pairs from the NCHW planes itself: bit for bit the result of
    repacking the input to 4-channel NHWC first (tmq_nchw_to_nhwc4) and running the opening on that."""
    import tmq_amd as t
    from tmq_amd import ops
    torch.manual_seed(B + C + H)
    net = torch.nn.Sequential(torch.nn.Conv2d(C, N, k, 2, pad, bias=False))
    ctrl = t.QuantizationControl()
    t.quantize_model(net, ctrl)
    net.to(cuda).eval()
    ctrl.quantize()
    t.compressed_state_dict(net, strong=False)
    conv = net[0]
    x = torch.randn((B, C, H, W), device=cuda).half()
    sp = conv._superpixel_plan(x)
    assert sp is not None
    nw, kxs, pl, pr = sp
    scale = torch.rand(N, device=cuda) - 0.3
    bias = torch.randn(N, device=cuda)
    xs = ops.nchw_to_nhwc4(x).view(B, H, W // 2, 8).permute(0, 3, 1, 2)
    want = ops.ternary_conv2d_relu_maxpool(xs, nw, (2, 1), ((pad, pad), (pl, pr)), 1, scale, bias)
    got = ops.ternary_conv2d_relu_maxpool_planar(x, nw, (2, 1), ((pad, pad), (pl, pr)), 1, scale, bias)
    assert got.shape == want.shape and torch.equal(got, want)
    # a view that is not contiguous, and fp32 input (repacked first), give the same
    wide = torch.randn((B, C, H, W + 4), device=cuda).half()
    wide[..., 2:W + 2] = x
    assert torch.equal(ops.ternary_conv2d_relu_maxpool_planar(wide[..., 2:W + 2], nw, (2, 1), ((pad, pad), (pl, pr)), 1, scale, bias), want)
    assert torch.equal(ops.ternary_conv2d_relu_maxpool_planar(x.float(), nw, (2, 1), ((pad, pad), (pl, pr)), 1, scale, bias), want)
