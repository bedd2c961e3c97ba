"""tmq_ternary_conv2d_view: a convolution whose output positions are scattered into a strided NHWC destination
(how a transposed convolution with groups == 1 is written in one pass, tmq/tmq.py:1007-1042 plans GEMM + F.fold).

Bar: bit-identical to tmq_ternary_conv2d followed by a strided copy of the kept window (the same kernel computes the
same sums; only the addresses of its stores change), every element outside the destination view untouched, for every
kernel family a convolution can take (direct-to-LDS tiles on 64-channel and few-channel inputs, register-staged tiles,
the eight-wavefront 64 x 256 tiles, the split-reduction kernel), fp16 and fp32 outputs, residual and ReLU; and
ConvTranspose2d at sizes beyond the exact small cases of test_dwconv_gpu.py against F.conv_transpose2d (fp64 and the
layer's own float forward).
"""
import ctypes

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu


# (B, C, H, W, N, k, pad, dil): which kernel the dispatch of tmq_ternary_conv2d picks for it
CASES = [
    (4, 64, 20, 20, 64, 3, 1, 1),       # tile_dma_kernel, ConvLoader64, 64 x 64 tiles
    (2, 64, 40, 40, 192, 3, 1, 1),      # 129 .. 256 channels over >= 8192 positions: tile_solo_kernel 64 x 256
    (3, 16, 17, 19, 40, 3, 1, 1),       # few-channel loader
    (2, 12, 9, 11, 24, (3, 2), (1, 0), 1),   # register-staged loader, 8-byte aligned pixels
    (2, 5, 9, 11, 7, 3, 1, 1),          # scalar loader, odd channel counts (scalar stores)
    (2, 128, 14, 14, 128, 3, 1, 1),     # split reduction inside the workgroup (mid_kernel, ConvRows)
    (1, 256, 7, 7, 512, 3, 1, 1),       # the same with four wavefronts per tile
    (2, 64, 12, 12, 64, 2, 0, 2),       # dilation
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_view_equals_dense_then_copy(cuda, case, dtype):
    from tmq_amd import ops
    B, C, H, W, N, k, pad, dil = case
    print("conv view", case, dtype, flush=True)
    pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    g = torch.Generator(device=cuda).manual_seed(C * 1000 + N)
    Wt = torch.randint(-1, 2, (N, C) + pair(k), device=cuda, generator=g).float()
    nw = ops.NativeWeights(ops.compactify_ternary(Wt), N, conv_kernel=pair(k))
    x = torch.randn((B, C, H, W), device=cuda, generator=g).half().contiguous(memory_format=torch.channels_last)
    scale = (torch.rand(N, device=cuda, generator=g) + 0.5) * 0.05
    bias = torch.randn(N, device=cuda, generator=g)
    dense = ops.ternary_conv2d(x, nw, 1, pad, dil, scale, bias, out_dtype=dtype)
    ho, wo = dense.shape[2:]
    # the window of the computed grid that is kept, and where it lands in a larger interleaved tensor
    for (h0, w0, hc, wc), (sy, sx), (oy, ox) in [((0, 0, ho, wo), (2, 2), (1, 0)), ((1, 2, ho - 2, wo - 3), (3, 2), (2, 1)),
                                                 ((0, 0, ho, wo), (1, 1), (0, 0))]:
        big = torch.full((B, N, oy + sy * hc + 1, ox + sx * wc + 2), 7.0, dtype=dtype, device=cuda).contiguous(memory_format=torch.channels_last)
        want = big.clone()
        want[:, :, oy:oy + sy * hc:sy, ox:ox + sx * wc:sx] = dense[:, :, h0:h0 + hc, w0:w0 + wc]
        target = big[:, :, oy:oy + sy * hc:sy, ox:ox + sx * wc:sx]
        assert target.shape[2:] == (hc, wc)
        ops.ternary_conv2d_into(target, x, nw, 1, pad, dil, scale, bias, first=(h0, w0))
        assert torch.equal(big, want), (case, (h0, w0, hc, wc), (sy, sx))
    # residual (read at the destination's own offsets) and ReLU
    res_big = torch.randn((B, N, 2 * ho, 2 * wo), device=cuda, generator=g).to(dtype).contiguous(memory_format=torch.channels_last)
    res = res_big[:, :, 1::2, 0::2]
    dense_r = ops.ternary_conv2d(x, nw, 1, pad, dil, scale, bias, residual=res.contiguous(memory_format=torch.channels_last),
                                 relu=True, out_dtype=dtype)
    big = torch.zeros_like(res_big)
    ops.ternary_conv2d_into(big[:, :, 1::2, 0::2], x, nw, 1, pad, dil, scale, bias, residual=res, relu=True)
    assert torch.equal(big[:, :, 1::2, 0::2], dense_r)
    assert int(big[:, :, 0::2].count_nonzero()) == 0 and int(big[:, :, :, 1::2].count_nonzero()) == 0


def test_view_in_place_residual_and_argument_checks(cuda):
    """The residual may be the destination itself (accumulating phases); malformed views are refused."""
    from tmq_amd import ops, _capi
    g = torch.Generator(device=cuda).manual_seed(5)
    Wt = torch.randint(-1, 2, (64, 64, 3, 3), device=cuda, generator=g).float()
    nw = ops.NativeWeights(ops.compactify_ternary(Wt), 64, conv_kernel=(3, 3))
    x = torch.randint(-3, 4, (2, 64, 10, 10), device=cuda, generator=g).half().contiguous(memory_format=torch.channels_last)
    big = torch.randint(-5, 6, (2, 64, 20, 20), device=cuda, generator=g).float().contiguous(memory_format=torch.channels_last)
    want = big.clone()
    want[:, :, 0::2, 1::2] += F.conv2d(x.float(), Wt, None, 1, 1)
    ops.ternary_conv2d_into(big[:, :, 0::2, 1::2], x, nw, 1, 1, 1, residual=big[:, :, 0::2, 1::2])
    assert torch.equal(big, want)
    with pytest.raises(RuntimeError):
        ops.ternary_conv2d_into(big[:, :32, 0::2, 1::2], x, nw, 1, 1, 1)                 # channel slice: pixels are not N wide
    with pytest.raises(RuntimeError):
        ops.ternary_conv2d_into(big.contiguous()[:, :, 0::2, 1::2], x, nw, 1, 1, 1)      # NCHW memory
    lib = _capi.load()
    shp = _capi.ConvShape(2, 64, 10, 10, 64, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1)
    ep = _capi.Epilogue(None, None, None, 0, _capi.F32)
    for bad in [_capi.OutputView(0, 0, 11, 10, 400, 40, 2), _capi.OutputView(-1, 0, 5, 5, 400, 40, 2),
                _capi.OutputView(3, 0, 8, 10, 400, 40, 2), _capi.OutputView(0, 0, 10, 10, -1, 40, 2)]:
        assert lib.tmq_ternary_conv2d_view(ops.ptr(x), ctypes.byref(shp), ops.ptr(nw.buf), ctypes.byref(ep), ops.ptr(big),
                                           ctypes.byref(bad), None) == -1        # TMQ_ERR_INVALID_ARG
    before = big.clone()                                                                # an empty window: nothing is written
    assert lib.tmq_ternary_conv2d_view(ops.ptr(x), ctypes.byref(shp), ops.ptr(nw.buf), ctypes.byref(ep), ops.ptr(big),
                                       ctypes.byref(_capi.OutputView(0, 0, 0, 10, 400, 40, 2)), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(big, before)


@pytest.mark.parametrize("cin,cout,k,stride,pad,opad,hw,batch", [
    (64, 64, 4, 2, 1, 0, (32, 32), 8),         # the usual decoder layer at a size that fills the chip
    (128, 64, 3, 2, 1, 1, (16, 16), 4),        # odd kernel: phases with 2 x 2, 2 x 1, 1 x 2 and 1 x 1 taps
    (256, 128, 2, 2, 0, 0, (14, 14), 2),       # non-overlapping up-sampling: every phase a 1 x 1 convolution
    (64, 192, 5, 3, 2, 1, (20, 24), 4)])       # stride 3, 129 .. 256 output channels
def test_transposed_layer_one_pass(cuda, cin, cout, k, stride, pad, opad, hw, batch):
    import tmq_amd as t
    torch.manual_seed(cin + cout + k)
    net = torch.nn.Sequential(torch.nn.ConvTranspose2d(cin, cout, k, stride, pad, output_padding=opad, bias=True))
    ctrl = t.QuantizationControl()
    t.quantize_model(net, ctrl)
    net.to(cuda).eval()
    ctrl.quantize()
    layer = net[0]
    Wt = layer.weight.data.clone()
    assert set(Wt.unique().tolist()) <= {-1.0, 0.0, 1.0}
    x = torch.randn((batch, cin) + hw, device=cuda)
    x16 = x.half()
    with torch.no_grad():
        ref = net(x16.float()).double()                    # the layer's own float forward on the ternarised weights
    plain = F.conv_transpose2d(x16.double(), Wt.double(), layer.bias.data.double(), stride, pad, opad)
    assert ((ref - plain).abs().max() / plain.abs().max()).item() <= 2e-5
    t.compressed_state_dict(net, strong=False)
    assert layer.weight.dtype == torch.int32
    launches = []
    from tmq_amd import ops
    orig = ops.ternary_conv2d_into

    def counted(*a, **kw):
        launches.append(1)
        return orig(*a, **kw)

    ops.ternary_conv2d_into = counted
    try:
        got = net(x16)
    finally:
        ops.ternary_conv2d_into = orig
    sy = stride if isinstance(stride, int) else stride[0]
    assert 1 <= len(launches) <= sy * sy                   # one launch per phase, nothing else
    assert got.shape == ref.shape
    err = ((got.double() - ref).abs().max() / ref.abs().max()).item()
    assert err <= 2e-5, err
