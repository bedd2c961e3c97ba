"""Depthwise ternary convolution (groups == channels) through the C ABI: the patch form against the CPU
oracle, the image form against the patch form / torch's grouped convolution, the layer API end to end."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _ternary(rng, shape, p0=0.5):
    u = rng.random(shape)
    return np.where(u < (1 - p0) / 2, 1.0, np.where(u < 1 - p0, -1.0, 0.0)).astype(np.float32)


@pytest.mark.parametrize("P,T,C", [(1, 1, 1), (7, 9, 16), (50, 9, 40), (33, 25, 8), (100, 4, 5), (64, 9, 96)])
def test_patches_form_matches_oracle(cuda, oracle, P, T, C):
    from tmq_amd import ops
    rng = np.random.default_rng(P + T + C)
    W = _ternary(rng, (C, 1, T, 1))
    words = oracle.pack(W.reshape(C, T))                         # [T][ceil(C/16)]
    x = rng.standard_normal((P, T, C)).astype(np.float32)
    want = oracle.dwconv_patches(x, words)
    tw = torch.from_numpy(words.view(np.int32)).to(cuda)
    assert torch.equal(ops.compactify_ternary(torch.from_numpy(W).to(cuda)).view(-1), tw.view(-1))
    for tx, tol in ((torch.from_numpy(x), 2e-6), (torch.from_numpy(x).half(), 1e-3)):
        got = ops.ternary_dwconv_cuda(tx.to(cuda).view(1, P, T * C), tw, 1, T, C)
        assert tuple(got.shape) == (1, P, C) and got.dtype == torch.float32
        err = np.max(np.abs(got.cpu().numpy().reshape(P, C) - want)) / max(1e-30, np.max(np.abs(want)))
        assert err <= tol
    ext = ops.ext
    if ext is not None:
        assert torch.equal(ext.ternary_dwconv_cuda(torch.from_numpy(x).to(cuda).view(1, P, T * C), tw, 1, T, C),
                           ops.ternary_dwconv_cuda(torch.from_numpy(x).to(cuda).view(1, P, T * C), tw, 1, T, C))


@pytest.mark.parametrize("B,C,H,W,k,stride,pad,dil", [
    (2, 16, 9, 9, 3, 1, 1, 1), (1, 40, 12, 11, (3, 5), (2, 1), (1, 2), 1), (3, 8, 7, 7, 3, 2, 0, 1),
    (2, 5, 6, 6, 3, 1, 1, 1), (1, 96, 14, 14, 3, 1, 2, 2), (2, 32, 8, 8, 5, 1, ((2, 1), (0, 3)), 1),
    # square 5 x 5 and 7 x 7 windows on the several-positions-per-thread kernel: strides 1 and 2, ragged widths
    (2, 24, 13, 11, 5, 1, 2, 1), (1, 16, 14, 15, 5, 2, 2, 1), (2, 8, 9, 10, 7, 1, 3, 1), (1, 40, 15, 13, 7, 2, 3, 1),
    (1, 8, 3, 3, 7, 1, 3, 1), (1, 16, 20, 17, 5, (1, 2), (2, 0), 1),
    # rectangular and dilated windows on the same kernel: 1 .. 5 or 7 columns, any number of rows, horizontal stride and
    # dilation of 1 or 2, any vertical ones
    (2, 16, 12, 13, (1, 7), 1, (0, 3), 1), (1, 24, 11, 12, (5, 2), (1, 2), (2, 1), 1), (2, 8, 10, 10, 4, 2, 1, 1),
    (1, 32, 16, 15, 3, 2, 2, 2), (1, 16, 17, 16, (3, 5), 1, (3, 4), (3, 2)), (2, 8, 9, 9, (7, 1), 1, (3, 0), 1),
    (1, 8, 18, 19, (2, 7), 1, (1, 6), (1, 2)), (1, 16, 21, 22, (9, 4), (3, 2), (4, 3), (1, 2)), (2, 8, 8, 30, (1, 5), (1, 2), (0, 4), (1, 2)),
    # what stays on the one-position-per-thread kernel: 6 columns, horizontal dilation 3, horizontal stride 3
    (1, 8, 9, 12, (2, 6), 1, (0, 2), 1), (1, 8, 10, 14, 3, 1, 3, 3), (1, 16, 9, 13, 3, 3, 1, 1),
    # channel counts that are a multiple of 4 but not of 8: pixels start on 8 bytes, whole groups of 8 channels come as
    # two 8-byte loads and the last, partial group reads on into the next pixel (element by element at the last pixel)
    (2, 12, 9, 10, 3, 1, 1, 1), (1, 100, 14, 13, 5, 2, 2, 1), (3, 20, 8, 8, (3, 5), 1, (1, 2), 1), (1, 4, 6, 7, 3, 1, 1, 1),
    (2, 36, 7, 9, 3, 2, 0, 2),
])
def test_image_form_exact_on_integers(cuda, B, C, H, W, k, stride, pad, dil):
    """Small-integer activations: every product and sum is exact, so the result must equal torch's
    grouped convolution on the expanded weights bit for bit; then scale / bias / residual / ReLU / fp16."""
    from tmq_amd import ops
    pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    k, stride, dil = pair(k), pair(stride), pair(dil)
    g = torch.Generator(device=cuda).manual_seed(B + C + H)
    Wt = torch.randint(-1, 2, (C, 1, k[0], k[1]), device=cuda, generator=g).float()
    x = torch.randint(-4, 5, (B, C, H, W), device=cuda, generator=g).float()
    words = ops.compactify_ternary(Wt)
    assert tuple(words.shape) == (1, k[0], k[1], (C + 15) // 16)
    y = ops.ternary_dwconv2d(x.half(), words, k, stride, pad, dil)
    if isinstance(pad, tuple) and isinstance(pad[0], tuple):
        (pt, pb), (pl, pr) = pad
        ref = torch.nn.functional.conv2d(torch.nn.functional.pad(x, (pl, pr, pt, pb)), Wt, None, stride, 0, dil, groups=C)
    else:
        ref = torch.nn.functional.conv2d(x, Wt, None, stride, pad, dil, groups=C)
    assert y.shape == ref.shape and y.is_contiguous(memory_format=torch.channels_last)
    assert torch.equal(y, ref)
    scale = torch.pow(2.0, torch.randint(-2, 3, (C,), device=cuda, generator=g).float())
    bias = torch.randint(-9, 10, (C,), device=cuda, generator=g).float()
    res = torch.randint(-5, 6, ref.shape, device=cuda, generator=g).half().contiguous(memory_format=torch.channels_last)
    y16 = ops.ternary_dwconv2d(x.half(), words, k, stride, pad, dil, scale, bias, residual=res, relu=True,
                               out_dtype=torch.float16)
    want = torch.relu(ref * scale.view(1, -1, 1, 1) + bias.view(1, -1, 1, 1) + res.float())
    assert y16.dtype == torch.float16 and torch.equal(y16.float(), want.half().float())


def test_depthwise_layer_compact_inference(cuda):
    """quantize_model -> ternarise -> compressed_state_dict switches a depthwise Conv2d to compact
    weights; its compact forward must equal the float forward on the ternarised weights."""
    import tmq_amd as t
    torch.manual_seed(3)
    net = torch.nn.Sequential(torch.nn.Conv2d(24, 24, 3, 1, 1, groups=24, bias=True), torch.nn.ReLU(),
                              torch.nn.Conv2d(24, 10, 1, bias=False))
    ctrl = t.QuantizationControl()
    t.quantize_model(net, ctrl)
    net.to(cuda).eval()
    x = torch.randint(-3, 4, (2, 24, 10, 10), device=cuda).float()
    ctrl.quantize()
    want = net(x)
    t.compressed_state_dict(net, strong=False)
    assert net[0].weight.dtype == torch.int32
    got = net(x)
    assert torch.allclose(got, want, rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("cin,cout,k,stride,pad,opad,dil", [
    (16, 8, 3, 2, 1, 1, 1), (24, 40, 2, 2, 0, 0, 1), (8, 8, 3, 1, 1, 0, 1), (32, 5, (3, 2), (2, 1), (1, 0), 0, 1),
    (16, 16, 4, 2, 1, 0, 1),            # the usual decoder layer: four phases of 2 x 2 taps
    (8, 8, 2, 3, 0, 1, 1),              # kernel smaller than the stride: phases without any tap (bias only)
    (8, 4, 3, 2, 2, 1, 1),              # padding as large as the kernel reaches
    (4, 6, 3, 2, 1, 0, 2),              # dilation 2 at stride 2: every tap lands in the even phase
    (8, 8, 5, 3, 2, 2, 1), (8, 8, 3, 1, 3, 0, 1),   # stride 3; padding beyond the kernel (results to skip)
    (64, 24, (3, 5), (2, 3), (1, 2), (1, 2), (1, 2)), (5, 7, 4, 4, 0, 3, 1)])
def test_transposed_layer_compact_inference(cuda, cin, cout, k, stride, pad, opad, dil):
    """ConvTranspose2d: the compact forward (one stride-1 implicit-GEMM convolution per phase of the output
    grid) must equal the float forward on the ternarised weights; small integers make that exact."""
    import tmq_amd as t
    torch.manual_seed(cin + cout)
    net = torch.nn.Sequential(torch.nn.ConvTranspose2d(cin, cout, k, stride, pad, output_padding=opad, bias=True, dilation=dil))
    ctrl = t.QuantizationControl()
    t.quantize_model(net, ctrl)
    net.to(cuda).eval()
    with torch.no_grad():
        net[0].bias.copy_(torch.randint(-4, 5, (cout,)).float())
    x = torch.randint(-3, 4, (2, cin, 6, 5), device=cuda).float()
    ctrl.quantize()
    want = net(x)
    t.compressed_state_dict(net, strong=False)
    assert net[0].weight.dtype == torch.int32
    got = net(x)
    assert got.shape == want.shape and torch.equal(got, want)


@pytest.mark.parametrize("B,P,T,C", [(1, 1, 1, 1), (1, 7, 9, 16), (3, 50, 9, 40), (2, 130, 4, 5), (2, 64, 25, 96), (1, 200, 6, 70)])
def test_transposed_column_form_matches_oracle(cuda, oracle, B, P, T, C):
    """out[b][c T + t][p] = in[b][p][c] * T[c][t]: a product with +1 / -1 / 0, bit-identical to the oracle
    (signed zeros included), for every batch entry; 2-, 3- and 4-D calling conventions; the extension."""
    from tmq_amd import ops
    rng = np.random.default_rng(B + P + T + C)
    W = _ternary(rng, (C, T))
    words = oracle.pack(W)                                       # [T][ceil(C/16)]
    x = rng.standard_normal((B, P, C)).astype(np.float32)
    x[0, 0, 0] = -0.0
    want = oracle.dwconvtrans_cols(x, words, T)
    # the restatement itself against the textbook outer product
    assert np.array_equal(want, np.einsum("bpc,ct->bctp", x, W).reshape(B, C * T, P))
    tw = torch.from_numpy(words.view(np.int32)).to(cuda).view(1, T, 1, -1)
    tx = torch.from_numpy(x).to(cuda)
    got = ops.ternary_dwconvtrans_cuda(tx, tw, 1, T)
    assert tuple(got.shape) == (B, C * T, P) and got.dtype == torch.float32
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    got4 = ops.ternary_dwconvtrans_cuda(tx.view(B, 1, P, C), tw, T, 1)
    assert tuple(got4.shape) == (B, 1, C * T, P) and torch.equal(got4.view(B, C * T, P), got)
    got2 = ops.ternary_dwconvtrans_cuda(tx[0], tw, 1, T)
    assert tuple(got2.shape) == (C * T, P) and torch.equal(got2, got[0])
    ext = ops.ext
    if ext is not None:
        assert torch.equal(ext.ternary_dwconvtrans_cuda(tx, tw, 1, T), got)
        assert torch.equal(ext.ternary_dwconvtrans_cuda(tx.view(B, 1, P, C), tw, 1, T), got4)
        with pytest.raises(RuntimeError):
            ext.ternary_dwconvtrans_cuda(tx, tw, 2, T)          # taps do not match the words
    with pytest.raises(RuntimeError):
        ops.ternary_dwconvtrans_cuda(tx.half(), tw, 1, T)


@pytest.mark.parametrize("B,C,H,W,k,stride,pad,opad,dil", [
    (2, 16, 5, 5, 3, 2, 1, 1, 1), (1, 40, 6, 7, (3, 2), (2, 3), (1, 0), (1, 2), 1), (3, 8, 4, 4, 3, 1, 1, 0, 1),
    (2, 5, 6, 6, 2, 2, 0, 0, 1), (1, 96, 7, 7, 3, 2, 2, 1, 2), (2, 32, 3, 8, 4, (3, 1), 0, 0, (1, 2)),
])
def test_transposed_image_form_exact_on_integers(cuda, B, C, H, W, k, stride, pad, opad, dil):
    """Small-integer activations: the gathered transposed convolution must equal torch's grouped
    conv_transpose2d on the expanded weights bit for bit, and equal columns + F.fold; then the epilogue."""
    from tmq_amd import ops
    pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    k, stride, pad, opad, dil = pair(k), pair(stride), pair(pad), pair(opad), pair(dil)
    g = torch.Generator(device=cuda).manual_seed(B + C + H)
    Wt = torch.randint(-1, 2, (C, 1, k[0], k[1]), device=cuda, generator=g).float()
    x = torch.randint(-4, 5, (B, C, H, W), device=cuda, generator=g).float()
    words = ops.compactify_ternary(Wt)
    y = ops.ternary_dwconvtrans2d(x.half(), words, k, stride, pad, opad, dil)
    ref = torch.nn.functional.conv_transpose2d(x, Wt, None, stride, pad, opad, groups=C, dilation=dil)
    assert y.shape == ref.shape and y.is_contiguous(memory_format=torch.channels_last)
    assert torch.equal(y, ref)
    # the reference's route: columns, then col2im
    cols = ops.ternary_dwconvtrans_cuda(x.reshape(B, C, H * W).transpose(1, 2).contiguous(), words, k[1], k[0])
    folded = torch.nn.functional.fold(cols, output_size=tuple(ref.shape[-2:]), kernel_size=k, dilation=dil, stride=stride,
                                      padding=pad)
    if opad == (0, 0):
        assert torch.equal(folded, ref)
    scale = torch.pow(2.0, torch.randint(-2, 3, (C,), device=cuda, generator=g).float())
    bias = torch.randint(-9, 10, (C,), device=cuda, generator=g).float()
    res = torch.randint(-5, 6, ref.shape, device=cuda, generator=g).half().contiguous(memory_format=torch.channels_last)
    y2 = ops.ternary_dwconvtrans2d(x.half(), words, k, stride, pad, opad, dil, scale=scale, bias=bias, residual=res, relu=True,
                                   out_dtype=torch.float16)
    want = torch.relu(ref * scale.view(1, -1, 1, 1) + bias.view(1, -1, 1, 1) + res.float()).half()
    assert torch.equal(y2, want)


def test_depthwise_transposed_layer_compact_inference(cuda):
    """A depthwise nn.ConvTranspose2d through quantize_model -> ternarise -> compact weights."""
    import tmq_amd as t
    torch.manual_seed(5)
    net = torch.nn.Sequential(torch.nn.ConvTranspose2d(24, 24, 3, 2, 1, output_padding=1, groups=24, bias=True))
    ctrl = t.QuantizationControl()
    t.quantize_model(net, ctrl)
    net.to(cuda).eval()
    with torch.no_grad():
        net[0].bias.copy_(torch.randint(-4, 5, (24,)).float())
    x = torch.randint(-3, 4, (2, 24, 6, 5), device=cuda).float()
    ctrl.quantize()
    want = net(x)
    t.compressed_state_dict(net, strong=False)
    assert net[0].weight.dtype == torch.int32 and tuple(net[0].weight.shape) == (1, 3, 3, 2)
    got = net(x)
    assert got.shape == want.shape and torch.equal(got, want)
