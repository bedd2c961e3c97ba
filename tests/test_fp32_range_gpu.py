"""fp32 activations of any magnitude. The kernels carry them as fp16 terms; the bindings first scale the
tensor by a power of two (tmq_f32_prescale, exact) and undo it in the epilogue, so results must match an
fp64 product for tensors scaled far outside fp16's range -- as they do in the reference, which multiplies
in fp32 (tmq/tmq_cuda.cu:242-427). Tolerances: 1e-5 relative for linear layers (two fp16 terms, 22 bits),
2e-3 for convolutions (one fp16 term per input, 2^-11 each)."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

MAGNITUDES = [1.0, 1e-6, 1e5, 3e-30, 2e30]


def _layer(cuda, N, K, seed):
    from tmq_amd import ops
    g = torch.Generator().manual_seed(seed)
    W = torch.randint(-1, 2, (N, K), generator=g).float()
    packed = ops.compactify_ternary(W.to(cuda))
    return W, packed, ops.NativeWeights(packed, N)


@pytest.mark.parametrize("mag", MAGNITUDES)
@pytest.mark.parametrize("M,K,N", [(1, 4096, 512), (8, 2048, 256), (5, 300, 70), (40, 1024, 256), (600, 4096, 2048)])
def test_fp32_activations_of_any_magnitude(cuda, M, K, N, mag):
    from tmq_amd import ops
    W, packed, nw = _layer(cuda, N, K, 1)
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(M, K, generator=g) * mag).float()
    x[0, :7] = torch.tensor([0.0, -0.0, 1e-3, -1e-4, 3e-7, 1.0, -2.5]) * mag     # a wide spread inside one tensor
    scale = 0.5 + torch.rand(N, generator=g)
    bias = torch.randn(N, generator=g) * mag
    want = (x.double() @ W.double().t()) * scale.double() + bias.double()
    ref = want.abs().max().item()
    got = ops.ternary_linear(x.to(cuda), nw, scale=scale.to(cuda), bias=bias.to(cuda)).cpu().double()
    assert torch.isfinite(got).all()
    assert (got - want).abs().max().item() <= 1e-5 * ref, (got - want).abs().max().item() / ref
    # the reference's binding names (ctypes form and, when built, the extension)
    plain = x.double() @ W.double().t()
    for b in ([ops] + ([ops.ext] if ops.ext is not None else [])):
        if M == 1:
            y = b.ternary_mvm_cuda(x.to(cuda), packed, N).cpu().double()
            assert (y - plain).abs().max().item() <= 1e-5 * plain.abs().max().item()
        y = b.ternary_mmm_cuda(x.to(cuda), packed, N).cpu().double()
        assert (y - plain).abs().max().item() <= 1e-5 * plain.abs().max().item()


def test_prescale_values_and_the_switch(cuda):
    from tmq_amd import ops
    for n in (1, 5, 4096, 65536, 65537, 300001):
        x = torch.randn(n, generator=torch.Generator().manual_seed(n)).to(cuda)
        for mag, special in ((1.0, None), (7e-12, float("nan")), (9e20, float("inf")), (0.0, None)):
            xm = x * mag
            if special is not None and n > 3:
                xm[2] = special                                   # takes no part in the maximum
            scale = torch.rand(9, device=cuda) + 0.5
            ps, xs, adj = ops.f32_prescale(xm, scale, 9, want_copy=True)
            s, inv = ps.cpu().tolist()
            fin = xm[torch.isfinite(xm)]
            amax = fin.abs().max().item() if fin.numel() else 0.0
            if amax == 0.0:
                assert s == 1.0 and inv == 1.0
            else:
                assert 1024.0 <= s * amax < 2048.0, (n, mag, s, amax)
                assert np.log2(s) == int(np.log2(s)) and s * inv == 1.0      # a power of two and its reciprocal
            assert torch.equal(xs[torch.isfinite(xm)], fin * s)
            assert torch.equal(adj, scale * inv)
    # without the prescale a tensor beyond fp16's range overflows: the switch exists for callers who know (rows that
    # do not start on 16 bytes: aligned rows take kernels that scale every row themselves, switch or not)
    W, packed, nw = _layer(cuda, 64, 520, 3)
    x = (torch.randn(3 * 520 + 1, generator=torch.Generator().manual_seed(4)).to(cuda) * 1e6)[1:].view(3, 520)
    want = x.double().cpu() @ W.double().t()
    prev = ops.set_fp32_prescale(False)
    try:
        assert prev is True
        assert not torch.isfinite(ops.ternary_linear(x, nw)).all()
        small = ops.ternary_linear(x * 1e-6, nw).cpu().double()             # of order 1: fine either way
        assert (small - want * 1e-6).abs().max().item() <= 1e-5 * want.abs().max().item() * 1e-6
    finally:
        ops.set_fp32_prescale(prev)
    assert (ops.ternary_linear(x, nw).cpu().double() - want).abs().max().item() <= 1e-5 * want.abs().max().item()


@pytest.mark.parametrize("mag", [1e-6, 1e5])
def test_fp32_convolution_inputs_of_any_magnitude(cuda, mag):
    import tmq_amd as t
    from tmq_amd import ops
    g = torch.Generator().manual_seed(5)
    for cin, cout, k, stride, groups in ((16, 32, 3, 1, 1), (3, 16, 7, 2, 1), (32, 32, 3, 1, 32)):
        W = torch.randint(-1, 2, (cout, cin // groups, k, k), generator=g).float()
        x = torch.randn(2, cin, 16, 16, generator=g) * mag
        want = torch.nn.functional.conv2d(x.double(), W.double(), None, stride, k // 2, groups=groups)
        layer = t.Conv2d(cin, cout, k, stride=stride, padding=k // 2, groups=groups, bias=False)
        layer.weight = torch.nn.Parameter(W.clone())
        layer.original_shape = W.shape
        layer.to(cuda).eval()
        t.compressed_state_dict(torch.nn.Sequential(layer), strong=False)
        got = layer(x.to(cuda)).cpu().double()
        assert torch.isfinite(got).all()
        assert (got - want).abs().max().item() <= 2e-3 * want.abs().max().item(), (cin, cout, k, groups)


def test_relu_keeps_nan_in_both_output_types(cuda):
    """torch.relu(NaN) is NaN; the fused ReLU of the epilogues must agree for fp32 and fp16 outputs."""
    from tmq_amd import ops
    for M, K, N in ((1, 4096, 64), (20, 512, 64), (300, 512, 256)):
        W, packed, nw = _layer(cuda, N, K, 6)
        x = torch.randn(M, K, generator=torch.Generator().manual_seed(7)).half()
        x[0, 3] = float("nan")
        for dt in (torch.float32, torch.float16):
            y = ops.ternary_linear(x.to(cuda), nw, relu=True, out_dtype=dt)
            assert torch.isnan(y[0]).all(), (M, dt)
            assert not torch.isnan(y[1:]).any() and (y[1:] >= 0).all()


def test_fold_batchnorm_leaves_a_layer_with_its_own_batchnorm_alone(cuda):
    import tmq_amd as t
    from torch import nn
    torch.manual_seed(8)
    ctrl = t.QuantizationControl()
    net = nn.Sequential(nn.Linear(64, 32), nn.BatchNorm1d(32), nn.ReLU(), nn.Linear(32, 8), nn.BatchNorm1d(8))
    t.quantize_model(net, ctrl)
    net[0].implicit_bn()                                       # a BatchNorm inside the layer, then one outside
    with torch.no_grad():
        for m in list(net.modules()) + [net[0].bn]:
            if isinstance(m, nn.BatchNorm1d):
                m.running_mean.normal_()
                m.running_var.uniform_(0.5, 2.0)
                m.weight.uniform_(0.5, 1.5)
                m.bias.normal_()
        for l in (net[0], net[3]):
            l.weight.copy_(torch.randint(-1, 2, l.weight.shape).float())
    net.to(cuda).eval()
    x = torch.randn(16, 64, device=cuda)
    with torch.no_grad():
        want = net(x)
    t.compressed_state_dict(net, strong=False)
    with torch.no_grad():
        assert torch.allclose(net(x), want, rtol=1e-4, atol=1e-4 * want.abs().max().item())
        with pytest.raises(RuntimeError):
            t.fold_batchnorm(net, pairs=[("0", "1")])
        assert t.fold_batchnorm(net) == [("3", "4")]           # only the layer without a BatchNorm of its own
        assert isinstance(net[1], nn.BatchNorm1d) and isinstance(net[4], nn.Identity)
        assert torch.allclose(net(x), want, rtol=1e-4, atol=1e-4 * want.abs().max().item())


def test_native_weight_cache_follows_the_parameter_version(cuda):
    import tmq_amd as t
    from torch import nn
    lin = t.Linear(256, 32, bias=False)
    lin.to(cuda).eval()
    with torch.no_grad():
        lin.weight.copy_(torch.randint(-1, 2, lin.weight.shape).float())
    t.compressed_state_dict(nn.Sequential(lin), strong=False)
    x = torch.randn(4, 256, device=cuda).half()
    y0 = lin(x)
    from tmq_amd import ops
    new = ops.compactify_ternary(torch.randint(-1, 2, (32, 256), device=cuda).float())
    with torch.no_grad():
        lin.weight.copy_(new)                                  # same storage, the Parameter's version moves
    y1 = lin(x)
    want = x.float() @ ops.expand_ternary(new, [32, 256]).t()
    assert torch.allclose(y1, want, rtol=1e-5, atol=1e-3) and not torch.equal(y0, y1)
    lin.weight.data.copy_(ops.compactify_ternary(torch.zeros(32, 256, device=cuda)))   # unseen by any counter
    lin.invalidate_native()
    assert torch.equal(lin(x), torch.zeros_like(y1))


def test_empty_fp32_batches_give_empty_outputs(cuda):
    """An fp32 batch without entries returns an empty tensor (as the fp16 path does) instead of failing in the
    range prescale, for the convolution, the fused opening, the depthwise kernels and the transposed convolution."""
    import tmq_amd as t
    from tmq_amd import ops
    g = torch.Generator().manual_seed(8)
    for cin, cout, k, stride, groups in ((16, 32, 3, 1, 1), (3, 16, 7, 2, 1), (32, 32, 3, 1, 32)):
        W = torch.randint(-1, 2, (cout, cin // groups, k, k), generator=g).float()
        layer = t.Conv2d(cin, cout, k, stride=stride, padding=k // 2, groups=groups, bias=False)
        layer.weight = torch.nn.Parameter(W.clone())
        layer.original_shape = W.shape
        layer.to(cuda).eval()
        t.compressed_state_dict(torch.nn.Sequential(layer), strong=False)
        for dtype in (torch.float32, torch.float16):
            y = layer(torch.empty(0, cin, 16, 16, device=cuda, dtype=dtype))
            assert y.shape[0] == 0 and y.shape[1] == cout and y.numel() == 0
    W = torch.randint(-1, 2, (16, 8, 3, 3), generator=g).float()
    nw = ops.NativeWeights(ops.compactify_ternary(W.to(cuda)), 16, conv_kernel=(3, 3))
    y = ops.ternary_conv2d_relu_maxpool(torch.empty(0, 8, 16, 16, device=cuda), nw, 1, 1)
    assert y.shape == (0, 16, 8, 8)
    net = torch.nn.Sequential(torch.nn.ConvTranspose2d(8, 4, 3, 2, 1, bias=False))
    ctrl = t.QuantizationControl()
    t.quantize_model(net, ctrl)
    net.to(cuda).eval()
    ctrl.quantize()
    t.compressed_state_dict(net, strong=False)
    y = net(torch.empty(0, 8, 6, 6, device=cuda))
    assert y.shape[0] == 0 and y.shape[1] == 4 and y.numel() == 0


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(7,), (3, 5, 9, 11), (2, 64, 56, 56), (4, 3, 224, 224), (1, 1, 1, 4099)])
def test_one_call_conversion_equals_prescale_then_split(cuda, shape):
    """tmq_f32_to_f16_prescaled (what a convolution on fp32 activations runs in front of it): the same prescale, the
    same fp16 term and the same adjusted scale as tmq_f32_prescale + tmq_split_f32_scaled, in two launches."""
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(sum(shape))
    for mag in (1.0, 3e-20, 7e25):
        x = torch.randn(shape, device=cuda, generator=g) * mag
        if len(shape) == 4:
            x = x.contiguous(memory_format=torch.channels_last)
        x[(0,) * len(shape)] = float("inf") if mag == 1.0 else 0.0     # non-finite values take no part in the maximum
        scale = torch.rand(24, device=cuda, generator=g) + 0.5
        ps, _, adj = ops.f32_prescale(x, scale, 24)
        want = ops.split_f32(x, ps, want_lo=False)[0]
        hi, adj2 = ops.f32_to_f16_prescaled(x, scale, 24)
        assert hi.dtype == torch.float16 and hi.shape == x.shape and hi.stride() == x.stride()
        assert torch.equal(hi.view(torch.int16), want.view(torch.int16))
        assert torch.equal(adj2, adj)
        hi3, adj3 = ops.f32_to_f16_prescaled(x, None, 24)
        assert torch.equal(hi3.view(torch.int16), want.view(torch.int16)) and torch.equal(adj3, ops.f32_prescale(x, None, 24)[2])


def test_switch_sends_many_rows_against_a_narrow_layer_to_the_one_pass_kernel(cuda):
    """With the prescale switched off (values promised to lie in fp16's range), a thousand fp32 rows or more against at
    most 128 channels skip the row-pair route, whose split pass would move the rows three times: same values to fp32
    rounding either way."""
    from tmq_amd import ops
    W, packed, nw = _layer(cuda, 16, 1024, 9)
    x = torch.randn(2048, 1024, generator=torch.Generator().manual_seed(10)).to(cuda)
    want = x.double() @ W.to(cuda).double().t()
    y_pairs = ops.ternary_linear(x, nw)
    prev = ops.set_fp32_prescale(False)
    try:
        y_plain = ops.ternary_linear(x, nw)
    finally:
        ops.set_fp32_prescale(prev)
    for y in (y_pairs, y_plain):
        assert ((y.double() - want).abs().max() / want.abs().max()).item() <= 1e-5
