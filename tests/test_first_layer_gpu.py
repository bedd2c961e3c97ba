"""A network's first convolution (at most 4 input channels, horizontal stride 2) takes the super-pixel
route in Conv2d.compact_forward; it must give what the float forward gives on the ternarised weights.
Small-integer inputs make every product and sum exact, so the comparison is bit for bit."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("cin,cout,k,stride,pad,H,W", [
    (3, 64, 7, 2, 3, 32, 32), (1, 16, 3, 2, 1, 9, 12), (4, 24, 5, 2, 2, 10, 16), (3, 40, (3, 4), (1, 2), (0, 1), 7, 20),
    (2, 8, 3, 2, 0, 8, 8), (3, 32, (7, 6), 2, (3, 2), 16, 24), (3, 16, 2, 2, 0, 6, 8),
])
def test_first_layer_compact_equals_float(cuda, cin, cout, k, stride, pad, H, W):
    import tmq_amd as t
    torch.manual_seed(cin + cout + H)
    net = torch.nn.Sequential(torch.nn.Conv2d(cin, cout, k, stride, pad, bias=True))
    ctrl = t.QuantizationControl()
    t.quantize_model(net, ctrl)
    net.to(cuda).eval()
    with torch.no_grad():
        net[0].bias.copy_(torch.randint(-4, 5, (cout,)).float())
    x = torch.randint(-3, 4, (2, cin, H, W), device=cuda).float()
    ctrl.quantize()
    want = net(x)
    t.compressed_state_dict(net, strong=False)
    assert net[0].weight.dtype == torch.int32
    assert net[0]._superpixel_plan(x) is not None
    got = net(x)
    assert got.shape == want.shape and torch.equal(got, want)
    assert torch.equal(net(x.half()), want)                                 # fp16 input, same integers
    # an odd width or horizontal stride 1 falls back to the generic loader
    assert net[0]._superpixel_plan(x[..., :W - 1]) is None


@pytest.mark.parametrize("cin,cout,k,stride,pad,H,W", [
    (3, 64, 3, 1, 1, 32, 32), (1, 16, 5, 1, 2, 28, 28), (4, 24, 3, 1, 0, 8, 8), (2, 8, 1, 1, 0, 6, 8), (4, 64, 3, 1, 1, 16, 24),
    (3, 40, (3, 5), (2, 1), (1, 0), 9, 12), (3, 32, 7, 1, 3, 16, 16), (3, 8, 3, 1, (0, 3), 8, 12), (3, 16, (3, 1), 1, (0, 1), 8, 12),
])
def test_first_layer_stride_one_compact_equals_float(cuda, cin, cout, k, stride, pad, H, W):
    """Horizontal stride 1: the pixel-pair route (input pixel pairs as 8 channels, output pixel pairs as 2 N
    filters), also with the epilogue's residual and ReLU, from fp32 and from fp16 NCHW inputs."""
    import tmq_amd as t
    torch.manual_seed(cin + cout + H)
    net = torch.nn.Sequential(torch.nn.Conv2d(cin, cout, k, stride, pad, bias=True))
    ctrl = t.QuantizationControl()
    t.quantize_model(net, ctrl)
    net.to(cuda).eval()
    with torch.no_grad():
        net[0].bias.copy_(torch.randint(-4, 5, (cout,)).float())
    x = torch.randint(-3, 4, (2, cin, H, W), device=cuda).float()
    ctrl.quantize()
    want = net(x)
    t.compressed_state_dict(net, strong=False)
    assert net[0]._pixelpair_plan(x) is not None and net[0]._superpixel_plan(x) is None
    got = net(x)
    assert got.shape == want.shape and torch.equal(got, want)
    assert torch.equal(net(x.half()), want)
    res = torch.randint(-5, 6, want.shape, device=cuda).float()
    fused = net[0].compact_forward(x, residual=res, relu=True)
    assert torch.equal(fused.float(), torch.relu(want + res))
    prev = t.set_compact_output_dtype(torch.float16)          # with the opening's max-pool behind it (fp16 outputs)
    try:
        pooled = net[0].compact_forward(x, relu=True, pool=True)
    finally:
        t.set_compact_output_dtype(prev)
    assert torch.equal(pooled.float(), torch.nn.functional.max_pool2d(torch.relu(want), 3, 2, 1))
    # the same image in channels-last memory: the generic loader for two or three channels
    xl = x.contiguous(memory_format=torch.channels_last)
    if cin in (2, 3):
        assert net[0]._pixelpair_plan(xl) is None
    elif cin == 4:      # four channels in channels-last memory are the pixel pairs already: the route without its repack
        assert net[0]._pixelpair_plan(xl) is not None
        assert torch.equal(net(xl.half()), want)
    assert torch.equal(net(xl), want)
    # an odd width, an even window width or a dilated window keep the generic loader
    assert net[0]._pixelpair_plan(x[..., :W - 1].contiguous()) is None
