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
