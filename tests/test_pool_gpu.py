"""Max-pool, global average pool and the NCHW -> NHWC4 input repack for fp16 NHWC feature maps, through
the C ABI, against PyTorch's own ops (a maximum and a copy are exact; the mean is compared in fp32)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,C,H,W,k,s,p", [(2, 64, 112, 112, 3, 2, 1), (1, 8, 7, 9, 2, 2, 0), (3, 40, 13, 11, (3, 2), (2, 1), (1, 1)),
                                           (2, 5, 9, 9, 3, 1, 1), (1, 16, 6, 6, 3, 3, 0), (2, 24, 5, 5, 5, 1, 2),
                                           (2, 8, 5, 7, 3, 1, 1), (1, 24, 3, 3, 3, 2, 1), (3, 16, 2, 9, 3, (1, 2), 1)])
def test_maxpool_equals_torch(cuda, B, C, H, W, k, s, p):
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(B + C + H)
    x = torch.randn((B, C, H, W), device=cuda, generator=g).half()
    x[0, 0, 0, 0] = float("-inf")
    want = torch.nn.functional.max_pool2d(x.float(), k, s, p).half()
    got = ops.maxpool2d_nhwc(x.contiguous(memory_format=torch.channels_last), k, s, p)
    assert got.shape == want.shape and got.is_contiguous(memory_format=torch.channels_last)
    assert torch.equal(got, want)
    assert torch.equal(ops.maxpool2d_nhwc(x, k, s, p), want)            # NCHW input is converted first
    with pytest.raises(RuntimeError):
        ops.maxpool2d_nhwc(x, 2, 2, 2)                                    # pad more than half the window


@pytest.mark.parametrize("B,C,H,W", [(64, 512, 7, 7), (3, 40, 5, 9), (2, 5, 3, 3), (1, 8, 1, 1)])
def test_global_average_pool(cuda, B, C, H, W):
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(C + H)
    x = torch.randn((B, C, H, W), device=cuda, generator=g).half().contiguous(memory_format=torch.channels_last)
    want = x.double().mean(dim=(2, 3))
    got32 = ops.avgpool_global_nhwc(x, out_dtype=torch.float32)
    assert got32.shape == (B, C) and got32.dtype == torch.float32
    assert torch.allclose(got32.double(), want, rtol=1e-6, atol=1e-6)
    got16 = ops.avgpool_global_nhwc(x)
    assert got16.dtype == torch.float16 and torch.equal(got16, got32.half())
    # integers: sums are exact, the mean is one fp32 multiply by 1 / (H W)
    xi = torch.randint(-8, 9, (B, C, H, W), device=cuda, generator=g).half().contiguous(memory_format=torch.channels_last)
    exact = xi.float().sum(dim=(2, 3)) * torch.tensor(1.0 / (H * W), dtype=torch.float32, device=cuda)
    assert torch.equal(ops.avgpool_global_nhwc(xi, out_dtype=torch.float32), exact)


@pytest.mark.parametrize("B,C,H,W,dtype", [(4, 3, 224, 224, torch.float16), (2, 3, 8, 12, torch.float32), (1, 1, 5, 4, torch.float16),
                                           (3, 4, 6, 8, torch.float32), (2, 4, 6, 8, torch.float16), (3, 1, 5, 16, torch.float16),
                                           (2, 3, 3, 8, torch.float16), (5, 2, 7, 24, torch.float16)])
def test_input_repack(cuda, B, C, H, W, dtype):
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(B + C + H)
    x = torch.randn((B, C, H, W), device=cuda, generator=g).to(dtype)
    want = torch.zeros((B, H, W, 4), dtype=torch.float16, device=cuda)
    want[..., :C] = x.permute(0, 2, 3, 1).half()
    got = ops.nchw_to_nhwc4(x)
    assert got.shape == want.shape and torch.equal(got, want)
    with pytest.raises(RuntimeError):
        ops.nchw_to_nhwc4(torch.zeros((1, 5, 4, 4), device=cuda))
    with pytest.raises(RuntimeError):
        ops.nchw_to_nhwc4(torch.zeros((1, 3, 4, 6), device=cuda))


@pytest.mark.parametrize("B,C,H,W,N", [(64, 512, 7, 7, 102), (3, 512, 7, 7, 1000), (5, 256, 4, 5, 10), (2, 8, 3, 3, 17), (1, 264, 1, 1, 33),
                                       (2, 1024, 2, 2, 10), (2, 20, 3, 3, 5)])
def test_head_pool_and_classifier_in_one_launch(cuda, B, C, H, W, N):
    """tmq_avgpool_linear: the classifier applied to the global average pool. The means are the pooling kernel's
    (bit for bit: small integers make the product exact as well); on random data the product matches the two-call form
    to fp32 rounding and an fp64 product of the fp16 means to 1e-5. More than 512 channels, or channels not in
    groups of 8, take the two calls."""
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(B + C + N)
    Wt = torch.randint(-1, 2, (N, C), device=cuda, generator=g).float()
    nw = ops.NativeWeights(ops.compactify_ternary(Wt), N)
    scale = torch.rand(N, device=cuda, generator=g) + 0.5
    bias = torch.randn(N, device=cuda, generator=g)
    # exact case: integer activations whose sums divide evenly (H W copies of one value per channel)
    v = torch.randint(-8, 9, (B, C, 1, 1), device=cuda, generator=g).half()
    xi = v.expand(B, C, H, W).contiguous(memory_format=torch.channels_last)
    two = ops.ternary_linear(ops.avgpool_global_nhwc(xi), nw)
    one = ops.avgpool_linear(xi, nw)
    if (H * W) & (H * W - 1) == 0:                              # 1 / (H W) exact: the means are the integers themselves
        assert torch.equal(two, v.view(B, C).float() @ Wt.t())
    assert torch.equal(one, two)
    x = torch.randn((B, C, H, W), device=cuda, generator=g).half().contiguous(memory_format=torch.channels_last)
    means = ops.avgpool_global_nhwc(x)
    if C <= 512:                                                # an identity classifier hands the means through: every bit equal
        eye = ops.NativeWeights(ops.compactify_ternary(torch.eye(C, device=cuda)), C)
        assert torch.equal(ops.avgpool_linear(x, eye), means.float())
    ref = (means.double() @ Wt.double().t()) * scale.double() + bias.double()
    for relu, dt in ((False, torch.float32), (True, torch.float16)):
        want = torch.relu(ref) if relu else ref
        got = ops.avgpool_linear(x, nw, scale, bias, relu=relu, out_dtype=dt)
        two = ops.ternary_linear(means, nw, scale, bias, relu=relu, out_dtype=dt)
        tol = 1e-5 if dt == torch.float32 else 2e-3
        assert got.dtype == dt and ((got.double() - want).abs().max() / want.abs().max().clamp_min(1e-30)).item() <= tol
        assert ((got.double() - two.double()).abs().max() / want.abs().max().clamp_min(1e-30)).item() <= tol
