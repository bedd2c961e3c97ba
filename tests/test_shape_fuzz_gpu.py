"""Seeded walks over the shapes that decide which kernel family a ternary product takes: single rows and
few rows (8-bit GEMV, weight stream, short reductions, skinny), mid-size dense products (split reduction,
tile kernels; fp32 rows as fp16 row pairs), convolutions (three loaders, two tile families, the split-reduction form) and the fused
opening (one kernel or two), convolutions written into strided views, transposed convolutions and depthwise windows.
Every case is checked against an fp64 product of the same operands
(a11 / a12: tmq/tmq_cuda.cu:478-549, tmq/tmq.py:662-688, 822-871 compute the same sums in fp32), the fused
opening bit for bit against the two separate kernels. Each walk stops at its first failure and prints the
case before it runs it, so that a fault names its shape. About 100 cases per walk, about a minute in all.
"""
import random

import pytest
import torch
import torch.nn.functional as F

pytestmark = pytest.mark.gpu

TOL = 2e-5          # observed: <= 3e-6; the contract is 1e-3 relative


def _linear_case(ops, dev, i, M, K, N, dt):
    print("fuzz linear", i, (M, K, N, str(dt)), flush=True)
    g = torch.Generator(device=dev).manual_seed(1000 + i)
    W = torch.randint(-1, 2, (N, K), device=dev, generator=g, dtype=torch.int8)
    nw = ops.NativeWeights(ops.compactify_ternary(W), N)
    x = torch.randn((M, K), device=dev, generator=g).to(dt)
    scale = 0.5 + torch.rand(N, device=dev, generator=g)
    bias = torch.randn(N, device=dev, generator=g)
    relu = bool(i & 1)
    y = ops.ternary_linear(x, nw, scale, bias, relu=relu)
    ref = (x.double() @ W.double().t()) * scale.double() + bias.double()
    if relu:
        ref = ref.clamp_min(0)
    err = ((y.double() - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()
    assert y.shape == ref.shape and err <= TOL, ((M, K, N, dt), err)


def test_walk_single_and_few_rows(cuda):
    from tmq_amd import ops
    rnd = random.Random(1)
    for i in range(110):
        K = rnd.choice([256 * rnd.randint(1, 70), 64 * rnd.randint(1, 300), rnd.randint(1, 20000)])
        N = rnd.choice([rnd.randint(1, 300), 16 * rnd.randint(1, 700), rnd.randint(1, 12000)])
        M = 1 if i % 3 else rnd.randint(2, 20)
        _linear_case(ops, cuda, i, M, K, N, rnd.choice([torch.float16, torch.float32]))


def test_walk_mid_size_dense(cuda):
    from tmq_amd import ops
    rnd = random.Random(2)
    for i in range(70):
        M = rnd.choice([rnd.randint(17, 600), rnd.randint(600, 3300)])
        K = rnd.choice([64 * rnd.randint(8, 80), 256 * rnd.randint(2, 20), rnd.randint(100, 3000)])
        N = rnd.choice([128, 130, 256, 1000, 4096, 16 * rnd.randint(8, 300), rnd.randint(129, 5000)])
        _linear_case(ops, cuda, 500 + i, M, K, N, torch.float16)


def test_walk_mid_size_fp32_rows(cuda):
    """fp32 activations (the reference's convention): row pairs through the fp16 kernels where K is a multiple of 64,
    the kernels that split on the fly elsewhere."""
    from tmq_amd import ops
    rnd = random.Random(7)
    for i in range(60):
        M = rnd.choice([rnd.randint(2, 40), rnd.randint(17, 600), rnd.randint(600, 2500)])
        K = rnd.choice([64 * rnd.randint(4, 80), 256 * rnd.randint(2, 40), rnd.randint(100, 3000)])
        N = rnd.choice([64, 130, 256, 1000, 4096, 16 * rnd.randint(8, 300), rnd.randint(1, 5000)])
        _linear_case(ops, cuda, 900 + i, M, K, N, torch.float32)


def test_walk_convolutions(cuda):
    from tmq_amd import ops
    rnd = random.Random(3)
    done = 0
    for i in range(140):
        C = rnd.choice([64, 64, 128, 192, 256, 512, 8, 16, 3, 40])
        k = rnd.choice([1, 3, 3, 3, 5])
        s = rnd.choice([1, 1, 2])
        p = rnd.randint(0, k // 2 + 1)
        N = rnd.choice([16, 64, 100, 128, 200, 256, 384, 512])
        B = rnd.randint(1, 24)
        H, W = rnd.randint(k, 40), rnd.randint(k, 40)
        if B * H * W * C * N * k * k > 3e11:
            continue
        desc = (B, C, H, W, N, k, s, p)
        print("fuzz conv", i, desc, flush=True)
        g = torch.Generator(device=cuda).manual_seed(2000 + i)
        Wt = torch.randint(-1, 2, (N, C, k, k), device=cuda, generator=g).float()
        x = torch.randn((B, C, H, W), device=cuda, generator=g).half()
        scale = (torch.rand(N, device=cuda, generator=g) + 0.5) * 0.05
        bias = torch.randn(N, device=cuda, generator=g)
        nw = ops.NativeWeights(ops.compactify_ternary(Wt), N, conv_kernel=(k, k))
        res = None
        if i % 4 == 0:
            ho, wo = (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1
            res = torch.randn((B, N, ho, wo), device=cuda, generator=g).contiguous(memory_format=torch.channels_last)
        y = ops.ternary_conv2d(x, nw, s, p, 1, scale, bias, residual=res, relu=bool(i & 1))
        ref = F.conv2d(x.double(), Wt.double(), None, s, p) * scale.double().view(1, -1, 1, 1) + bias.double().view(1, -1, 1, 1)
        if res is not None:
            ref = ref + res.double()
        if i & 1:
            ref = ref.clamp_min(0)
        err = ((y.double() - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()
        assert y.shape == ref.shape and err <= TOL, (desc, err)
        done += 1
    assert done >= 100


def test_walk_fused_opening(cuda):
    from tmq_amd import ops
    rnd = random.Random(4)
    for i in range(100):
        C = rnd.choice([8, 8, 8, 16, 32])
        while True:
            ky, kx = rnd.randint(1, 7), rnd.randint(1, 7)
            if C * ky * kx <= 256 or rnd.random() < 0.05:
                break
        sy, sx = rnd.randint(1, 3), rnd.randint(1, 3)
        dy, dx = rnd.randint(1, 2), rnd.randint(1, 2)
        pad = ((rnd.randint(0, 3), rnd.randint(0, 3)), (rnd.randint(0, 3), rnd.randint(0, 3)))
        N = rnd.choice([8, 16, 24, 32, 40, 48, 56, 64])
        B = rnd.randint(1, 3)
        H, W = rnd.randint((ky - 1) * dy + 1, 70), rnd.randint((kx - 1) * dx + 1, 70)
        desc = (B, C, H, W, N, (ky, kx), (sy, sx), pad, (dy, dx))
        print("fuzz opening", i, desc, flush=True)
        g = torch.Generator(device=cuda).manual_seed(3000 + i)
        Wt = torch.randint(-1, 2, (N, C, ky, kx), device=cuda, generator=g).float()
        x = torch.randn((B, C, H, W), device=cuda, generator=g).half().contiguous(memory_format=torch.channels_last)
        scale = (torch.rand(N, device=cuda, generator=g) - 0.3) * 0.2
        bias = torch.randn(N, device=cuda, generator=g)
        nw = ops.NativeWeights(ops.compactify_ternary(Wt), N, conv_kernel=(ky, kx))
        full = ops.ternary_conv2d(x, nw, (sy, sx), pad, (dy, dx), scale, bias, relu=True, out_dtype=torch.float16)
        want = ops.maxpool2d_nhwc(full, 3, 2, 1)
        got = ops.ternary_conv2d_relu_maxpool(x, nw, (sy, sx), pad, (dy, dx), scale, bias)
        assert got.shape == want.shape and torch.equal(got, want), desc
        if i % 10 == 0:
            ref = F.conv2d(x.double(), Wt.double(), None, (sy, sx), 0, (dy, dx)) if pad == ((0, 0), (0, 0)) else None
            if ref is not None:
                ref = (ref * scale.double().view(1, -1, 1, 1) + bias.double().view(1, -1, 1, 1)).clamp_min(0)
                err = ((full.double() - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()
                assert err <= 2e-3, (desc, err)          # fp16 outputs


def test_walk_convolutions_into_views(cuda):
    """tmq_ternary_conv2d_view over all loaders and tile families: a random window of the computed grid, written into a
    strided destination, must equal the dense call followed by a copy bit for bit, and touch nothing else."""
    from tmq_amd import ops
    rnd = random.Random(5)
    done = 0
    for i in range(110):
        C = rnd.choice([64, 128, 8, 16, 32, 24, 5, 192])
        k = (rnd.randint(1, 4), rnd.randint(1, 4))
        N = rnd.choice([8, 16, 40, 64, 128, 192, 256, 7])
        B = rnd.randint(1, 6)
        H, W = rnd.randint(k[0], 30), rnd.randint(k[1], 30)
        pad = ((rnd.randint(0, 2), rnd.randint(0, 2)), (rnd.randint(0, 2), rnd.randint(0, 2)))
        dil = (rnd.randint(1, 2), rnd.randint(1, 2))
        if (k[0] - 1) * dil[0] + 1 > H + sum(pad[0]) or (k[1] - 1) * dil[1] + 1 > W + sum(pad[1]):
            continue
        dtype = rnd.choice([torch.float16, torch.float32])
        desc = (B, C, H, W, N, k, pad, dil, str(dtype))
        print("fuzz view", i, desc, flush=True)
        g = torch.Generator(device=cuda).manual_seed(5000 + i)
        Wt = torch.randint(-1, 2, (N, C) + k, device=cuda, generator=g).float()
        nw = ops.NativeWeights(ops.compactify_ternary(Wt), N, conv_kernel=k)
        x = torch.randn((B, C, H, W), device=cuda, generator=g).half().contiguous(memory_format=torch.channels_last)
        scale = torch.rand(N, device=cuda, generator=g) * 0.1
        bias = torch.randn(N, device=cuda, generator=g)
        dense = ops.ternary_conv2d(x, nw, 1, pad, dil, scale, bias, out_dtype=dtype)
        ho, wo = dense.shape[2:]
        h0, w0 = rnd.randint(0, ho - 1), rnd.randint(0, wo - 1)
        hc, wc = rnd.randint(1, ho - h0), rnd.randint(1, wo - w0)
        sy, sx, oy, ox = rnd.randint(1, 3), rnd.randint(1, 3), rnd.randint(0, 2), rnd.randint(0, 2)
        big = torch.full((B, N, oy + sy * hc + 1, ox + sx * wc + 1), 3.0, dtype=dtype, device=cuda).contiguous(memory_format=torch.channels_last)
        want = big.clone()
        want[:, :, oy:oy + sy * hc:sy, ox:ox + sx * wc:sx] = dense[:, :, h0:h0 + hc, w0:w0 + wc]
        ops.ternary_conv2d_into(big[:, :, oy:oy + sy * hc:sy, ox:ox + sx * wc:sx], x, nw, 1, pad, dil, scale, bias, first=(h0, w0))
        assert torch.equal(big, want), desc
        done += 1
    assert done >= 80


def test_walk_transposed_and_depthwise(cuda):
    """Transposed convolutions (one stride-1 convolution per output phase, written in place; a14 / f4:
    tmq/tmq.py:1007-1042) and depthwise windows of every shape (tmq/tmq_cuda.cu:166-238) on small integers, where every
    product and sum is exact: equal to torch's own operators on the ternarised weights bit for bit."""
    import tmq_amd as t
    from tmq_amd import ops
    rnd = random.Random(6)
    for i in range(45):
        cin, cout = rnd.choice([4, 8, 16, 64, 24]), rnd.choice([4, 8, 16, 64, 40])
        k = (rnd.randint(1, 5), rnd.randint(1, 5))
        s = (rnd.randint(1, 3), rnd.randint(1, 3))
        d = (rnd.randint(1, 2), rnd.randint(1, 2))
        p = (rnd.randint(0, 2), rnd.randint(0, 2))
        op = (rnd.randint(0, max(s[0], d[0]) - 1), rnd.randint(0, max(s[1], d[1]) - 1))
        H, W, B = rnd.randint(1, 9), rnd.randint(1, 9), rnd.randint(1, 3)
        ho = (H - 1) * s[0] - 2 * p[0] + d[0] * (k[0] - 1) + 1 + op[0]
        wo = (W - 1) * s[1] - 2 * p[1] + d[1] * (k[1] - 1) + 1 + op[1]
        if ho <= 0 or wo <= 0:
            continue
        desc = (cin, cout, k, s, p, op, d, (B, H, W))
        print("fuzz transposed", i, desc, flush=True)
        torch.manual_seed(6000 + i)
        net = torch.nn.Sequential(torch.nn.ConvTranspose2d(cin, cout, k, s, p, output_padding=op, bias=True, dilation=d))
        ctrl = t.QuantizationControl()
        t.quantize_model(net, ctrl)
        net.to(cuda).eval()
        with torch.no_grad():
            net[0].bias.copy_(torch.randint(-4, 5, (cout,)).float())
        x = torch.randint(-3, 4, (B, cin, H, W), device=cuda).float()
        ctrl.quantize()
        want = net(x)
        t.compressed_state_dict(net, strong=False)
        got = net(x)
        assert got.shape == want.shape and torch.equal(got, want), desc
    for i in range(110):
        C = rnd.choice([8, 16, 24, 40, 5, 96])
        k = (rnd.randint(1, 9), rnd.randint(1, 8))
        s = (rnd.randint(1, 3), rnd.randint(1, 3))
        d = (rnd.randint(1, 3), rnd.randint(1, 3))
        p = (rnd.randint(0, 4), rnd.randint(0, 4))
        B, H, W = rnd.randint(1, 3), rnd.randint(1, 24), rnd.randint(1, 24)
        if (k[0] - 1) * d[0] + 1 > H + 2 * p[0] or (k[1] - 1) * d[1] + 1 > W + 2 * p[1]:
            continue
        desc = (B, C, H, W, k, s, p, d)
        print("fuzz depthwise", i, desc, flush=True)
        g = torch.Generator(device=cuda).manual_seed(7000 + i)
        Wt = torch.randint(-1, 2, (C, 1) + k, device=cuda, generator=g).float()
        x = torch.randint(-4, 5, (B, C, H, W), device=cuda, generator=g).float()
        y = ops.ternary_dwconv2d(x.half(), ops.compactify_ternary(Wt), k, s, p, d)
        ref = F.conv2d(x, Wt, None, s, p, d, groups=C)
        assert y.shape == ref.shape and torch.equal(y.float(), ref), desc
