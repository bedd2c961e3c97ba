"""The benchmark configurations at their full sizes and with their own seeds, against references that
do not come from this library:

  * ternary linear, K = N = 4096, M in {1, 16, 256, 4096}: weights from seed 10 (P(0) = .5), one fp32
    scale per channel from seed 11 (U(0.5, 1.5)), fp16 N(0, 1) activations from seed 12 -- against an
    fp64 product of the expanded weights computed on the CPU, 1e-3 relative (the stated tolerance);
  * ResNet-18 / 102 classes at batch 64: the deployment runner and the torch.fx-fused fp16 graph against
    an fp32 PyTorch model on the ternary-valued weights that rounds its activations to fp16 at the same
    points the fused kernels do (after every folded BatchNorm / residual / ReLU epilogue), 1e-3 relative.
"""
import copy

import numpy as np
import pytest
import torch
from torch import nn

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def layer4096(cuda):
    from tmq_amd import ops
    K = N = 4096
    gen = lambda s: torch.Generator(device="cpu").manual_seed(s)
    u = torch.rand(N, K, generator=gen(10))
    W = torch.where(u < .25, 1.0, torch.where(u < .5, -1.0, 0.0))
    scale = 0.5 + torch.rand(N, generator=gen(11))
    packed = ops.compactify_ternary(W.to(cuda))
    return W, scale, packed, ops.NativeWeights(packed, N)


@pytest.mark.parametrize("M", [1, 16, 256, 4096])
def test_config3_ternary_linear_at_full_size_against_cpu_fp64(cuda, oracle, layer4096, M):
    from tmq_amd import ops
    W, scale, packed, nw = layer4096
    x = torch.randn(M, 4096, generator=torch.Generator(device="cpu").manual_seed(12)).half()
    want = (x.double() @ W.double().t()) * scale.double()                     # CPU, fp64
    got = ops.ternary_linear(x.to(cuda), nw, scale=scale.to(cuda)).cpu().double()
    err = (got - want).abs().max().item() / want.abs().max().item()
    assert err <= 1e-3, err
    # what fp32 accumulation actually gives (M = 1 with fp16 activations: the 8-bit matrix instructions, whose
    # 32-product adder rounds a little more coarsely)
    tight = 1e-5 if M == 1 else 2e-6
    assert err <= tight, err
    if M <= 16:
        # the oracle's own GEMM on the packed words (fp64 accumulation over the reference's code map)
        words = packed.cpu().numpy().view(np.uint32)
        o = oracle.gemm(x.float().numpy(), words, 4096) * scale.numpy().astype(np.float64)
        assert np.max(np.abs(got.numpy() - o)) / np.max(np.abs(o)) <= tight
    # the reference's binding names on the same data (fp16 and fp32 activations)
    xb = x.to(cuda)
    y = (ops.ternary_mvm_cuda(xb, packed, 4096) if M == 1 else ops.ternary_mmm_cuda(xb, packed, 4096)).cpu().double()
    assert (y * scale.double() - want).abs().max().item() / want.abs().max().item() <= tight
    if M <= 256:
        y32 = ops.ternary_mmm_cuda(xb.float(), packed, 4096).cpu().double()
        assert (y32 * scale.double() - want).abs().max().item() / want.abs().max().item() <= tight


def _faithful_reference(model, x):
    """fp32 PyTorch forward of bench_models.ResNet18 (ternary-valued fp32 weights, eval BatchNorm as the
    affine map scale = gamma / sqrt(var + eps), bias = beta - mean * scale) with activations rounded to fp16
    wherever the fused kernels store them."""
    F = nn.functional

    def conv(x16, conv, bn, relu, res=None):
        acc = F.conv2d(x16.float(), conv.weight.float(), None, conv.stride, conv.padding)
        inv = (bn.running_var + bn.eps).rsqrt() * bn.weight
        y = acc * inv.view(1, -1, 1, 1) + (bn.bias - bn.running_mean * inv).view(1, -1, 1, 1)
        if res is not None:
            y = y + res.float()
        return (y.relu() if relu else y).half()

    with torch.no_grad():
        y = conv(x.half(), model.conv1, model.bn1, True)
        y = F.max_pool2d(y.float(), 3, 2, 1).half()
        for layer in (model.layer1, model.layer2, model.layer3, model.layer4):
            for blk in layer:
                idt = y if blk.downsample is None else conv(y, blk.downsample[0], blk.downsample[1], False)
                h = conv(y, blk.conv1, blk.bn1, True)
                y = conv(h, blk.conv2, blk.bn2, True, idt)
        feat = y.float().mean(dim=(2, 3)).half()
        return F.linear(feat.float(), model.fc.weight.float(), model.fc.bias.float())


def _calibrated_resnet(cuda, batch):
    import tmq_amd as t
    from bench_models import ResNet18, randomize_ternary_, calibrate_batchnorm_
    torch.manual_seed(20)
    model = ResNet18(102)
    ctrl = t.QuantizationControl()
    t.quantize_model(model, ctrl)
    randomize_ternary_(model, torch.Generator().manual_seed(20))
    model.to(cuda)
    x = torch.randn(batch, 3, 224, 224, generator=torch.Generator().manual_seed(20)).half().to(cuda)
    # Unscaled ternary weights multiply the activation scale by ~sqrt(fan_in / 2) per layer: set the BatchNorm
    # statistics from the batch so that activations stay O(1) in fp16, and give the affine part some life.
    calibrate_batchnorm_(model, x[:8], torch.Generator().manual_seed(21))
    model.eval()
    return t, model, x


@pytest.mark.parametrize("batch", [64, 3])
def test_config4_resnet18_fused_paths_against_fp16_faithful_reference(cuda, batch):
    t, model, x = _calibrated_resnet(cuda, batch)
    ref_model = copy.deepcopy(model)                      # keeps the fp32 ternary-valued weights
    want = _faithful_reference(ref_model, x)
    assert torch.isfinite(want).all() and want.abs().max().item() > 1e-2
    t.compressed_state_dict(model, strong=False)          # every layer to compact weights
    from bench_models import FusedTernaryResNet18
    got = FusedTernaryResNet18(model)(x).float()
    scale = want.abs().max().item()
    err = (got - want).abs().max().item() / scale
    assert err <= 1e-3, ("fused runner", err)
    assert (got.argmax(1) == want.argmax(1)).float().mean().item() >= 0.98
    # the same network through the Python API: fold BatchNorm, fp16 between the layers, the library's pooling,
    # ReLU / residual into the epilogues (torch.fx); the user's model code unchanged
    prev = t.set_compact_output_dtype(torch.float16)
    try:
        with torch.no_grad():
            t.fold_batchnorm(model)
            t.use_native_pooling(model)
            gm, sites = t.fuse_epilogues(model)
            assert sites == 18
            got_fx = gm(x).float()
    finally:
        t.set_compact_output_dtype(prev)
    err_fx = (got_fx - want).abs().max().item() / scale
    assert err_fx <= 1e-3, ("fx-fused fp16 graph", err_fx)
