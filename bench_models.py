"""ResNet-18 for the inference / QAT workloads of BASELINE.json (configs[3] and configs[4]).

torchvision is not available offline, so the network is defined here: the standard BasicBlock
[2, 2, 2, 2] layout with plain nn.Conv2d / nn.Linear layers (bias-free convolutions, BatchNorm
after every convolution), so that tmq_amd.quantize_model swaps them exactly as it would swap
torchvision's. `FusedTernaryResNet18` is the deployment form: it reads the compact weights of
a quantized model and runs every convolution as one ternary implicit-GEMM launch with the
eval-mode BatchNorm folded into the per-channel epilogue, ReLU and the residual add fused, and fp16
channels_last activations between layers.
"""
import torch
from torch import nn


class BasicBlock(nn.Module):
    def __init__(self, cin, cout, stride):
        super().__init__()
        self.conv1 = nn.Conv2d(cin, cout, 3, stride, 1, bias=False)
        self.bn1 = nn.BatchNorm2d(cout)
        self.conv2 = nn.Conv2d(cout, cout, 3, 1, 1, bias=False)
        self.bn2 = nn.BatchNorm2d(cout)
        self.downsample = None
        if stride != 1 or cin != cout:
            self.downsample = nn.Sequential(nn.Conv2d(cin, cout, 1, stride, 0, bias=False), nn.BatchNorm2d(cout))

    def forward(self, x):
        idt = x if self.downsample is None else self.downsample(x)
        out = torch.relu(self.bn1(self.conv1(x)))
        out = self.bn2(self.conv2(out))
        return torch.relu(out + idt)


class ResNet18(nn.Module):
    def __init__(self, num_classes=102):
        super().__init__()
        self.conv1 = nn.Conv2d(3, 64, 7, 2, 3, bias=False)
        self.bn1 = nn.BatchNorm2d(64)
        self.maxpool = nn.MaxPool2d(3, 2, 1)
        chans, layers, cin = (64, 128, 256, 512), [], 64
        for li, c in enumerate(chans):
            layers.append(nn.Sequential(BasicBlock(cin, c, 1 if li == 0 else 2), BasicBlock(c, c, 1)))
            cin = c
        self.layer1, self.layer2, self.layer3, self.layer4 = layers
        self.avgpool = nn.AdaptiveAvgPool2d(1)
        self.fc = nn.Linear(512, num_classes)

    def forward(self, x):
        x = self.maxpool(torch.relu(self.bn1(self.conv1(x))))
        x = self.layer4(self.layer3(self.layer2(self.layer1(x))))
        return self.fc(torch.flatten(self.avgpool(x), 1))


def randomize_ternary_(model, generator, p0=0.5):
    """Fill every conv / linear weight with i.i.d. ternary values, P(0) = p0, and every BatchNorm
    with running_mean ~ N(0, 0.1), running_var ~ U(0.5, 2), gamma 1, beta 0 (BASELINE configs[3])."""
    with torch.no_grad():
        for m in model.modules():
            w = getattr(m, "weight", None)
            if isinstance(m, nn.BatchNorm2d):
                m.running_mean.copy_(0.1 * torch.randn(m.num_features, generator=generator))
                m.running_var.copy_(0.5 + 1.5 * torch.rand(m.num_features, generator=generator))
                m.weight.fill_(1.0)
                m.bias.zero_()
            elif w is not None and w.dim() in (2, 4) and w.dtype == torch.float32:
                u = torch.rand(w.shape, generator=generator)
                w.copy_(torch.where(u < (1 - p0) / 2, 1.0, torch.where(u < 1 - p0, -1.0, 0.0)))


class FusedTernaryResNet18:
    """Deployment runner over a tmq_amd-quantized ResNet18 whose layers hold compact weights."""

    def __init__(self, model: ResNet18):
        from tmq_amd import ops
        self.ops = ops
        self.dev = model.fc.weight.device
        self.stem = self._stem(model.conv1, model.bn1)
        self.blocks = []
        for layer in (model.layer1, model.layer2, model.layer3, model.layer4):
            for blk in layer:
                ds = None if blk.downsample is None else self._conv(blk.downsample[0], blk.downsample[1])
                self.blocks.append((self._conv(blk.conv1, blk.bn1), self._conv(blk.conv2, blk.bn2), ds))
        self.fc = (ops.NativeWeights(model.fc.weight.data, model.fc.original_shape[0]),
                   model.fc.bias.data.float() if model.fc.bias is not None else None)

    def _stem(self, conv, bn):
        """The 7x7 / stride 2 / pad 3 stem on 3 channels as the layer's own super-pixel rewrite
        (tmq_amd.Conv2d._superpixel_plan): a 7x4 / stride (2, 1) convolution over pairs of RGB0 pixels
        read as one pixel of 8 channels; the reduction is 7 x 4 x 8 = 224 long."""
        probe = torch.empty((1, 3, 224, 224), dtype=torch.float16, device=self.dev)
        plan = conv._superpixel_plan(probe)
        assert plan is not None, "the stem does not qualify for the super-pixel rewrite"
        nw, kxs, pl, pr = plan
        pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
        (sy, _), (py, _) = pair(conv.stride), pair(conv.padding)
        inv = (bn.running_var + bn.eps).rsqrt() * bn.weight
        return nw, inv.float().contiguous(), (bn.bias - bn.running_mean * inv).float().contiguous(), (sy, 1), ((py, py), (pl, pr))

    def _conv(self, conv, bn):
        ops = self.ops
        N, C, ky, kx = (int(v) for v in conv.original_shape)
        nw = ops.NativeWeights(conv.weight.data, N, conv_kernel=(ky, kx))
        # eval-mode BatchNorm folded into the epilogue: y = gamma (acc - mean) / sqrt(var + eps) + beta
        inv = (bn.running_var + bn.eps).rsqrt() * bn.weight
        scale = inv.float().contiguous()
        bias = (bn.bias - bn.running_mean * inv).float().contiguous()
        pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
        return nw, scale, bias, pair(conv.stride), pair(conv.padding)

    def _run(self, x, layer, relu, residual=None):
        nw, scale, bias, stride, pad = layer
        return self.ops.ternary_conv2d(x, nw, stride, pad, 1, scale, bias, residual=residual, relu=relu,
                                       out_dtype=torch.float16)

    @torch.no_grad()
    def __call__(self, x):
        B, C, H, W = x.shape
        nhwc4 = self.ops.nchw_to_nhwc4(x)
        xs = nhwc4.view(B, H, W // 2, 8).permute(0, 3, 1, 2)      # [B, 8, H, W / 2], channels_last memory
        nw, scale, bias, stride, pad = self.stem
        y = self.ops.ternary_conv2d_relu_maxpool(xs, nw, stride, pad, 1, scale, bias)      # conv1 + bn1 + relu + maxpool
        for c1, c2, ds in self.blocks:
            idt = y if ds is None else self._run(y, ds, relu=False)
            h = self._run(y, c1, relu=True)
            y = self._run(h, c2, relu=True, residual=idt)
        feat = self.ops.avgpool_global_nhwc(y)
        nw, bias = self.fc
        return self.ops.ternary_linear(feat, nw, bias=bias)
