"""ResNet-18 for the inference / QAT workloads of BASELINE.json (configs[3] and configs[4]).

torchvision is not available offline, so the network is defined here: the standard BasicBlock
[2, 2, 2, 2] layout with plain nn.Conv2d / nn.Linear layers (bias-free convolutions, BatchNorm
after every convolution), so that tmq_amd.quantize_model swaps them exactly as it would swap
torchvision's. The deployment form of the network is the package's `tmq_amd.ResNetRunner`.
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


def calibrate_batchnorm_(model, x, generator):
    """Give every BatchNorm the statistics of the batch x (one fp32 training-mode forward with momentum 1) and a
    gamma ~ U(0.75, 1.25), beta ~ N(0, 0.2), so that the activations of a network with unscaled ternary weights
    stay of order one in every layer. Without it each 3 x 3 convolution multiplies the activation scale by
    ~sqrt(fan_in / 2) (17 at 64 channels) while BatchNorm divides by at most sqrt(2): the fp16 activations of the
    literal BASELINE configs[3] network overflow from the end of layer1 on."""
    momenta = []
    for m in model.modules():
        if isinstance(m, nn.BatchNorm2d):
            momenta.append((m, m.momentum))
            m.momentum = 1.0
    was_training = model.training
    model.train()
    with torch.no_grad():
        model(x.float())
        dev = x.device
        for m in model.modules():
            if isinstance(m, nn.BatchNorm2d):
                m.weight.copy_((0.75 + 0.5 * torch.rand(m.num_features, generator=generator)).to(dev))
                m.bias.copy_((0.2 * torch.randn(m.num_features, generator=generator)).to(dev))
        if getattr(model, "fc", None) is not None and model.fc.bias is not None:
            model.fc.bias.copy_((0.1 * torch.randn(model.fc.bias.numel(), generator=generator)).to(dev))
    for m, mom in momenta:
        m.momentum = mom
    model.train(was_training)


def FusedTernaryResNet18(model):
    """The deployment runner of a tmq_amd-quantized ResNet18 whose layers hold compact weights: the package's
    generic residual-network runner (tmq_amd.ResNetRunner)."""
    from tmq_amd import ResNetRunner
    return ResNetRunner(model)
