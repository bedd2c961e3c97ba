"""Deployment helpers over compact (2-bit) TMQ layers: the fusions the reference's README lists as future
work (README.md:150-155) behind two calls.

  optimize_for_inference(model)   any model whose TMQ layers hold compact weights: fold eval-mode BatchNorm
                                  into the layers' epilogues, hand fp16 channels_last between the layers, use
                                  the library's pooling kernels, move ReLU / residual additions into the
                                  kernels' epilogues (torch.fx) and record the forward as one HIP graph per
                                  input shape. Returns the callable.
  FoldedConv / FoldedStem /       the hand-written form of the same thing for residual networks of the
  ResNetRunner                    torchvision layout (conv1, bn1, maxpool, layer1.., avgpool, fc): one launch per
                                  convolution with BatchNorm, ReLU and the residual add in its epilogue.

Both compute what the compact layers' own forward (tmq/tmq.py:662-688, 822-871) computes, followed by the
model's BatchNorm / ReLU / additions; only the number of launches and the activation dtype (fp16) differ.
"""
import torch
from torch import nn

from . import ops
from . import tmq as _tmq


def _pair(v):
    return tuple(v) if isinstance(v, (tuple, list)) else (v, v)


def _folded_affine(bn, n, device):
    """(scale [n], bias [n]) of an eval-mode BatchNorm as y = scale * x + bias; (None, None) without one."""
    if bn is None or isinstance(bn, nn.Identity):
        return None, None
    if not isinstance(bn, (nn.BatchNorm1d, nn.BatchNorm2d)) or not bn.track_running_stats or bn.num_features != n:
        raise RuntimeError("expected a BatchNorm with running statistics and one feature per output channel")
    inv = (bn.running_var.float() + bn.eps).rsqrt()
    g = inv * bn.weight.float() if bn.affine else inv
    h = (bn.bias.float() if bn.affine else torch.zeros_like(g)) - bn.running_mean.float() * g
    return g.to(device).contiguous(), h.to(device).contiguous()


def _layer_affine(layer, bn):
    """Epilogue constants of a compact layer followed by `bn`: the layer's own post-scale, bias and any BatchNorm
    already folded into it (fold_batchnorm), then bn on top: bn(s * acc + b) = (g * s) * acc + (g * b + h)."""
    n = int(layer.original_shape[0])
    dev = layer.weight.device
    layer._update_scale()
    scale, bias = layer._epilogue(n, dev)
    g, h = _folded_affine(bn, n, dev)
    if g is None:
        return scale, bias
    return (g if scale is None else g * scale).contiguous(), (h if bias is None else g * bias + h).contiguous()


class FoldedConv:
    """A compact Conv2d (groups == 1) with the eval-mode BatchNorm that follows it folded into the kernel's
    per-channel epilogue. Call: y = relu?(bn(conv(x)) + residual), fp16 channels_last in and out, one launch."""

    def __init__(self, conv, bn=None):
        if not (isinstance(conv, _tmq.Conv2d) and not isinstance(conv, _tmq.ConvTranspose2d) and conv.compact and conv.groups == 1):
            raise RuntimeError("FoldedConv: expected a compact tmq_amd.Conv2d with groups == 1")
        n, c, ky, kx = (int(v) for v in conv.original_shape)
        self.weights = ops.NativeWeights(conv.weight.data, n, conv_kernel=(ky, kx))
        self.scale, self.bias = _layer_affine(conv, bn)
        self.stride, self.padding, self.dilation = _pair(conv.stride), _pair(conv.padding), _pair(conv.dilation)

    def __call__(self, x, relu=False, residual=None, out_dtype=torch.float16):
        return ops.ternary_conv2d(x, self.weights, self.stride, self.padding, self.dilation, self.scale, self.bias,
                                  residual=residual, relu=relu, out_dtype=out_dtype)


class FoldedStem:
    """A network's opening, max_pool(relu(bn(conv(x))), 3, 2, 1), on an NCHW image of at most 4 channels: the
    convolution (horizontal stride 2) runs over pairs of pixels read as one pixel of 8 channels, which the kernel gathers
    from the NCHW planes itself (Conv2d._superpixel_plan: a 7 x 7 / 2 stem reduces over 7 x 4 x 8 = 224 indices), and
    convolution, BatchNorm, ReLU and pooling are one kernel that never writes the convolution's output. A layer the
    rewrite does not apply to runs as FoldedConv + the pooling kernel (same bits)."""

    def __init__(self, conv, bn=None):
        if not (isinstance(conv, _tmq.Conv2d) and not isinstance(conv, _tmq.ConvTranspose2d) and conv.compact and conv.groups == 1):
            raise RuntimeError("FoldedStem: expected a compact tmq_amd.Conv2d with groups == 1")
        self.conv = conv
        self.scale, self.bias = _layer_affine(conv, bn)
        self.plain = None
        self._plans = {}                # image width -> (native weights, stride, padding) or False

    def _plan(self, x):
        plan = self._plans.get(x.shape[-1])
        if plan is None:
            sp = self.conv._superpixel_plan(x) if x.dtype == torch.float16 else None
            plan = False
            if sp is not None:
                nw, _, pl, pr = sp
                (sy, _), (py, _) = _pair(self.conv.stride), _pair(self.conv.padding)
                plan = (nw, (sy, 1), ((py, py), (pl, pr)))
            self._plans[x.shape[-1]] = plan
        return plan

    def __call__(self, x):
        if x.dtype != torch.float16:
            x = x.to(torch.float16)
        plan = self._plan(x)
        if plan is False:
            if self.plain is None:
                self.plain = FoldedConv(self.conv)
                self.plain.scale, self.plain.bias = self.scale, self.bias
            return ops.maxpool2d_nhwc(self.plain(x, relu=True), 3, 2, 1)
        nw, stride, pad = plan
        # the kernel reads the NCHW planes itself, as pairs of pixels: no repacked copy of the input
        return ops.ternary_conv2d_relu_maxpool_planar(x, nw, stride, pad, 1, self.scale, self.bias)


class ResNetRunner:
    """Inference runner for a residual network of the torchvision layout whose convolutions and classifier are
    compact TMQ layers: attributes conv1, bn1, maxpool (3 x 3 / 2 / 1), layer1 .. layerN (sequences of blocks with
    conv1 / bn1 / conv2 / bn2 [/ conv3 / bn3] and an optional downsample = (conv, bn)), avgpool (global), fc.
    Every convolution is one ternary implicit-GEMM launch with BatchNorm, ReLU and the residual add in its epilogue,
    activations are fp16 channels_last between the layers, the opening is one kernel (FoldedStem). ResNet-18 at
    batch 64 is 21 launches. Takes an fp16 (or fp32) NCHW batch, returns fp32 logits."""

    def __init__(self, model):
        self.stem = FoldedStem(model.conv1, model.bn1)
        self.blocks = []
        k = 1
        while hasattr(model, "layer%d" % k):
            for blk in getattr(model, "layer%d" % k):
                ds = None
                if getattr(blk, "downsample", None) is not None:
                    ds = FoldedConv(blk.downsample[0], blk.downsample[1] if len(blk.downsample) > 1 else None)
                convs = [FoldedConv(blk.conv1, blk.bn1), FoldedConv(blk.conv2, blk.bn2)]
                if hasattr(blk, "conv3"):
                    convs.append(FoldedConv(blk.conv3, blk.bn3))
                self.blocks.append((convs, ds))
            k += 1
        fc = model.fc
        if not (isinstance(fc, _tmq.Linear) and fc.compact and fc.bn is None):
            raise RuntimeError("ResNetRunner: expected a compact tmq_amd.Linear classifier")
        self.fc = (ops.NativeWeights(fc.weight.data, int(fc.original_shape[0])),) + _layer_affine(fc, None)

    @torch.no_grad()
    def __call__(self, x):
        y = self.stem(x)
        for convs, ds in self.blocks:
            idt = y if ds is None else ds(y)
            h = y
            for conv in convs[:-1]:
                h = conv(h, relu=True)
            y = convs[-1](h, relu=True, residual=idt)
        nw, scale, bias = self.fc
        return ops.avgpool_linear(y, nw, scale=scale, bias=bias)      # global average pool + classifier, one launch


class InferenceSession:
    """What optimize_for_inference returns: call it like the model. `module` is the fx GraphModule with the fused
    epilogues (it shares the model's parameters), `fused_sites` the number of ReLU / residual sites moved into
    kernels, `folded` the (layer, BatchNorm) names folded. reset() drops the recorded HIP graphs (after weights were
    overwritten in place or submodules swapped)."""

    def __init__(self, module, runner, folded, fused_sites):
        self.module, self._runner, self.folded, self.fused_sites = module, runner, folded, fused_sites

    def reset(self):
        if isinstance(self._runner, _tmq.GraphedForward):
            self._runner.reset()

    def __call__(self, x):
        # the layers hand on fp16 while this session runs, whatever the global setting is for other models
        prev = _tmq.set_compact_output_dtype(torch.float16)
        try:
            with torch.no_grad():
                return self._runner(x)
        finally:
            _tmq.set_compact_output_dtype(prev)


def optimize_for_inference(model: nn.Module, graph: bool = True) -> InferenceSession:
    """Everything this library can take out of an inference forward, in the order the steps need: eval mode,
    fold_batchnorm (BatchNorm into the compact layers' epilogues), fp16 channels_last between the layers,
    use_native_pooling, fuse_epilogues (ReLU / residual additions / the opening's max-pool into the kernels, by
    torch.fx; the model's code is not touched) and, with graph=True, GraphedForward (one HIP graph per input shape,
    re-recorded when the layers' weights move). The model's TMQ layers must already hold compact weights
    (compressed_state_dict / load_compressed_state_dict); the model is modified in place (BatchNorm modules become
    nn.Identity, pooling modules are wrapped). ResNet-18 at batch 64: 1.9 ms per forward as loaded, 0.43 ms through
    the returned session."""
    layers = [m for m in model.modules() if isinstance(m, _tmq.TMQLayer)]
    if not layers:
        raise RuntimeError("optimize_for_inference: the model has no TMQ layers")
    loose = [m.layer_name or type(m).__name__ for m in layers if not m.compact]
    if loose:
        raise RuntimeError("optimize_for_inference: these layers do not hold compact weights yet (call "
                           "compressed_state_dict(model) or load a compressed state dict first): " + ", ".join(map(str, loose[:8])))
    model.eval()
    folded = _tmq.fold_batchnorm(model)
    _tmq.use_native_pooling(model)
    prev = _tmq.set_compact_output_dtype(torch.float16)
    try:
        gm, sites = _tmq.fuse_epilogues(model)
    finally:
        _tmq.set_compact_output_dtype(prev)
    return InferenceSession(gm, _tmq.GraphedForward(gm) if graph else gm, folded, sites)
