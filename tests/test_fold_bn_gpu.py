"""fold_batchnorm: eval-mode BatchNorm folded into the compact layers' epilogues must give the
unfolded model's outputs (fp32 rounding apart), replace the BatchNorm modules and refuse misuse."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _randomize_bn(net, g):
    for m in net.modules():
        if isinstance(m, (torch.nn.BatchNorm1d, torch.nn.BatchNorm2d)):
            m.running_mean.copy_(torch.randn(m.num_features, generator=g) * 0.3)
            m.running_var.copy_(torch.rand(m.num_features, generator=g) + 0.5)
            m.weight.data.copy_(torch.rand(m.num_features, generator=g) + 0.5)
            m.bias.data.copy_(torch.randn(m.num_features, generator=g) * 0.2)


def test_fold_into_conv_and_linear(cuda):
    import tmq_amd as t
    g = torch.Generator().manual_seed(1)
    torch.manual_seed(1)
    net = torch.nn.Sequential(torch.nn.Conv2d(3, 16, 3, 2, 1, bias=True), torch.nn.BatchNorm2d(16), torch.nn.ReLU(),
                              torch.nn.Conv2d(16, 64, 3, 1, 1, bias=False), torch.nn.BatchNorm2d(64), torch.nn.ReLU(),
                              torch.nn.Conv2d(64, 64, 3, 1, 1, groups=64, bias=False), torch.nn.BatchNorm2d(64),
                              torch.nn.AdaptiveAvgPool2d(1), torch.nn.Flatten(),
                              torch.nn.Linear(64, 10), torch.nn.BatchNorm1d(10))
    ctrl = t.QuantizationControl(post_scale=True)
    t.quantize_model(net, ctrl)
    _randomize_bn(net, g)
    net.to(cuda).eval()
    ctrl.quantize()
    t.compressed_state_dict(net, strong=False)
    x = torch.randn(4, 3, 16, 16, device=cuda)
    with torch.no_grad():
        want = net(x)
        done = t.fold_batchnorm(net)
        assert done == [("0", "1"), ("3", "4"), ("6", "7"), ("10", "11")]
        assert all(isinstance(net[i], torch.nn.Identity) for i in (1, 4, 7, 11))
        got = net(x)
    assert torch.allclose(got, want, rtol=2e-3, atol=2e-3)
    assert t.fold_batchnorm(net) == []                                        # nothing left to fold
    with pytest.raises(RuntimeError):
        t.expand_compact_layers(net)


def test_fold_resnet_and_explicit_pairs(cuda):
    import tmq_amd as t
    from bench_models import ResNet18, randomize_ternary_
    torch.manual_seed(2)
    model = ResNet18(10)
    ctrl = t.QuantizationControl()
    t.quantize_model(model, ctrl)
    randomize_ternary_(model, torch.Generator().manual_seed(2))
    model.to(cuda)
    ctrl.inference()
    x = torch.randn(2, 3, 64, 64, device=cuda)
    # unscaled ternary weights blow the activation scale up layer by layer: calibrate the BatchNorm
    # statistics on the batch so that the fp16 inputs of the compact convolutions stay finite
    for m in model.modules():
        if isinstance(m, torch.nn.BatchNorm2d):
            m.momentum = 1.0
    model.train()
    with torch.no_grad():
        model(x)
    model.eval()
    t.compressed_state_dict(model, strong=False)
    with torch.no_grad():
        want = model(x)
        assert torch.isfinite(want).all()
        with pytest.raises(RuntimeError):
            t.fold_batchnorm(model, pairs=[("layer1.0.conv1", "layer2.0.bn1")])   # 64 outputs, 128 features
        assert t.fold_batchnorm(model, pairs=[("conv1", "bn1")]) == [("conv1", "bn1")]
        done = t.fold_batchnorm(model)
        assert len(done) == 19 and ("layer2.0.downsample.0", "layer2.0.downsample.1") in done
        assert not any(isinstance(m, torch.nn.BatchNorm2d) for m in model.modules())
        got = model(x)
        # fp16 between the layers: same network within fp16 rounding of the activations
        prev = t.set_compact_output_dtype(torch.float16)
        try:
            got16 = model(x)
            # the library's own fp16 NHWC pooling in place of PyTorch's: the same values (max is exact, the
            # mean accumulates in fp32 either way)
            names = t.use_native_pooling(model)
            assert names == ["maxpool", "avgpool"]
            got16p = model(x)
            # ReLU and residual additions into the convolutions' epilogues: 8 blocks x (relu(conv1), relu(conv2 + r))
            # and the stem's relu
            gm, sites = t.fuse_epilogues(model)
            assert sites == 18                                 # ... and the head: average pool + fc in one call
            assert not any(n.op == "call_function" and n.target in (torch.relu, torch.add) for n in gm.graph.nodes)
            assert "maxpool" not in [n.target for n in gm.graph.nodes if n.op == "call_module"]     # taken into the stem's call
            got16f = gm(x)
        finally:
            t.set_compact_output_dtype(prev)
        got32f = gm(x)                                     # the fused graph in fp32 as well
        assert torch.allclose(got32f, got, rtol=1e-4, atol=1e-4 * want.abs().max().item())
        assert got16f.dtype == torch.float16
        assert torch.allclose(got16f.float(), got16.float(), rtol=5e-3, atol=5e-3 * want.abs().max().item())
        # fp32 tensors pass through the replaced modules to PyTorch's pooling
        assert torch.allclose(model(x), got, rtol=1e-5, atol=1e-5 * want.abs().max().item())
    assert got16p.dtype == torch.float16
    assert torch.allclose(got16p.float(), got16.float(), rtol=2e-3, atol=2e-3 * want.abs().max().item())
    assert torch.allclose(got, want, rtol=5e-3, atol=5e-3 * want.abs().max().item())
    assert got16.dtype == torch.float16 and torch.allclose(got16.float(), want, rtol=3e-2, atol=3e-2 * want.abs().max().item())
    with pytest.raises(ValueError):
        t.set_compact_output_dtype(torch.bfloat16)


class _Patterns(torch.nn.Module):
    """One site of every pattern fuse_epilogues recognises, and three it must leave alone."""

    def __init__(self):
        super().__init__()
        nn = torch.nn
        self.a = nn.Conv2d(8, 16, 3, 1, 1, bias=True)         # relu module
        self.act = nn.ReLU(inplace=True)
        self.b = nn.Conv2d(16, 16, 3, 1, 1, bias=False)        # += residual, then .relu()
        self.c = nn.Conv2d(16, 16, 1, bias=False)              # residual on the left, no relu
        self.d = nn.Conv2d(16, 16, 3, 1, 1, groups=16, bias=False)   # depthwise, F.relu
        self.e = nn.Conv2d(16, 16, 1, bias=False)              # used twice: stays
        self.f = nn.Conv2d(16, 16, 1, bias=False)              # BatchNorm in between: stays
        self.bn = nn.BatchNorm2d(16)
        self.g = nn.Conv2d(16, 16, 1, bias=False)              # x + x of its own output: stays
        self.head = nn.Linear(16, 10)                          # torch.relu on a linear layer

    def forward(self, x):
        h = self.act(self.a(x))
        y = self.b(h)
        y += h
        y = y.relu()
        z = h + self.c(y)
        z = torch.nn.functional.relu(self.d(z))
        e = self.e(z)
        z = e + torch.tanh(e)
        z = torch.relu(self.bn(self.f(z)))
        g = self.g(z)
        z = g + g
        return torch.relu(self.head(z.mean(dim=(2, 3))))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_fuse_epilogues_patterns(cuda, dtype):
    import tmq_amd as t
    torch.manual_seed(3)
    net = _Patterns()
    ctrl = t.QuantizationControl(post_scale=True)
    t.quantize_model(net, ctrl)
    _randomize_bn(net, torch.Generator().manual_seed(3))
    net.to(cuda).eval()
    ctrl.quantize()
    t.compressed_state_dict(net, strong=False)
    x = torch.randn(3, 8, 12, 10, device=cuda)
    prev = t.set_compact_output_dtype(dtype)
    try:
        with torch.no_grad():
            want = net(x)
            gm, sites = t.fuse_epilogues(net)
            got = gm(x)
    finally:
        t.set_compact_output_dtype(prev)
    assert sites == 5                                          # a, b, c, d, head
    calls = [n.target for n in gm.graph.nodes if n.op == "call_module"]
    assert sum(str(c).startswith("_fused_") for c in calls) == 5
    assert {"e", "f", "g", "bn"} <= set(calls) and not {"a", "b", "c", "d", "head", "act"} & set(calls)
    tol = 2e-3 if dtype == torch.float16 else 1e-5
    assert got.dtype == want.dtype and torch.allclose(got.float(), want.float(), rtol=tol, atol=tol * want.abs().max().item())


class _Opening(torch.nn.Module):
    def __init__(self, pool):
        super().__init__()
        nn = torch.nn
        self.conv1 = nn.Conv2d(3, 64, 7, 2, 3, bias=False)
        self.bn1 = nn.BatchNorm2d(64)
        self.relu = nn.ReLU(inplace=True)
        self.maxpool = pool
        self.conv2 = nn.Conv2d(64, 16, 1, bias=True)

    def forward(self, x):
        return self.conv2(self.maxpool(self.relu(self.bn1(self.conv1(x)))))


@pytest.mark.parametrize("native_pooling", [False, True])
def test_fuse_epilogues_takes_the_opening_maxpool(cuda, native_pooling):
    """maxpool(relu(conv(x))) with a 3 x 3 / 2 / 1 pool becomes one call: the same bits as the separate modules in
    fp16, PyTorch's pooling as before in fp32; any other pool stays a module of its own."""
    import tmq_amd as t
    nn = torch.nn
    for pool, taken in ((nn.MaxPool2d(3, 2, 1), True), (nn.MaxPool2d(2, 2), False), (nn.MaxPool2d(3, 2, 1, ceil_mode=True), False)):
        torch.manual_seed(4)
        net = _Opening(pool)
        ctrl = t.QuantizationControl(post_scale=True)
        t.quantize_model(net, ctrl)
        _randomize_bn(net, torch.Generator().manual_seed(4))
        net.to(cuda).eval()
        ctrl.quantize()
        t.compressed_state_dict(net, strong=False)
        x = torch.randn(3, 3, 64, 72, device=cuda)
        with torch.no_grad():
            t.fold_batchnorm(net)
            if native_pooling:
                t.use_native_pooling(net)
            want32 = net(x)
            prev = t.set_compact_output_dtype(torch.float16)
            try:
                want16 = net(x)
                gm, sites = t.fuse_epilogues(net)
                got16 = gm(x)
            finally:
                t.set_compact_output_dtype(prev)
            got32 = gm(x)
        calls = [n.target for n in gm.graph.nodes if n.op == "call_module"]
        assert sites == 1 and ("maxpool" in calls) == (not taken)
        assert got16.dtype == torch.float16 and torch.equal(got16, want16)
        assert got32.dtype == torch.float32 and torch.allclose(got32, want32, rtol=1e-5, atol=1e-5 * want32.abs().max().item())


def test_graphed_forward_replays_equal_eager(cuda):
    """The fused inference graph of a small network recorded as a HIP graph: every replay, with eager work and
    synchronisations in between and with new inputs, gives the eager result; a second input shape records its own
    graph."""
    import tmq_amd as t
    torch.manual_seed(6)
    net = _Opening(torch.nn.MaxPool2d(3, 2, 1))
    ctrl = t.QuantizationControl(post_scale=True)
    t.quantize_model(net, ctrl)
    _randomize_bn(net, torch.Generator().manual_seed(6))
    net.to(cuda).eval()
    ctrl.quantize()
    t.compressed_state_dict(net, strong=False)
    prev = t.set_compact_output_dtype(torch.float16)
    try:
        with torch.no_grad():
            t.fold_batchnorm(net)
            t.use_native_pooling(net)
            gm, _ = t.fuse_epilogues(net)
            graphed = t.GraphedForward(gm)
            for rep in range(4):
                x = torch.randn(3, 3, 64, 72, device=cuda).half()
                want = gm(x)
                torch.cuda.synchronize()
                got = graphed(x)
                assert torch.equal(got, want), rep
                _ = gm(torch.randn(2, 3, 32, 40, device=cuda).half())        # eager work between the replays
            x2 = torch.randn(1, 3, 48, 48, device=cuda).half()
            assert torch.equal(graphed(x2), gm(x2)) and len(graphed._graphs) == 2
            with pytest.raises(RuntimeError):
                graphed(x2.cpu())
    finally:
        t.set_compact_output_dtype(prev)


def test_graphed_forward_follows_changed_weights(cuda):
    """A recorded graph replays raw addresses of the layers' native weight buffers: after the weights of a layer
    were replaced (load_state_dict and its like rebuild those buffers) the next call must record anew and give the
    eager result of the new weights; reset() does the same on request; so does a changed output dtype."""
    import tmq_amd as t
    torch.manual_seed(7)

    def make(seed):
        torch.manual_seed(seed)
        net = _Opening(torch.nn.MaxPool2d(3, 2, 1))
        ctrl = t.QuantizationControl(post_scale=True)
        t.quantize_model(net, ctrl)
        _randomize_bn(net, torch.Generator().manual_seed(6))
        net.to(cuda).eval()
        ctrl.quantize()
        return net

    net, other = make(7), make(8)
    sd_other = t.compressed_state_dict(other, strong=False)
    t.compressed_state_dict(net, strong=False)
    x = torch.randn(2, 3, 64, 72, device=cuda).half()
    prev = t.set_compact_output_dtype(torch.float16)
    try:
        with torch.no_grad():
            graphed = t.GraphedForward(net)
            first = graphed(x).clone()
            assert torch.equal(first, net(x))
            # new weights into the same modules: the compact tensors (and with them the native buffers) are replaced
            t.load_compressed_state_dict(net, sd_other)
            junk = [torch.full((1 << 18,), 7, dtype=torch.int32, device=cuda) for _ in range(8)]   # reuse freed memory
            want = net(x)
            assert not torch.equal(want, first)
            got = graphed(x)
            assert torch.equal(got, want)
            del junk
            # a switch the recording depends on
            t.set_compact_output_dtype(torch.float32)
            want32 = net(x)
            got32 = graphed(x)
            assert got32.dtype == want32.dtype and torch.equal(got32, want32)
            graphed.reset()
            assert graphed._graphs == {} and torch.equal(graphed(x), want32)
    finally:
        t.set_compact_output_dtype(prev)


def test_optimize_for_inference_one_call(cuda):
    """optimize_for_inference = fold_batchnorm + fp16 hand-over + native pooling + fuse_epilogues + GraphedForward:
    same values as those steps applied by hand, the global output dtype left as it was, misuse refused."""
    import tmq_amd as t
    torch.manual_seed(9)

    def make():
        torch.manual_seed(9)
        net = _Opening(torch.nn.MaxPool2d(3, 2, 1))
        ctrl = t.QuantizationControl(post_scale=True)
        t.quantize_model(net, ctrl)
        _randomize_bn(net, torch.Generator().manual_seed(9))
        net.to(cuda).eval()
        ctrl.quantize()
        return net

    net = make()
    with pytest.raises(RuntimeError):
        t.optimize_for_inference(net)                            # layers not compact yet
    t.compressed_state_dict(net, strong=False)
    by_hand = make()
    t.compressed_state_dict(by_hand, strong=False)
    x = torch.randn(3, 3, 64, 72, device=cuda).half()
    prev = t.set_compact_output_dtype(torch.float16)
    try:
        with torch.no_grad():
            t.fold_batchnorm(by_hand)
            t.use_native_pooling(by_hand)
            want = t.fuse_epilogues(by_hand)[0](x)
    finally:
        t.set_compact_output_dtype(prev)
    assert prev == torch.float32
    session = t.optimize_for_inference(net)
    assert session.fused_sites >= 1 and len(session.folded) >= 1
    for _ in range(3):
        got = session(x)
        assert torch.equal(got, want)
    assert t.set_compact_output_dtype(torch.float32) == torch.float32        # untouched outside the call
    eager = t.optimize_for_inference(net, graph=False)            # idempotent on an already optimised model
    assert torch.equal(eager(x), want)


class _SmallImageNet(torch.nn.Module):
    """A CIFAR-style network: 3 x 3 / stride 1 opening on three channels, one residual block, a linear head."""

    def __init__(self):
        super().__init__()
        nn = torch.nn
        self.conv1 = nn.Conv2d(3, 32, 3, 1, 1, bias=False)
        self.bn1 = nn.BatchNorm2d(32)
        self.conv2 = nn.Conv2d(32, 32, 3, 1, 1, bias=False)
        self.bn2 = nn.BatchNorm2d(32)
        self.head = nn.Linear(32, 10)

    def forward(self, x):
        h = torch.relu(self.bn1(self.conv1(x)))
        y = torch.relu(self.bn2(self.conv2(h)) + h)
        return self.head(y.mean(dim=(2, 3)))


@pytest.mark.parametrize("in_dtype", [torch.float16, torch.float32])
def test_optimize_for_inference_stride_one_opening(cuda, in_dtype):
    """The opening of a small-image network (horizontal stride 1) runs in its pixel-pair form inside the optimised
    model, eager and as graph replays, with the folded BatchNorm and the ReLU in its epilogue: same values as the
    generic loader gives for the same model, and the float model's within fp16 tolerance."""
    import tmq_amd as t

    def make():
        torch.manual_seed(21)
        net = _SmallImageNet()
        ctrl = t.QuantizationControl(post_scale=True)
        t.quantize_model(net, ctrl)
        _randomize_bn(net, torch.Generator().manual_seed(21))
        net.to(cuda).eval()
        ctrl.quantize()
        return net

    net = make()
    x = torch.randn(8, 3, 32, 32, device=cuda).to(in_dtype)
    with torch.no_grad():
        want = net(x.float())
    t.compressed_state_dict(net, strong=False)
    generic = make()
    t.compressed_state_dict(generic, strong=False)
    generic.conv1._pixelpair_plan = lambda x: None
    assert net.conv1._pixelpair_plan(x) is not None
    session = t.optimize_for_inference(net)
    reference = t.optimize_for_inference(generic, graph=False)(x)
    for _ in range(3):
        got = session(x)
        assert torch.allclose(got.float(), reference.float(), rtol=2e-3, atol=2e-3 * want.abs().max().item())
        assert torch.allclose(got.float(), want, rtol=3e-2, atol=3e-2 * want.abs().max().item())
