"""The whole-step multi-tensor launches: S(w) of every layer (+ the quantization loss) in one forward
launch, g*S'(w) + (u/n)*Q'(w) of every layer in one backward launch, and the autograd node that the
Python API builds from them.

Bar: bit-exact against the CPU oracle per tensor (the kernels spell the reference's fp32 op chain),
1e-6 relative for the loss sums. The API-level tests capture the gradient that reaches each layer's
soft weights (dL/dy, computed by PyTorch's own convolution backward) and require weight.grad to be the
oracle's chain applied to exactly that gradient, bit for bit.
"""
import numpy as np
import pytest
import torch
from torch import nn

pytestmark = pytest.mark.gpu

SIZES = [1, 5, 63, 64, 2047, 2048, 2049, 9408, 36864, 147456 + 3, 4096, 7]


def _tensors(sizes, seed):
    rng = np.random.default_rng(seed)
    ws, gs = [], []
    for n in sizes:
        w = rng.uniform(-1.02, 1.02, n).astype(np.float32)
        m = rng.random(n) < 0.1
        w[m] = (rng.integers(-1, 2, n) + rng.uniform(-0.02, 0.02, n)).astype(np.float32)[m]
        ws.append(w)
        gs.append(rng.standard_normal(n).astype(np.float32))
    return ws, gs


def _bits(t):
    return t.detach().cpu().numpy().reshape(-1).view(np.uint32)


def _expected_dw(oracle, w, g, up, d, sharp, p):
    """The reference's two backward terms, each rounded to fp32, added once."""
    t1 = oracle.softstep_bwd(w, g, d, 1.0) if g is not None else None
    t2 = None
    if up is not None:
        s = np.float32(up) / np.float32(w.size)
        t2 = oracle.deriv_bwd(w, np.full(w.size, s, dtype=np.float32), sharp, p)
    if t1 is None:
        return t2
    return t1 if t2 is None else (t1 + t2).astype(np.float32)


def _backends():
    from tmq_amd import ops
    out = [("ctypes", ops)]
    if ops.ext is not None:
        out.append(("extension", ops.ext))
    return out


@pytest.mark.parametrize("d", [0.1, 2.236133, 6.0])
def test_forward_all_matches_oracle_per_tensor(cuda, oracle, d):
    ws, _ = _tensors(SIZES, 11)
    tws = [torch.from_numpy(w).to(cuda) for w in ws]
    for name, b in _backends():
        ys, loss = b.softstep_fwd_all(tws, d, True, 5.0, 5e-4)
        assert len(ys) == len(ws)
        total = np.float32(0)
        for i, (w, y) in enumerate(zip(ws, ys)):
            assert y.shape == tws[i].shape and y.data_ptr() % 256 == 0
            assert np.array_equal(_bits(y), oracle.softstep_fwd(w, d).view(np.uint32)), (name, i)
            mean = np.float32(oracle.deriv_fwd(w, 5.0, 5e-4).astype(np.float64).sum() / w.size)
            total = mean if i == 0 else np.float32(total + mean)
        assert abs(loss.item() - float(total)) <= 1e-6 * abs(float(total)), (name, loss.item(), float(total))
        ys2, none = b.softstep_fwd_all(tws, d, False, 5.0, 0.0)
        assert none is None
        for y, y2 in zip(ys, ys2):
            assert torch.equal(y, y2)
    for w, tw in zip(ws, tws):
        assert np.array_equal(_bits(tw), w.view(np.uint32)), "inputs must not be mutated"


@pytest.mark.parametrize("d,use_loss", [(0.1, True), (3.0004, True), (6.0, False)])
def test_backward_all_matches_oracle_per_tensor(cuda, oracle, d, use_loss):
    ws, gs = _tensors(SIZES, 12)
    tws = [torch.from_numpy(w).to(cuda) for w in ws]
    tgs = [torch.from_numpy(g).to(cuda) for g in gs]
    tgs[3] = None                                  # a layer the forward pass did not use
    tgs[8] = None
    up = 0.73 if use_loss else None
    tup = torch.tensor(up, device=cuda) if use_loss else None
    for name, b in _backends():
        dws = b.softstep_bwd_all(tws, tgs, tup, d, 5.0, 5e-4)
        for i, w in enumerate(ws):
            g = gs[i] if tgs[i] is not None else None
            want = _expected_dw(oracle, w, g, up, d, 5.0, 5e-4)
            if want is None:
                assert dws[i] is None, (name, i)
                continue
            assert np.array_equal(_bits(dws[i]), want.view(np.uint32)), (name, i, np.abs(dws[i].cpu().numpy() - want).max())


def test_more_tensors_than_one_launch_holds(cuda, oracle):
    """150 tensors: three launches of at most 64; the loss total carries over between them in order."""
    sizes = [int(s) for s in np.random.default_rng(5).integers(1, 5000, 150)]
    ws, gs = _tensors(sizes, 13)
    tws = [torch.from_numpy(w).to(cuda) for w in ws]
    tgs = [torch.from_numpy(g).to(cuda) for g in gs]
    from tmq_amd import ops
    ys, loss = ops.softstep_fwd_all(tws, 4.72, True, 5.0, 1e-3)
    total = np.float32(0)
    for i, (w, y) in enumerate(zip(ws, ys)):
        assert np.array_equal(_bits(y), oracle.softstep_fwd(w, 4.72).view(np.uint32)), i
        mean = np.float32(oracle.deriv_fwd(w, 5.0, 1e-3).astype(np.float64).sum() / w.size)
        total = mean if i == 0 else np.float32(total + mean)
    assert abs(loss.item() - float(total)) <= 2e-6 * abs(float(total))
    tup = torch.tensor(1.0, device=cuda)
    dws = ops.softstep_bwd_all(tws, tgs, tup, 4.72, 5.0, 1e-3)
    for i, w in enumerate(ws):
        want = _expected_dw(oracle, w, gs[i], 1.0, 4.72, 5.0, 1e-3)
        assert np.array_equal(_bits(dws[i]), want.view(np.uint32)), i


def test_unaligned_views_and_errors(cuda, oracle):
    from tmq_amd import ops, _capi
    base = torch.from_numpy(np.random.default_rng(3).uniform(-1, 1, 5000).astype(np.float32)).to(cuda)
    views = [base[1:1001], base[1003:4000]]          # 4-byte aligned only
    ys, _ = ops.softstep_fwd_all(views, 3.0004)
    for v, y in zip(views, ys):
        assert np.array_equal(_bits(y), oracle.softstep_fwd(v.cpu().numpy(), 3.0004).view(np.uint32))
    with pytest.raises(ValueError):
        ops.softstep_fwd_all([], 3.0)
    with pytest.raises(RuntimeError):
        ops.softstep_fwd_all([base.cpu()], 3.0)
    with pytest.raises(ValueError):
        ops.softstep_fwd_all([base.half()], 3.0)
    with pytest.raises(_capi.TmqError):
        ops.softstep_fwd_all([base], -1.0)
    assert ops.softstep_bwd_all([base], [None], None, 3.0) == [None]


# ---- the autograd node behind the API ----------------------------------------------------------------
def _capture_upstream(ctrl):
    """Record dL/dy for every layer: wrap the controller's hand-out of soft weights with a tensor hook."""
    seen = {}
    inner = ctrl._soft_weight_of

    def wrapped(node):
        y = inner(node)
        if y is not None and y.requires_grad:
            y.register_hook(lambda g, node=node: seen.__setitem__(id(node), seen.get(id(node), 0) + g.detach().clone()))
        return y
    ctrl._soft_weight_of = wrapped
    return seen


def _check_grads(oracle, ctrl, seen, up, p, nodes=None):
    for node in (nodes if nodes is not None else ctrl._registry.values()):
        w = node.weight.detach().cpu().numpy().reshape(-1)
        g = seen.get(id(node))
        g = g.cpu().numpy().reshape(-1) if g is not None else None
        want = _expected_dw(oracle, w, g, up, ctrl.digamma, 5.0, p)
        got = node.weight.grad
        if want is None:
            assert got is None
            continue
        assert got.shape == node.weight.shape and got.is_contiguous()
        assert np.array_equal(_bits(got), want.view(np.uint32)), (node.layer_name, np.abs(got.cpu().numpy().reshape(-1) - want).max())


def test_resnet18_step_gradients_equal_oracle_chain(cuda, oracle):
    """ResNet-18 / 102 classes, all 21 quantized layers: one multi-tensor launch forward, one backward;
    every weight.grad equals the oracle chain applied to the gradient PyTorch delivered for that layer."""
    import tmq_amd as t
    from bench_models import ResNet18
    torch.manual_seed(30)
    model = ResNet18(102)
    ctrl = t.QuantizationControl(epoch_knots=t.QuantizationScheduleBuilder.default_schedule(150), qpenalty_range=(5e-4, 5e-4))
    t.quantize_model(model, ctrl)
    model.to(cuda).train()
    for e in range(76):
        ctrl.step(e)
    assert len(ctrl._registry) == 21 and abs(ctrl.digamma - 2.236133) < 1e-5
    x = torch.randn(4, 3, 64, 64, generator=torch.Generator().manual_seed(30)).to(cuda)
    labels = torch.randint(0, 102, (4,), generator=torch.Generator().manual_seed(31)).to(cuda)
    opt = torch.optim.Adam(model.parameters(), lr=0.1)
    launches = []
    from tmq_amd import tmq as tm
    fwd, bwd = tm._b.softstep_fwd_all, tm._b.softstep_bwd_all

    class Spy:
        softstep_fwd_all = staticmethod(lambda *a: (launches.append("fwd"), fwd(*a))[1])
        softstep_bwd_all = staticmethod(lambda *a: (launches.append("bwd"), bwd(*a))[1])

        def __getattr__(self, k):
            return getattr(tm._b_real, k)
    tm._b_real, tm._b = tm._b, Spy()
    try:
        for it in range(2):                        # the second step fuses the loss into the forward launch
            seen = _capture_upstream(ctrl)
            opt.zero_grad(set_to_none=True)
            del launches[:]
            out = model(x)
            ql = ctrl.quantization_loss()
            (nn.functional.cross_entropy(out, labels) + 3.0 * ql).backward()
            del ctrl.__dict__["_soft_weight_of"]
            if it == 0:
                assert launches == ["fwd", "bwd", "bwd"]          # loss asked for the first time: its own node
                # (two backward launches add up through autograd; compare with tolerance only)
            else:
                assert launches == ["fwd", "bwd"], launches
                _check_grads(oracle, ctrl, seen, 3.0, 5e-4)
                want_ql = np.float32(0)
                for i, node in enumerate(ctrl._registry.values()):
                    w = node.weight.detach().cpu().numpy().reshape(-1)
                    m = np.float32(oracle.deriv_fwd(w, 5.0, 5e-4).astype(np.float64).sum() / w.size)
                    want_ql = m if i == 0 else np.float32(want_ql + m)
                assert abs(ql.item() - float(want_ql)) <= 1e-6 * float(want_ql)
            opt.step()
            ctrl.clamp()
            for node in ctrl._registry.values():
                assert node.weight.min() >= -1 and node.weight.max() <= 1
    finally:
        tm._b = tm._b_real
        del tm._b_real


def _small_net(t, cuda, qpen=5e-4):
    ctrl = t.QuantizationControl(epoch_knots=(15, 60, 70, 80, 100), qpenalty_range=(qpen, qpen))
    ctrl.digamma = 3.0004
    torch.manual_seed(3)
    net = nn.Sequential(nn.Conv2d(3, 8, 3, padding=1), nn.ReLU(), nn.Conv2d(8, 8, 3, padding=1), nn.ReLU(),
                        nn.AdaptiveAvgPool2d(1), nn.Flatten(), nn.Linear(8, 5))
    t.quantize_model(net, ctrl)
    return ctrl, net.to(cuda).train()


def test_two_passes_accumulate_and_eval_pass_in_between(cuda, oracle):
    """Gradient accumulation (two forward / backward passes on unchanged weights) sums the oracle's
    gradients; a no-grad evaluation pass in between starts a pass of its own and leaves no graph."""
    import tmq_amd as t
    ctrl, net = _small_net(t, cuda)
    x1, x2 = torch.randn(2, 3, 8, 8, device=cuda), torch.randn(2, 3, 8, 8, device=cuda)
    ctrl.quantization_loss()                      # from now on the forward launch carries the loss
    wants = None
    for x in (x1, x2):
        seen = _capture_upstream(ctrl)
        (net(x).square().mean() + ctrl.quantization_loss()).backward()
        del ctrl.__dict__["_soft_weight_of"]
        with torch.no_grad():
            y_eval = net(x)
        assert not y_eval.requires_grad
        now = []
        for node in ctrl._registry.values():
            w = node.weight.detach().cpu().numpy().reshape(-1)
            now.append(_expected_dw(oracle, w, seen[id(node)].cpu().numpy().reshape(-1), 1.0, ctrl.digamma, 5.0, 5e-4))
        wants = now if wants is None else [(a + b).astype(np.float32) for a, b in zip(wants, now)]
    for node, want in zip(ctrl._registry.values(), wants):
        assert np.array_equal(_bits(node.weight.grad), want.view(np.uint32)), node.layer_name


def test_shared_layer_partial_use_frozen_weight_and_other_penalty(cuda, oracle):
    import tmq_amd as t
    ctrl, net = _small_net(t, cuda)
    conv1, conv2, fc = net[0], net[2], net[6]
    ctrl.quantization_loss()
    # (a) conv2 used twice in one pass, fc not used at all, conv1 frozen
    conv1.weight.requires_grad_(False)
    seen = _capture_upstream(ctrl)
    x = torch.randn(2, 3, 8, 8, device=cuda)
    h = torch.relu(conv1(x))
    out = conv2(torch.relu(conv2(h)))
    (out.square().mean() + 2.0 * ctrl.quantization_loss()).backward()
    del ctrl.__dict__["_soft_weight_of"]
    assert conv1.weight.grad is None
    w2 = conv2.weight.detach().cpu().numpy().reshape(-1)
    # the second use started a pass of its own (each layer's soft weights are handed out once per pass);
    # the loss node belongs to that last pass. Total gradient = sum of the S' terms + the loss term.
    g2 = seen[id(conv2)].cpu().numpy().reshape(-1)
    got = conv2.weight.grad.cpu().numpy().reshape(-1)
    ref = _expected_dw(oracle, w2, g2, 2.0, ctrl.digamma, 5.0, 5e-4)
    assert np.max(np.abs(got - ref)) <= 2e-6 * max(1e-3, np.abs(ref).max())
    wf = fc.weight.detach().cpu().numpy().reshape(-1)
    want_fc = _expected_dw(oracle, wf, None, 2.0, ctrl.digamma, 5.0, 5e-4)
    assert np.array_equal(_bits(fc.weight.grad), want_fc.view(np.uint32))
    # (b) a penalty other than the controller's: the stand-alone loss node, same values as per-layer calls
    for p_ in net.parameters():
        p_.grad = None
    ql = ctrl.quantization_loss(penalty=1e-2)
    per = sum(node.quantization_loss(1e-2, 5.0) for node in ctrl._registry.values())
    assert abs(ql.item() - per.item()) <= 1e-6 * abs(per.item())
    ql.backward()
    want_fc = _expected_dw(oracle, wf, None, 1.0, ctrl.digamma, 5.0, 1e-2)
    assert np.array_equal(_bits(fc.weight.grad), want_fc.view(np.uint32))
    assert conv1.weight.grad is None


def test_changed_hardness_or_weights_start_a_new_pass(cuda, oracle):
    import tmq_amd as t
    ctrl, net = _small_net(t, cuda, qpen=0.0)
    x = torch.randn(2, 3, 8, 8, device=cuda)
    with torch.no_grad():
        a = net(x)
        ctrl.digamma = 6.0
        b = net(x)
        assert not torch.equal(a, b)
        ctrl._soft_weight_of(net[2])                              # opens a pass; net[0]'s result is still unclaimed
        net[0].weight.mul_(0.5)                                   # in place: the version counter moves
        y = ctrl._soft_weight_of(net[0])
        assert np.array_equal(_bits(y), oracle.softstep_fwd(net[0].weight.cpu().numpy().reshape(-1), 6.0).view(np.uint32))
        ctrl._soft_weight_of(net[2])
        net[0].weight.data = net[0].weight.data * 0.5              # new storage
        y = ctrl._soft_weight_of(net[0])
        assert np.array_equal(_bits(y), oracle.softstep_fwd(net[0].weight.cpu().numpy().reshape(-1), 6.0).view(np.uint32))
    ctrl.inference()
    with torch.no_grad():
        c = net(x)                                                # inference mode: raw weights, no staircase
    assert torch.isfinite(c).all()


class _TwoHeads(nn.Module):
    """A trunk and two heads of which a forward uses one."""

    def __init__(self):
        super().__init__()
        self.trunk = nn.Linear(32, 48)
        self.head_a = nn.Linear(48, 8)
        self.head_b = nn.Linear(48, 8)

    def forward(self, x, which):
        h = torch.relu(self.trunk(x))
        return self.head_a(h) if which == "a" else self.head_b(h)


def test_branches_used_in_alternate_steps_backward_each_step(cuda, oracle):
    """A registered layer that the previous forward skipped must not be handed that pass's result once its
    autograd node has run backward (no quantization loss in the step, so only the soft-step node exists)."""
    import tmq_amd as t
    torch.manual_seed(11)
    net = _TwoHeads()
    ctrl = t.QuantizationControl(epoch_knots=t.QuantizationScheduleBuilder.default_schedule(150))
    t.quantize_model(net, ctrl)
    net.to(cuda).train()
    x = torch.randn(4, 32, device=cuda)
    for step, which in enumerate("abab"):
        for p in net.parameters():
            p.grad = None
        net(x, which).square().mean().backward()                 # raised "backward through the graph a second time"
        used, idle = (net.head_a, net.head_b) if which == "a" else (net.head_b, net.head_a)
        assert used.weight.grad is not None and idle.weight.grad is None, step
        assert torch.isfinite(net.trunk.weight.grad).all()
    # two forwards, then one backward through both: the second head still joins the first pass's node
    for p in net.parameters():
        p.grad = None
    (net(x, "a").square().mean() + net(x, "b").square().mean()).backward()
    assert net.head_a.weight.grad is not None and net.head_b.weight.grad is not None


def test_layer_the_controller_cannot_serve_does_not_relaunch_the_others(cuda, oracle):
    """A registered layer whose weights the multi-tensor launch cannot take (here: a compact layer) goes its own
    way without restarting the pass of the layers that are served."""
    import tmq_amd as t
    from tmq_amd import tmq as tmq_mod
    torch.manual_seed(12)
    net = nn.Sequential(nn.Linear(16, 16), nn.ReLU(), nn.Linear(16, 16), nn.ReLU(), nn.Linear(16, 4))
    ctrl = t.QuantizationControl()
    t.quantize_model(net, ctrl)
    net.to(cuda).train()
    calls = []
    orig = tmq_mod._StepState.run.__func__
    tmq_mod._StepState.run = classmethod(lambda cls, c: (calls.append(1), orig(cls, c))[1])
    try:
        st = tmq_mod._StepState.run(ctrl)
        ctrl._step = st
        calls.clear()
        st.unserved.add(id(net[2]))                              # as run() marks a layer it leaves out
        assert ctrl._soft_weight_of(net[2]) is None and calls == []
        y0 = ctrl._soft_weight_of(net[0])
        assert y0 is st.ys[0] and calls == []
    finally:
        tmq_mod._StepState.run = classmethod(orig)
