"""End-to-end parity of the Python API on the GPU.

Config 1 (README MLP, one QAT step): the golden fixture was recorded from the reference's own CPU
path (tests/golden/make_reference_golden.py). The TMQ kernels are bit-exact; F.linear, BatchNorm,
cross-entropy and Adam are PyTorch's on either device and differ in summation order, hence the
tolerances below (1e-5 relative on losses, 2e-6 of the gradient's scale on gradients).
"""
import os

import numpy as np
import pytest
import torch
from torch import nn

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = np.load(os.path.join(ROOT, "tests", "golden", "reference_golden.npz"))


class MLP(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc1 = nn.Linear(256, 128)
        self.bn1 = nn.BatchNorm1d(128)
        self.fc2 = nn.Linear(128, 10)
        self.bn2 = nn.BatchNorm1d(10)

    def forward(self, x):
        return self.bn2(self.fc2(torch.relu(self.bn1(self.fc1(x)))))


@pytest.mark.parametrize("case", range(int(GOLD["mlp_cases"])))
def test_readme_mlp_qat_step_matches_reference_cpu_path(cuda, case):
    import tmq_amd as t
    pre = f"mlp{case}_"
    epoch, qpen = int(GOLD[pre + "epoch"]), float(GOLD[pre + "qpenalty"])
    torch.manual_seed(0)
    model = MLP()
    qr = None if (qpen == 0.0) else (qpen, qpen)
    ctrl = t.QuantizationControl(epoch_knots=t.QuantizationScheduleBuilder.default_schedule(150), qpenalty_range=qr)
    t.quantize_model(model, ctrl)
    sd = {k[len(pre) + 5:]: torch.from_numpy(GOLD[k]) for k in GOLD.files if k.startswith(pre + "init.")}
    model.load_state_dict(sd)
    model.to(cuda)
    for e in range(epoch + 1):
        ctrl.step(e)
    assert ctrl.digamma == float(GOLD[pre + "digamma"]) and ctrl.qpenalty == qpen
    x = torch.from_numpy(GOLD[pre + "x"]).to(cuda)
    labels = torch.from_numpy(GOLD[pre + "labels"]).to(cuda)
    opt = torch.optim.Adam(model.parameters(), lr=1e-3)
    model.train()
    opt.zero_grad()
    loss = nn.functional.cross_entropy(model(x), labels)
    ql = ctrl.quantization_loss()
    (loss + ql).backward()
    assert abs(loss.item() - float(GOLD[pre + "loss"])) <= 1e-5 * abs(float(GOLD[pre + "loss"]))
    assert abs(ql.item() - float(GOLD[pre + "qloss"])) <= 1e-5 * abs(float(GOLD[pre + "qloss"])) + 1e-12
    for name, p in model.named_parameters():
        key = pre + "grad." + name
        if key not in GOLD.files:
            continue
        want = GOLD[key]
        got = p.grad.cpu().numpy()
        tol = 2e-6 * max(1e-3, np.max(np.abs(want))) if "weight" in name else 1e-6 + 1e-4 * np.max(np.abs(want))
        assert np.max(np.abs(got - want)) <= tol + 2e-5 * np.max(np.abs(want)), (name, np.max(np.abs(got - want)))
    wptr = model.fc1.weight.data_ptr()
    opt.step()
    ctrl.clamp()
    assert model.fc1.weight.data_ptr() == wptr              # clamp works in place
    for k in GOLD.files:
        if k.startswith(pre + "after.") and k.endswith("weight") and "fc" in k:
            got = model.state_dict()[k[len(pre) + 6:]].cpu().numpy()
            assert np.max(np.abs(got - GOLD[k])) <= 2e-5, k        # Adam's sign-like first step amplifies tiny grad noise
            assert got.min() >= -1.0 and got.max() <= 1.0


def _oracle_step(weights, x, labels, digamma, qpen):
    """The same step with the oracle's torch op chain wrapped for autograd, on the CPU."""
    from oracle import torch_path as tp

    class S(torch.autograd.Function):
        @staticmethod
        def forward(ctx, w):
            ctx.save_for_backward(w)
            return tp.softstep_fwd(w, digamma)

        @staticmethod
        def backward(ctx, g):
            return tp.softstep_bwd(ctx.saved_tensors[0], digamma, 1.0, g)

    class Q(torch.autograd.Function):
        @staticmethod
        def forward(ctx, w):
            ctx.save_for_backward(w)
            return tp.deriv_fwd(w, 5.0, qpen)

        @staticmethod
        def backward(ctx, g):
            return tp.deriv_bwd(ctx.saved_tensors[0], 5.0, qpen, g)

    ws = [w.clone().requires_grad_(True) for w in weights]
    h = torch.relu(nn.functional.linear(x, S.apply(ws[0])))
    out = nn.functional.linear(h, S.apply(ws[1]))
    loss = nn.functional.cross_entropy(out, labels)
    ql = sum(torch.mean(Q.apply(w)) for w in ws)
    (loss + ql).backward()
    return loss.item(), float(ql), [w.grad for w in ws]


@pytest.mark.parametrize("digamma,qpen", [(0.1, 0.0), (2.236133, 5e-4), (6.0, 2e-3)])
def test_two_layer_step_matches_oracle_chain(cuda, digamma, qpen):
    import tmq_amd as t
    g = torch.Generator().manual_seed(7)
    w1 = 2 * torch.rand(64, 96, generator=g) - 1
    w2 = 2 * torch.rand(10, 64, generator=g) - 1
    x = torch.randn(32, 96, generator=g)
    labels = torch.randint(0, 10, (32,), generator=g)
    ctrl = t.QuantizationControl(epoch_knots=(15, 60, 70, 80, 100), qpenalty_range=(qpen, qpen))
    ctrl.digamma = digamma
    l1 = t.Linear(96, 64, bias=False, ctrl=ctrl, quant_mode=t.QuantMode.TERNARY)
    l2 = t.Linear(64, 10, bias=False, ctrl=ctrl, quant_mode=t.QuantMode.TERNARY)
    ctrl.register_node("l1", l1)
    ctrl.register_node("l2", l2)
    l1.weight.data, l2.weight.data = w1.clone(), w2.clone()
    l1.to(cuda), l2.to(cuda)
    l1.train(), l2.train()
    loss = nn.functional.cross_entropy(l2(torch.relu(l1(x.to(cuda)))), labels.to(cuda))
    ql = ctrl.quantization_loss()
    (loss + ql).backward()
    oloss, oql, ograds = _oracle_step([w1, w2], x, labels, digamma, qpen)
    assert abs(loss.item() - oloss) <= 1e-5 * abs(oloss)
    assert abs(ql.item() - oql) <= 1e-5 * abs(oql) + 1e-12
    for lay, og in zip((l1, l2), ograds):
        err = (lay.weight.grad.cpu() - og).abs().max().item()
        assert err <= 3e-6 * max(1e-3, og.abs().max().item()) + 1e-9, err
    # per-layer API gives the same loss as the fused multi-tensor launch
    per = l1.quantization_loss(qpen, 5.0) + l2.quantization_loss(qpen, 5.0)
    assert abs(per.item() - ql.item()) <= 1e-6 * abs(ql.item()) + 1e-12
    # quantize: round(map(w)) equals the oracle, then idempotent
    ctrl.quantize()
    from tests import oracle_lib as oracle
    assert np.array_equal(l1.weight.data.cpu().numpy().reshape(-1), oracle.ternarize(w1.numpy(), digamma))
    before = l1.weight.data.clone()
    t.quantize_weights(nn.Sequential(l1, l2))
    assert torch.equal(l1.weight.data, before)


class SmallNet(nn.Module):
    def __init__(self):
        super().__init__()
        self.conv1 = nn.Conv2d(8, 16, 3, padding=1, bias=False)
        self.bn1 = nn.BatchNorm2d(16)
        self.conv2 = nn.Conv2d(16, 32, 3, stride=2, padding=1, bias=True)
        self.fc = nn.Linear(32, 10)

    def forward(self, x):
        x = torch.relu(self.bn1(self.conv1(x)))
        x = torch.relu(self.conv2(x))
        return self.fc(x.mean(dim=(2, 3)))


@pytest.mark.parametrize("strong", [False, True])
def test_compressed_state_dict_round_trip_and_compact_inference(cuda, strong, tmp_path):
    import tmq_amd as t
    torch.manual_seed(3)
    ctrl = t.QuantizationControl(epoch_knots=t.QuantizationScheduleBuilder.default_schedule(50))
    model = SmallNet()
    t.quantize_model(model, ctrl, prefix="")
    model.to(cuda)
    with torch.no_grad():
        model.conv2.bias.uniform_(-1, 1)
        model.bn1.running_mean.normal_(0, 0.1)
        model.bn1.running_var.uniform_(0.5, 2.0)
    ctrl.step(49)
    ctrl.quantize()                                   # weights are now exactly ternary
    model.eval()
    ctrl.inference()
    x = torch.randn(4, 8, 12, 12, device=cuda)
    ref = model(x)                                    # fp32 path on ternary-valued weights
    fp32_weights = {n: p.detach().clone() for n, p in model.named_parameters() if n.endswith("weight") and p.dim() > 1}
    sd = t.compressed_state_dict(model, strong=strong)
    kind = t.TensorType.COMPRESSED_TERNARY_32BIT if strong else t.TensorType.COMPACT_TERNARY_32BIT
    assert sd._metadata["conv1"]["tmq.tensor_type"] == kind.value
    assert tuple(sd._metadata["conv1"]["tmq.shape"]) == (16, 8, 3, 3) and sd._metadata["fc"]["tmq.quant"] == 1
    if strong:
        assert sd["conv1.weight"].dtype == torch.int8 and sd["conv1.weight"].dim() == 1
    else:
        assert sd["conv1.weight"].dtype == torch.int32 and tuple(sd["conv1.weight"].shape) == (8, 3, 3, 1)
        assert tuple(sd["fc.weight"].shape) == (32, 1)
    # the model itself was switched to compact inference and still gives the same answer
    assert model.conv1.compact and model.conv1.weight.dtype == torch.int32
    out_compact = model(x)
    assert (out_compact - ref).abs().max().item() <= 1e-3 * ref.abs().max().item()
    # save / load into a fresh model
    path = tmp_path / "m.pt"
    torch.save(sd, path)
    sd2 = torch.load(path, weights_only=False)
    ctrl2 = t.QuantizationControl()
    model2 = SmallNet()
    t.quantize_model(model2, ctrl2, prefix="")
    model2.to(cuda)
    t.load_compressed_state_dict(model2, sd2)
    model2.eval()
    assert model2.conv1.compact and model2.fc.compact and model2.conv1.weight.dtype == torch.int32
    assert model2.conv1.weight.is_cuda
    out2 = model2(x)
    assert (out2 - ref).abs().max().item() <= 1e-3 * ref.abs().max().item()
    # expand back to fp32 weights: exactly the ternary weights we started from
    t.expand_compact_layers(model2)
    for n, w in fp32_weights.items():
        assert torch.equal(dict(model2.named_parameters())[n].detach(), w), n
    assert not model2.conv1.compact
    out3 = model2(x)
    assert (out3 - ref).abs().max().item() <= 1e-5 * ref.abs().max().item()


def test_softstep_helpers_and_logging_api(cuda, oracle):
    import tmq_amd as t
    ctrl = t.QuantizationControl(epoch_knots=(15, 60, 70, 80, 100))
    ctrl.digamma = 3.0004
    w = torch.from_numpy(np.random.default_rng(0).uniform(-1.02, 1.02, 5000).astype(np.float32)).to(cuda)
    assert np.array_equal(t.SoftStep.map(w, ctrl).cpu().numpy(), oracle.softstep_map(w.cpu().numpy(), 3.0004))
    assert np.array_equal(t.SoftStep.dmap(w, ctrl).cpu().numpy(), oracle.softstep_dmap(w.cpu().numpy(), 3.0004))
    from oracle import torch_path as tp
    v = torch.from_numpy(np.random.default_rng(1).uniform(-4, 4, 5000).astype(np.float32))
    for fn, ofn in ((t.SoftStep.sigmoid, tp.sigmoid), (t.SoftStep.dsigmoid, tp.dsigmoid), (t.SoftStep.d2sigmoid, tp.d2sigmoid)):
        assert torch.equal(fn(v.to(cuda)).cpu(), ofn(v))
    lin = t.Linear(16, 8, ctrl=ctrl, quant_mode=t.QuantMode.TERNARY).to(cuda)
    ctrl.register_node("lin", lin)
    lin.train()
    lin(torch.randn(4, 16, device=cuda)).sum().backward()
    norms = ctrl.collect_grad_norms()
    assert set(norms) == {"lin"} and norms["lin"].item() > 0
    lin.weight.data.mul_(3.0)
    ctrl.clamp(slack=0.25)
    assert lin.weight.data.abs().max().item() <= 1.25
    lin.clamp((-0.5, 0.5))
    assert lin.weight.data.abs().max().item() <= 0.5
