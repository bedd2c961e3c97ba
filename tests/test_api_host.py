"""Host-side logic of the Python API (no GPU needed): the hardness / penalty schedule against the
table recorded from the reference's own QuantizationControl.step, model surgery, layer
construction and the refusal to compute on CPU tensors."""
import os

import numpy as np
import pytest
import torch
from torch import nn

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = np.load(os.path.join(ROOT, "tests", "golden", "reference_golden.npz"))


def _tmq():
    import tmq_amd
    return tmq_amd


def _run_schedule(ctrl, epochs):
    dg, qp = [], []
    for e in range(epochs):
        ctrl.step(e)
        dg.append(ctrl.digamma)
        qp.append(ctrl.qpenalty)
    return np.array(dg, np.float64), np.array(qp, np.float64)


@pytest.mark.parametrize("M", [50, 150])
@pytest.mark.parametrize("tag,qr", [("noq", None), ("q", (5e-4, 2e-3))])
def test_schedule_equals_reference_table(M, tag, qr):
    t = _tmq()
    ctrl = t.QuantizationControl(epoch_knots=t.QuantizationScheduleBuilder.default_schedule(M), qpenalty_range=qr)
    dg, qp = _run_schedule(ctrl, M)
    assert np.array_equal(dg, GOLD[f"sched_{M}_{tag}_digamma"])
    assert np.array_equal(qp, GOLD[f"sched_{M}_{tag}_qpenalty"])


def test_schedule_custom_knots_and_properties():
    t = _tmq()
    ctrl = t.QuantizationControl(epoch_knots=(20, 60, 70, 80, 100), digamma_range=(0.5, 12), qpenalty_range=(0, 1e-3))
    dg, qp = _run_schedule(ctrl, 100)
    assert np.array_equal(dg, GOLD["sched_custom_digamma"]) and np.array_equal(qp, GOLD["sched_custom_qpenalty"])
    # shape of the default schedule: flat warm-up, final plateau, saw-tooth restarts every 15 epochs
    ctrl = t.QuantizationControl(epoch_knots=t.QuantizationScheduleBuilder.default_schedule(150))
    dg, _ = _run_schedule(ctrl, 150)
    assert np.all(dg[:8] == 0.1) and np.all(dg[139:] == 6.0)
    for e, v in {21: 1.168421, 22: 0.560132, 39: 1.143947, 56: 1.548, 73: 1.854, 75: 2.236133, 79: 3.0004, 88: 4.72,
                 90: 2.16, 107: 2.466, 122: 6.0}.items():
        assert abs(dg[e] - v) < 1e-6, (e, dg[e], v)
    assert t.QuantizationScheduleBuilder.default_schedule(150) == (45, 120, 131, 139, 150)
    with pytest.raises(AssertionError):
        t.QuantizationScheduleBuilder.default_schedule(49)


def test_controller_construction_rules():
    t = _tmq()
    c = t.QuantizationControl()
    assert c.inference_mode and c.digamma == 0.1 and c.qpenalty == 0 and c.clamp_values == (-1., 1.)
    c.step(10)
    assert c.digamma == 0.1                      # no schedule, no stepping
    for bad in ((0.01, 6), (2, 6), (0.1, 21), (0.1, 2)):
        with pytest.raises(AssertionError):
            t.QuantizationControl(digamma_range=bad)
    with pytest.raises(AssertionError):
        t.QuantizationControl(epoch_knots=(5, 60, 70, 80, 100))
    c = t.QuantizationControl(epoch_knots=(15, 60, 70, 80, 100), qpenalty_range=(1e-4, 1e-3))
    assert not c.inference_mode and c.qpenalty == 1e-4 and c.qpenalty_sharpness == 5.0
    c.inference()
    assert c.inference_mode
    assert t.SoftStep.scalar_sigmoid(2.5) * 2 == pytest.approx(665 / 333, abs=1e-15)
    assert t.SoftStep.scalar_sigmoid(7.0) == 1.0 and t.SoftStep.scalar_dsigmoid(0.0) == 1.0


class MLP(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc1 = nn.Linear(256, 128)
        self.bn1 = nn.BatchNorm1d(128)
        self.fc2 = nn.Linear(128, 10)
        self.bn2 = nn.BatchNorm1d(10)

    def forward(self, x):
        return self.bn2(self.fc2(torch.relu(self.bn1(self.fc1(x)))))


def test_quantize_model_swaps_registers_and_initialises_like_the_reference():
    t = _tmq()
    torch.manual_seed(0)
    model = MLP()
    ctrl = t.QuantizationControl(epoch_knots=t.QuantizationScheduleBuilder.default_schedule(150))
    t.quantize_model(model, ctrl)
    assert isinstance(model.fc1, t.Linear) and isinstance(model.fc2, t.Linear) and isinstance(model.bn1, nn.BatchNorm1d)
    assert list(ctrl._registry.keys()) == [str(s) for s in GOLD["mlp0_registry"]] == [".fc1", ".fc2"]
    # same RNG consumption as the reference: the seeded initial weights are identical
    assert np.array_equal(model.fc1.weight.detach().numpy(), GOLD["mlp0_init.fc1.weight"])
    assert np.array_equal(model.fc2.weight.detach().numpy(), GOLD["mlp0_init.fc2.weight"])
    assert torch.all(model.fc1.bias == 0) and model.fc1.weight.requires_grad
    assert model.fc1.original_shape == (128, 256) and model.fc1.quantization == t.QuantMode.TERNARY
    assert model.fc1.post_scale_imm == 1.0 and not model.fc1.compact
    assert repr(model.fc1) == "Linear(128,256) [tmq] <.fc1>"


def test_quantize_model_prefix_and_exclusion(capsys):
    t = _tmq()
    net = nn.Sequential()
    net.add_module("stem", nn.Conv2d(3, 8, 3, padding=1))
    blk = nn.Sequential()
    blk.add_module("conv5", nn.Conv2d(8, 8, 3))
    blk.add_module("up", nn.ConvTranspose2d(8, 4, 2, stride=2))
    net.add_module("block", blk)
    net.add_module("head", nn.Linear(4, 2, bias=False))
    ctrl = t.QuantizationControl(epoch_knots=(15, 60, 70, 80, 100), post_scale=True)
    t.quantize_model(net, ctrl, prefix="model", exclude=["model.stem", "*conv5"])
    assert isinstance(net.stem, nn.Conv2d) and not isinstance(net.stem, t.Conv2d)
    assert isinstance(net.block.conv5, nn.Conv2d) and not isinstance(net.block.conv5, t.Conv2d)
    assert isinstance(net.block.up, t.ConvTranspose2d) and isinstance(net.head, t.Linear)
    assert list(ctrl._registry.keys()) == ["model.block.up", "model.head"]
    assert "Skipping excluded layer model.stem" in capsys.readouterr().out
    assert net.head.bias is None and tuple(net.block.up.weight.shape) == (8, 4, 2, 2)
    assert net.head.post_scale_imm == pytest.approx(1.0 / (4 * 2.0 / 3.0))      # fan-in x ternary variance
    assert net.block.up.post_scale_imm == pytest.approx(1.0 / (2 * 2 * 8 * 2.0 / 3.0))


def test_cpu_weights_are_refused_not_emulated():
    t = _tmq()
    ctrl = t.QuantizationControl(epoch_knots=(15, 60, 70, 80, 100), qpenalty_range=(1e-3, 1e-3))
    lin = t.Linear(8, 4, ctrl=ctrl, quant_mode=t.QuantMode.TERNARY)
    ctrl.register_node("lin", lin)
    lin.train()
    with pytest.raises(RuntimeError, match="GPU"):
        lin(torch.zeros(2, 8))
    with pytest.raises(RuntimeError, match="GPU"):
        ctrl.quantization_loss()
    with pytest.raises(RuntimeError, match="GPU"):
        ctrl.clamp()
    with pytest.raises(RuntimeError, match="GPU"):
        ctrl.quantize()
    assert t.CUDA_EXT_AVAILABLE and t.NATIVE_EXT_AVAILABLE


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    from tmq_amd import _capi
    monkeypatch.setattr(_capi, "_lib", None)
    monkeypatch.setattr(_capi, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError, match="no CPU or PyTorch fallback"):
        _capi.load()
