"""Writes tests/golden/reference_golden.npz by running the reference's own pure-Python CPU path.

Run in the build container only (imports /root/reference/tmq, whose native-extension imports are
optional and simply absent here). It records what nothing else pins numerically:
  * the stateful hardness / penalty schedule (QuantizationControl.step) for 50 and 150 epochs;
  * one QAT step of the README's MLP on the CPU path -- initial weights, inputs, loss, every
    weight gradient, and the weights after Adam + clamp -- at the first and the last epoch,
    without and with a quantization penalty.
The fixture holds data only.

    python3 tests/golden/make_reference_golden.py
"""
import os
import sys

import numpy as np
import torch
from torch import nn

HERE = os.path.dirname(os.path.abspath(__file__))
REF = os.environ.get("TMQ_REFERENCE", "/root/reference")


def main():
    sys.path.insert(0, REF)
    import tmq as ref  # noqa: E402  (prints two warnings about its missing native extensions)
    out = {}
    # ---- schedules -------------------------------------------------------------------------------------
    for M in (50, 150):
        for tag, qr in (("noq", None), ("q", (5e-4, 2e-3))):
            ctrl = ref.QuantizationControl(epoch_knots=ref.QuantizationScheduleBuilder.default_schedule(M),
                                           qpenalty_range=qr)
            dg, qp = [], []
            for e in range(M):
                ctrl.step(e)
                dg.append(ctrl.digamma)
                qp.append(ctrl.qpenalty)
            out[f"sched_{M}_{tag}_digamma"] = np.array(dg, np.float64)
            out[f"sched_{M}_{tag}_qpenalty"] = np.array(qp, np.float64)
    ctrl = ref.QuantizationControl(epoch_knots=(20, 60, 70, 80, 100), digamma_range=(0.5, 12), qpenalty_range=(0, 1e-3))
    dg, qp = [], []
    for e in range(100):
        ctrl.step(e)
        dg.append(ctrl.digamma)
        qp.append(ctrl.qpenalty)
    out["sched_custom_digamma"], out["sched_custom_qpenalty"] = np.array(dg), np.array(qp)

    # ---- README MLP, one QAT step on the CPU path -----------------------------------------------------------
    class MLP(nn.Module):
        def __init__(self):
            super().__init__()
            self.fc1 = nn.Linear(256, 128)
            self.bn1 = nn.BatchNorm1d(128)
            self.fc2 = nn.Linear(128, 10)
            self.bn2 = nn.BatchNorm1d(10)

        def forward(self, x):
            return self.bn2(self.fc2(torch.relu(self.bn1(self.fc1(x)))))

    case = 0
    for epoch in (0, 149):
        for qr in (None, (5e-4, 5e-4)):
            torch.manual_seed(0)
            model = MLP()
            ctrl = ref.QuantizationControl(epoch_knots=ref.QuantizationScheduleBuilder.default_schedule(150),
                                           qpenalty_range=qr)
            ref.quantize_model(model, ctrl)
            # the reference's Linear.forward is a debug wrapper that dumps files; use the math it wraps
            for m in (model.fc1, model.fc2):
                m.forward = m.forward_wrap
            x = torch.randn(64, 256)
            labels = torch.randint(0, 10, (64,))
            for e in range(epoch + 1):
                ctrl.step(e)
            opt = torch.optim.Adam(model.parameters(), lr=1e-3)
            init = {k: v.detach().clone().numpy() for k, v in model.state_dict().items()}
            model.train()
            opt.zero_grad()
            loss = nn.functional.cross_entropy(model(x), labels)
            ql = ctrl.quantization_loss()
            total = loss + ql
            total.backward()
            grads = {n: p.grad.detach().clone().numpy() for n, p in model.named_parameters() if p.grad is not None}
            opt.step()
            ctrl.clamp()
            after = {k: v.detach().clone().numpy() for k, v in model.state_dict().items()}
            pre = f"mlp{case}_"
            out[pre + "epoch"] = np.array(epoch)
            out[pre + "qpenalty"] = np.array(float(ctrl.qpenalty))
            out[pre + "digamma"] = np.array(float(ctrl.digamma))
            out[pre + "x"] = x.numpy()
            out[pre + "labels"] = labels.numpy()
            out[pre + "loss"] = np.array(float(loss))
            out[pre + "qloss"] = np.array(float(ql))
            for k, v in init.items():
                out[pre + "init." + k] = v
            for k, v in grads.items():
                out[pre + "grad." + k] = v
            for k, v in after.items():
                out[pre + "after." + k] = v
            out[pre + "registry"] = np.array(list(ctrl._registry.keys()))
            case += 1
    out["mlp_cases"] = np.array(case)
    np.savez_compressed(os.path.join(HERE, "reference_golden.npz"), **out)
    print("wrote reference_golden.npz with", len(out), "arrays")


if __name__ == "__main__":
    main()
