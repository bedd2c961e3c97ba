"""The allocation-free form of the fused soft-step pass (tmq_softstep_fused_noalloc): its block
partial sums live in a static device array of the library instead of a caller-provided workspace.
Checked through the C ABI against tmq_softstep_fused on the same inputs, bit for bit, on two calls
in a row (the second on a smaller tensor, so it meets what the first left in the array), and
against the CPU oracle."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _call(lib, entry, tw, tg, d, gl, workspace):
    from tmq_amd import _capi
    n = tw.numel()
    y, dw, wc = torch.empty_like(tw), torch.empty_like(tw), torch.empty_like(tw)
    loss = torch.full((1,), -1.0, dtype=torch.float64, device=tw.device)
    args = [_capi.ptr(tw), _capi.ptr(tg), _capi.ptr(y), _capi.ptr(dw), _capi.ptr(wc), _capi.ptr(loss)]
    if workspace is not None:
        args.append(_capi.ptr(workspace))
    args += [n, d, 5.0, 5e-4, ctypes.c_float(gl), -1.0, 1.0, _capi.stream_of(tw)]
    _capi.check(getattr(lib, entry)(*args), entry)
    torch.cuda.synchronize()
    return y, dw, wc, loss


def test_noalloc_fused_pass_equals_the_workspace_form(cuda, oracle):
    from tmq_amd import _capi
    lib = _capi.load()
    assert lib.tmq_softstep_fused_noalloc_max_elements() == 1 << 29
    rng = np.random.default_rng(77)
    for n, d in (((1 << 22) + 4099, 3.0004), (70001, 6.0), (5, 0.1)):   # second and third calls: smaller tensors
        w = rng.uniform(-1.02, 1.02, n).astype(np.float32)
        g = rng.standard_normal(n).astype(np.float32)
        tw, tg = torch.from_numpy(w).to(cuda), torch.from_numpy(g).to(cuda)
        gl = float(np.float32(1.0) / np.float32(n))
        ws = torch.empty(lib.tmq_softstep_fused_workspace_bytes(n), dtype=torch.uint8, device=cuda)
        want = _call(lib, "tmq_softstep_fused", tw, tg, d, gl, ws)
        got = _call(lib, "tmq_softstep_fused_noalloc", tw, tg, d, gl, None)
        for a, b, name in zip(got[:3], want[:3], ("y", "dw", "clamp")):
            assert torch.equal(a.view(torch.int32), b.view(torch.int32)), f"n={n}: {name} differs from tmq_softstep_fused"
        assert got[3].item() == want[3].item(), f"n={n}: loss sum {got[3].item()} vs {want[3].item()}"
        oy, odw, owc, osum = oracle.fused(w, g, d, 5.0, 5e-4, gl, -1.0, 1.0)
        assert np.array_equal(got[0].cpu().numpy().view(np.uint32), oy.view(np.uint32))
        assert np.array_equal(got[1].cpu().numpy().view(np.uint32), odw.view(np.uint32))
        assert np.array_equal(got[2].cpu().numpy().view(np.uint32), owc.view(np.uint32))
        assert abs(got[3].item() - osum) <= 1e-6 * abs(osum)


def test_noalloc_rejects_oversized_and_runs_without_loss(cuda):
    from tmq_amd import _capi
    lib = _capi.load()
    w = torch.zeros(16, device=cuda)
    too_many = (1 << 29) + 1
    rc = lib.tmq_softstep_fused_noalloc(_capi.ptr(w), None, _capi.ptr(w), None, None, None, too_many, 3.0, 5.0, 5e-4,
                                        ctypes.c_float(0.0), -1.0, 1.0, _capi.stream_of(w))
    assert rc == -4                       # TMQ_ERR_TOO_LARGE, nothing launched
    y = torch.empty_like(w)
    _capi.check(lib.tmq_softstep_fused_noalloc(_capi.ptr(w), None, _capi.ptr(y), None, None, None, 16, 6.0, 5.0, 5e-4,
                                               ctypes.c_float(0.0), -1.0, 1.0, _capi.stream_of(w)), "noalloc")
    torch.cuda.synchronize()
    assert torch.equal(y, torch.zeros_like(y))     # S(0) = 0
