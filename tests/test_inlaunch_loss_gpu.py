"""The loss reductions that finish inside their launch (tmq_*_inlaunch: fixed-point atomics, no finalisation
kernel) against the two-launch forms and the CPU oracle, through the C ABI.

Bar: every element-wise output bit-identical to the two-launch form (same kernel body); the loss within 1e-6
relative of the oracle's fp64 sum (a3: tmq/tmq.py:456-473 + 698-699 + 298-310) and within 1e-7 of the two-launch
form; bit-identical from run to run whatever the order in which blocks arrive; the state left zero by every call,
also after NaN weights and under HIP-graph replays.
"""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SIZES = [1, 5, 2047, 2048, 2049, 16 * 2048, 16 * 2048 + 1, 40000, 17 * 2048 - 3, (1 << 20) + 5]


def _inputs(n, seed):
    rng = np.random.default_rng(seed)
    w = rng.uniform(-1.02, 1.02, n).astype(np.float32)
    m = rng.random(n) < 0.10
    w[m] = (rng.integers(-1, 2, n) + rng.uniform(-0.02, 0.02, n)).astype(np.float32)[m]
    return w, rng.standard_normal(n).astype(np.float32)


def _fresh_state(cuda):
    from tmq_amd import _capi
    return torch.zeros(_capi.load().tmq_loss_state_bytes(), dtype=torch.uint8, device=cuda)


def _fused(cuda, tw, tg, d, state=None, want=(True, True, True)):
    """(y, dw, wc, loss) of the fused pass: in-launch when a state is given, else the two-launch form."""
    from tmq_amd import _capi
    lib = _capi.load()
    n = tw.numel()
    nan = float("nan")
    y = torch.full_like(tw, nan) if want[0] else None
    dw = torch.full_like(tw, nan) if want[1] else None
    wc = torch.full_like(tw, nan) if want[2] else None
    loss = torch.full((1,), nan, dtype=torch.float64, device=cuda)
    gl = ctypes.c_float(float(np.float32(1.0) / np.float32(max(n, 1))))
    p, s = _capi.ptr, _capi.stream_of(tw)
    if state is not None:
        rc = lib.tmq_softstep_fused_inlaunch(p(tw), p(tg) if dw is not None else None, p(y), p(dw), p(wc), p(loss), p(state),
                                             n, d, 5.0, 5e-4, gl, -1.0, 1.0, s)
    else:
        ws = torch.full((lib.tmq_softstep_fused_workspace_bytes(n),), 0xFF, dtype=torch.uint8, device=cuda)
        rc = lib.tmq_softstep_fused(p(tw), p(tg) if dw is not None else None, p(y), p(dw), p(wc), p(loss), p(ws), n, d, 5.0,
                                    5e-4, gl, -1.0, 1.0, s)
    _capi.check(rc, "fused")
    torch.cuda.synchronize()
    return y, dw, wc, loss


def _same_bits(a, b):
    return torch.equal(a.view(torch.int32), b.view(torch.int32))


@pytest.mark.parametrize("n", SIZES)
def test_fused_inlaunch_equals_two_launch_form_and_oracle(cuda, oracle, n):
    w, g = _inputs(n, 300 + n % 1000)
    tw, tg = torch.from_numpy(w).to(cuda), torch.from_numpy(g).to(cuda)
    state = _fresh_state(cuda)
    for d in (0.1, 3.0004, 6.0):
        want = _fused(cuda, tw, tg, d)
        got = _fused(cuda, tw, tg, d, state)
        for a, b, name in zip(got[:3], want[:3], ("y", "dw", "clamp")):
            assert _same_bits(a, b), (name, n, d)
        ref = oracle.sum64(oracle.deriv_fwd(w, 5.0, 5e-4))
        assert abs(got[3].item() - ref) <= 1e-6 * abs(ref), (got[3].item(), ref)
        assert abs(got[3].item() - want[3].item()) <= 1e-7 * abs(want[3].item())
        assert int(state.count_nonzero()) == 0, "the call must leave the state zero"
    # the loss alone, and with a subset of the outputs
    for sel in ((False, False, False), (True, False, False), (False, False, True)):
        got = _fused(cuda, tw, tg, 3.0004, state, sel)
        assert abs(got[3].item() - ref) <= 1e-6 * abs(ref) and int(state.count_nonzero()) == 0


def test_bit_identical_from_run_to_run(cuda):
    w, g = _inputs((1 << 22) + 77, 5)
    tw, tg = torch.from_numpy(w).to(cuda), torch.from_numpy(g).to(cuda)
    state = _fresh_state(cuda)
    seen = set()
    for _ in range(25):
        seen.add(_fused(cuda, tw, tg, 4.72, state, (False, False, False))[3].cpu().numpy().tobytes())
    assert len(seen) == 1


def test_nan_weights_poison_the_sum_and_the_state_recovers(cuda, oracle):
    n = 50000
    w, g = _inputs(n, 6)
    state = _fresh_state(cuda)
    for bad in (np.nan, np.inf):
        wb = w.copy()
        wb[31000] = bad
        got = _fused(cuda, torch.from_numpy(wb).to(cuda), torch.from_numpy(g).to(cuda), 3.0004, state)
        want = _fused(cuda, torch.from_numpy(wb).to(cuda), torch.from_numpy(g).to(cuda), 3.0004)
        assert np.isnan(got[3].item()) == np.isnan(want[3].item())
        assert np.isnan(got[3].item())
        assert int(state.count_nonzero()) == 0
        clean = _fused(cuda, torch.from_numpy(w).to(cuda), torch.from_numpy(g).to(cuda), 3.0004, state)
        ref = oracle.sum64(oracle.deriv_fwd(w, 5.0, 5e-4))
        assert abs(clean[3].item() - ref) <= 1e-6 * abs(ref)


def test_errors_and_limits(cuda):
    from tmq_amd import _capi
    lib = _capi.load()
    tw = torch.zeros(100, device=cuda)
    loss = torch.zeros(1, dtype=torch.float64, device=cuda)
    state = _fresh_state(cuda)
    p, s = _capi.ptr, _capi.stream_of(tw)
    gl = ctypes.c_float(0.01)
    assert lib.tmq_softstep_fused_inlaunch(p(tw), None, None, None, None, None, p(state), 100, 1.0, 5.0, 5e-4, gl, -1.0, 1.0, s) == -1
    assert lib.tmq_softstep_fused_inlaunch(p(tw), None, None, None, None, p(loss), None, 100, 1.0, 5.0, 5e-4, gl, -1.0, 1.0, s) == -1
    assert lib.tmq_softstep_fused_inlaunch(p(tw), None, None, None, None, p(loss), p(state), 0, 1.0, 5.0, 5e-4, gl, -1.0, 1.0, s) == -1
    assert lib.tmq_softstep_fused_inlaunch(p(tw), None, None, None, None, p(loss), ctypes.c_void_p(state.data_ptr() + 4), 100, 1.0,
                                           5.0, 5e-4, gl, -1.0, 1.0, s) == -1
    # more tensors than one launch's table holds: the caller is sent to the two-launch form
    arr = (_capi.StepTensor * 65)()
    outs = torch.zeros(65, 4, device=cuda)
    for i in range(65):
        arr[i].w, arr[i].g, arr[i].out, arr[i].n = tw.data_ptr(), None, outs[i].data_ptr(), 4
    tot = torch.zeros((), device=cuda)
    assert lib.tmq_softstep_fwd_multi_inlaunch(arr, 65, 1.0, 5.0, 5e-4, None, p(tot), p(state), s) == _capi.ERR_UNSUPPORTED
    assert lib.tmq_softstep_fwd_multi_inlaunch(arr, 3, 1.0, 5.0, 5e-4, None, None, p(state), s) == -1
    torch.cuda.synchronize()
    assert int(state.count_nonzero()) == 0


def _step_table(ws, ys):
    from tmq_amd import _capi
    arr = (_capi.StepTensor * len(ws))()
    for i, (w, y) in enumerate(zip(ws, ys)):
        arr[i].w, arr[i].g, arr[i].out, arr[i].n = (w.data_ptr() if w.numel() else None), None, \
            (y.data_ptr() if y.numel() else None), w.numel()
    return arr


@pytest.mark.parametrize("sizes", [[1], [2048], [9408, 36864, 36864, 147456 + 3, 7, 2049, 4096], [5, 0, 300000, 0, 64],
                                   [1000] * 64])
def test_multi_tensor_forward_with_loss(cuda, oracle, sizes):
    from tmq_amd import _capi
    lib = _capi.load()
    rng = np.random.default_rng(len(sizes))
    wn = [_inputs(n, 40 + i)[0] if n else np.zeros(0, np.float32) for i, n in enumerate(sizes)]
    ws = [torch.from_numpy(w).to(cuda) for w in wn]
    state = _fresh_state(cuda)
    d = 2.236133
    outs = {}
    for mode in ("two", "one", "one"):
        ys = [torch.full_like(w, float("nan")) for w in ws]
        per = torch.full((len(ws),), float("nan"), device=cuda)
        tot = torch.full((), float("nan"), device=cuda)
        arr = _step_table(ws, ys)
        s = _capi.stream_of(per)
        if mode == "two":
            wsp = torch.full((lib.tmq_softstep_multi_workspace_bytes(arr, len(ws)),), 0xFF, dtype=torch.uint8, device=cuda)
            rc = lib.tmq_softstep_fwd_multi(arr, len(ws), d, 5.0, 5e-4, _capi.ptr(per), _capi.ptr(tot), _capi.ptr(wsp), s)
        else:
            rc = lib.tmq_softstep_fwd_multi_inlaunch(arr, len(ws), d, 5.0, 5e-4, _capi.ptr(per), _capi.ptr(tot), _capi.ptr(state), s)
        _capi.check(rc, mode)
        torch.cuda.synchronize()
        if mode == "one":
            assert int(state.count_nonzero()) == 0
        outs[mode] = (ys, per.cpu().numpy(), tot.item())
    for a, b, w in zip(outs["one"][0], outs["two"][0], wn):
        assert _same_bits(a, b)
        assert np.array_equal(a.cpu().numpy().view(np.uint32), oracle.softstep_fwd(w, d).view(np.uint32))
    per1, per2 = outs["one"][1], outs["two"][1]
    means = np.array([oracle.sum64(oracle.deriv_fwd(w, 5.0, 5e-4)) / w.size if w.size else np.nan for w in wn])
    assert np.array_equal(np.isnan(per1), np.isnan(means)) and np.array_equal(np.isnan(per2), np.isnan(means))
    ok = ~np.isnan(means)
    assert np.all(np.abs(per1[ok] - means[ok]) <= 1e-6 * np.abs(means[ok]))
    assert np.all(np.abs(per1[ok] - per2[ok]) <= 2e-7 * np.abs(per2[ok]))
    if ok.all():
        run = np.float32(0)
        for i, m in enumerate(per2):
            run = np.float32(m) if i == 0 else np.float32(run + np.float32(m))
        assert outs["two"][2] == float(run)                     # fp32 running sum in table order, as the reference adds
        assert abs(outs["one"][2] - float(run)) <= 1e-6 * abs(float(run))   # the same means summed as integers
        assert abs(outs["one"][2] - float(np.sum(means))) <= 1e-6 * abs(float(np.sum(means)))
    else:
        assert np.isnan(outs["one"][2]) and np.isnan(outs["two"][2])


def test_quantization_loss_table_form(cuda, oracle):
    from tmq_amd import ops, _capi
    lib = _capi.load()
    sizes = [9408, 36864, 5, 147456, 2048, 52224]
    wn = [_inputs(n, 70 + i)[0] for i, n in enumerate(sizes)]
    table = ops.SegmentTable([torch.from_numpy(w).to(cuda) for w in wn])
    state = _fresh_state(cuda)
    per1 = torch.empty(len(sizes), device=cuda)
    tot1 = torch.empty(1, device=cuda)
    _capi.check(lib.tmq_qloss_multi_inlaunch(_capi.ptr(table.table), table.nseg, table.total_blocks, 5.0, 5e-4, _capi.ptr(per1),
                                             _capi.ptr(tot1), _capi.ptr(state), _capi.stream_of(per1)), "qloss inlaunch")
    per2 = torch.empty(len(sizes), device=cuda)
    tot2 = torch.empty(1, device=cuda)
    _capi.check(lib.tmq_qloss_multi(_capi.ptr(table.table), table.nseg, table.total_blocks, 5.0, 5e-4, _capi.ptr(per2),
                                    _capi.ptr(tot2), _capi.ptr(table.workspace), _capi.stream_of(per2)), "qloss")
    torch.cuda.synchronize()
    assert int(state.count_nonzero()) == 0
    means = np.array([oracle.sum64(oracle.deriv_fwd(w, 5.0, 5e-4)) / w.size for w in wn])
    assert np.all(np.abs(per1.cpu().numpy() - means) <= 1e-6 * np.abs(means))
    assert torch.allclose(per1, per2, rtol=2e-7, atol=0) and abs(tot1.item() - tot2.item()) <= 1e-6 * abs(tot2.item())
    # the Python wrapper takes the same route
    per3, tot3 = ops.qloss_multi(table, 5.0, 5e-4)
    assert torch.equal(per3, per1) and torch.equal(tot3, tot1)


def test_graph_replays_equal_eager(cuda):
    """The whole-step forward with its loss recorded as a HIP graph: the state is cleared by the launch itself
    (no memset node), so every replay, with eager launches on the same state in between, gives the eager values."""
    from tmq_amd import ops
    ws = [torch.from_numpy(_inputs(n, 90 + i)[0]).to(cuda) for i, n in enumerate([9408, 36864, 147456 + 3, 2049, 600000])]
    ys0, loss0 = ops.softstep_fwd_all(ws, 2.236133, True, 5.0, 5e-4)
    torch.cuda.synchronize()
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        ops.softstep_fwd_all(ws, 2.236133, True, 5.0, 5e-4)         # makes this stream's state outside the capture
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            ys, loss = ops.softstep_fwd_all(ws, 2.236133, True, 5.0, 5e-4)
    for rep in range(5):
        loss.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert loss.item() == loss0.item(), rep
        assert all(torch.equal(a, b) for a, b in zip(ys, ys0))
        _, eager = ops.softstep_fwd_all(ws, 2.236133, True, 5.0, 5e-4)   # eager work between the replays
        assert eager.item() == loss0.item()


def test_full_size_fused_pass(cuda):
    """BASELINE configs[1] at its full 2^26 elements: the in-launch loss against the two-launch form."""
    n = 1 << 26
    g0 = torch.Generator(device=cuda).manual_seed(1)
    tw = 2.04 * torch.rand(n, device=cuda, generator=g0) - 1.02
    tg = torch.randn(n, device=cuda, generator=g0)
    state = _fresh_state(cuda)
    want = _fused(cuda, tw, tg, 3.0004)
    got = _fused(cuda, tw, tg, 3.0004, state)
    for a, b in zip(got[:3], want[:3]):
        assert _same_bits(a, b)
    assert abs(got[3].item() - want[3].item()) <= 1e-7 * abs(want[3].item())
    assert int(state.count_nonzero()) == 0
