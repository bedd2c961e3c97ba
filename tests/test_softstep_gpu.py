"""GPU parity of the soft-step family: HIP kernels (through the C ABI) vs the CPU oracle.

Bar: bit-exact fp32 (a stricter form of the 1e-6 absolute tolerance the path is specified with;
the tolerance check is kept as a second assertion so a failure says how far off it is). NaN
positions must agree; NaN payloads are not compared.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

HARDNESS = [0.1, 1.1684210526315788, 3.0004, 4.72, 6.0]
SIZES = [1, 3, 4, 255, 4095, 4096, 4097, 3 * 4096 + 17, (1 << 20) + 5]


def _inputs(n, seed):
    rng = np.random.default_rng(seed)
    w = rng.uniform(-1.0, 1.0, n).astype(np.float32)
    m = rng.random(n) < 0.10
    w[m] = (rng.integers(-1, 2, n) + rng.uniform(-0.02, 0.02, n)).astype(np.float32)[m]
    g = rng.standard_normal(n).astype(np.float32)
    return w, g


def _special():
    v = [0.0, -0.0, 0.5, -0.5, 1.0, -1.0, 1.02, -1.02, 0.25, 0.9, 1e-40, -1e-40, 1e-8, -1e-8, 0.99999994, -0.99999994,
         1.5, -1.5, 2.0, -2.0, 3.7, np.nan, np.inf, -np.inf, 123456.0, 0.49999997, 0.50000006, -7.25, 1e30]
    return np.array(v, dtype=np.float32)


def assert_same(got, want, what, atol=1e-6):
    got = got.detach().cpu().numpy().reshape(-1) if isinstance(got, torch.Tensor) else np.asarray(got).reshape(-1)
    want = np.asarray(want, dtype=np.float32).reshape(-1)
    assert got.shape == want.shape, what
    gn, wn = np.isnan(got), np.isnan(want)
    assert np.array_equal(gn, wn), f"{what}: NaN positions differ"
    ok = ~gn
    fin = ok & np.isfinite(want)
    err = np.max(np.abs(got[fin].astype(np.float64) - want[fin].astype(np.float64))) if fin.any() else 0.0
    assert err <= atol, f"{what}: max abs err {err}"
    bad = np.nonzero(got[ok].view(np.uint32) != want[ok].view(np.uint32))[0]
    assert bad.size == 0, f"{what}: {bad.size} elements differ in bits, first at {bad[:5]} (max abs err {err})"


@pytest.mark.parametrize("d", HARDNESS)
@pytest.mark.parametrize("n", SIZES)
def test_unfused_ops_match_oracle(cuda, oracle, d, n):
    from tmq_amd import ops
    w, g = _inputs(n, 100 + n)
    tw, tg = torch.from_numpy(w).to(cuda), torch.from_numpy(g).to(cuda)
    assert_same(ops.fwd_softstep(tw, d), oracle.softstep_fwd(w, d), "fwd")
    assert_same(ops.bwd_softstep(tw, d, 1.0, tg), oracle.softstep_bwd(w, g, d, 1.0), "bwd")
    assert_same(ops.fwd_softstep_derivative(tw, 5.0, 5e-4), oracle.deriv_fwd(w, 5.0, 5e-4), "deriv fwd")
    assert_same(ops.bwd_softstep_derivative(tw, 5.0, 5e-4, tg), oracle.deriv_bwd(w, g, 5.0, 5e-4), "deriv bwd")
    assert_same(ops.fwd_softstep_derivative(tw, d, 0.37), oracle.deriv_fwd(w, d, 0.37), "deriv fwd (d)")
    assert_same(ops.bwd_softstep_derivative(tw, d, 0.37, tg), oracle.deriv_bwd(w, g, d, 0.37), "deriv bwd (d)")
    assert torch.equal(tw.cpu(), torch.from_numpy(w)), "inputs must not be mutated"


@pytest.mark.parametrize("d", HARDNESS + [0.05, 7.3, 20.0])
def test_special_values_and_scale(cuda, oracle, d):
    from tmq_amd import ops
    w = np.concatenate([_special(), _inputs(5000, 9)[0]])
    g = np.random.default_rng(2).standard_normal(w.size).astype(np.float32)
    tw, tg = torch.from_numpy(w).to(cuda), torch.from_numpy(g).to(cuda)
    assert_same(ops.fwd_softstep(tw, d), oracle.softstep_fwd(w, d), "fwd", atol=np.inf)
    assert_same(ops.bwd_softstep(tw, d, 0.37, tg), oracle.softstep_bwd(w, g, d, 0.37), "bwd", atol=np.inf)
    assert_same(ops.fwd_softstep_derivative(tw, d, 5e-4), oracle.deriv_fwd(w, d, 5e-4), "dfwd", atol=np.inf)
    assert_same(ops.bwd_softstep_derivative(tw, d, 5e-4, tg), oracle.deriv_bwd(w, g, d, 5e-4), "dbwd", atol=np.inf)


@pytest.mark.parametrize("d", HARDNESS + [5.0, 0.05, 2.236133, 7.3, 20.0])
def test_fast_division_equals_ieee_division_exhaustively(cuda, d):
    """The kernels use FMA sequences instead of IEEE division; the library proves on the device
    that they agree bit for bit: every fp32 argument in [-3, 3] for the three rational pieces,
    every mantissa for the division by the launch constant of this hardness."""
    import ctypes
    from tmq_amd import _capi
    counts = torch.zeros(5, dtype=torch.int64, device=cuda)
    _capi.check(_capi.load().tmq_selfcheck_division(float(d), ctypes.c_void_p(counts.data_ptr()),
                                                    _capi.stream_of(counts)), "selfcheck")
    c = counts.cpu().tolist()
    assert c[:4] == [0, 0, 0, 0], c
    assert c[4] == 2 * (0x40400000 + 1) + 2 * ((1 << 23) - 1), c     # |x| <= 3 incl. both zeros, plus every NaN


def test_unaligned_and_shaped_views(cuda, oracle):
    from tmq_amd import ops
    w, g = _inputs(10007, 4)
    base_w = torch.from_numpy(np.concatenate([[0.0], w]).astype(np.float32)).to(cuda)
    base_g = torch.from_numpy(np.concatenate([[0.0, 0.0, 0.0], g]).astype(np.float32)).to(cuda)
    tw, tg = base_w[1:], base_g[3:]                     # 4-byte aligned only
    assert tw.data_ptr() % 16 != 0
    assert_same(ops.fwd_softstep(tw, 3.0004), oracle.softstep_fwd(w, 3.0004), "fwd unaligned")
    assert_same(ops.bwd_softstep(tw, 3.0004, 1.0, tg), oracle.softstep_bwd(w, g, 3.0004), "bwd unaligned")
    w4 = torch.from_numpy(w[:9408]).to(cuda).view(64, 3, 7, 7)
    y = ops.fwd_softstep(w4, 4.72)
    assert y.shape == w4.shape
    assert_same(y, oracle.softstep_fwd(w[:9408], 4.72), "fwd 4-D")
    wt = torch.from_numpy(w[:10000]).to(cuda).view(100, 100).t()          # non-contiguous input
    assert_same(ops.fwd_softstep(wt, 4.72).contiguous(), oracle.softstep_fwd(w[:10000].reshape(100, 100).T.copy(), 4.72),
                "fwd transposed view")


def test_empty_and_errors(cuda):
    from tmq_amd import ops
    e = torch.empty(0, device=cuda)
    assert ops.fwd_softstep(e, 1.0).numel() == 0
    assert ops.bwd_softstep(e, 1.0, 1.0, e).numel() == 0
    with pytest.raises(RuntimeError):
        ops.fwd_softstep(torch.zeros(4), 1.0)                              # CPU tensor (tmq_cuda.cu:741)
    with pytest.raises(ValueError):
        ops.fwd_softstep(torch.zeros(4, device=cuda, dtype=torch.float16), 1.0)   # "Not implemented yet"
    with pytest.raises(ValueError):
        ops.fwd_softstep(torch.zeros(4, device=cuda, dtype=torch.float64), 1.0)
    with pytest.raises(RuntimeError):
        ops.bwd_softstep(torch.zeros(4, device=cuda), 1.0, 1.0, torch.zeros(5, device=cuda))


@pytest.mark.parametrize("n", [1, 4097, 100003, (1 << 20) + 5])
def test_clamp_and_ternarize_inplace(cuda, oracle, n):
    from tmq_amd import ops
    rng = np.random.default_rng(n)
    w = np.concatenate([rng.uniform(-1.5, 1.5, n).astype(np.float32), _special()])
    t = torch.from_numpy(w.copy()).to(cuda)
    p = t.data_ptr()
    ops.clamp_(t, -1.0, 1.0)
    assert t.data_ptr() == p
    assert_same(t, oracle.clamp(w, -1.0, 1.0), "clamp", atol=np.inf)
    t2 = torch.from_numpy(w.copy()).to(cuda)
    ops.clamp_(t2, -1.25, 1.25)
    assert_same(t2, oracle.clamp(w, -1.25, 1.25), "clamp slack", atol=np.inf)
    for d in (0.1, 3.0004, 6.0, 20.0):
        t3 = torch.from_numpy(w.copy()).to(cuda)
        ops.ternarize_(t3, d)
        assert_same(t3, oracle.ternarize(w, d), f"ternarize d={d}", atol=np.inf)
    t4 = torch.from_numpy(w.copy()).to(cuda)
    ops.ternarize_(t4)
    assert_same(t4, oracle.round_half_even(w), "round", atol=np.inf)


@pytest.mark.parametrize("d", HARDNESS)
@pytest.mark.parametrize("n", [5, 4096, 65536 + 3, (1 << 20) + 5])
def test_fused_pass_matches_oracle(cuda, oracle, d, n):
    from tmq_amd import ops
    w, g = _inputs(n, 7 + n)
    gl = float(np.float32(1.0) / np.float32(n))
    tw, tg = torch.from_numpy(w).to(cuda), torch.from_numpy(g).to(cuda)
    oy, odw, owc, osum = oracle.fused(w, g, d, 5.0, 5e-4, gl, -1.0, 1.0)
    y, dw, wc, loss = ops.softstep_fused(tw, tg, d, 5.0, 5e-4, gl, -1.0, 1.0)
    assert_same(y, oy, "fused y")
    assert_same(dw, odw, "fused dw")
    assert_same(wc, owc, "fused clamp")
    assert abs(loss.item() - osum) <= 1e-6 * abs(osum) + 1e-12, (loss.item(), osum)
    assert torch.equal(tw.cpu(), torch.from_numpy(w))
    # every subset of outputs gives the same values as the full pass
    for mask in range(1, 16):
        yy, dd, cc, ll = ops.softstep_fused(tw, tg, d, 5.0, 5e-4, gl, -1.0, 1.0, want_y=bool(mask & 1),
                                            want_dw=bool(mask & 2), want_clamp=bool(mask & 4),
                                            want_loss=bool(mask & 8))
        if mask & 1: assert torch.equal(yy, y)
        if mask & 2: assert torch.equal(dd, dw)
        if mask & 4: assert torch.equal(cc, wc)
        if mask & 8: assert ll.item() == loss.item()
    # in-place clamp variant
    tw2 = tw.clone()
    _, _, cc, _ = ops.softstep_fused(tw2, tg, d, 5.0, 5e-4, gl, -1.0, 1.0, clamp_inplace=True)
    assert cc.data_ptr() == tw2.data_ptr() and torch.equal(tw2, wc)


def test_multi_tensor_forms(cuda, oracle):
    from tmq_amd import ops
    shapes = [(64, 3, 7, 7), (128, 256), (10, 128), (1,), (0,), (4097,), (512, 512, 3, 3)]
    rng = np.random.default_rng(21)
    ws = [rng.uniform(-1.3, 1.3, int(np.prod(s))).astype(np.float32).reshape(s) for s in shapes]
    tws = [torch.from_numpy(w.copy()).to(cuda) for w in ws]
    grads = [torch.zeros_like(t) for t in tws]
    scal = [float(np.float32(1.0) / np.float32(max(1, w.size))) for w in ws]
    table = ops.SegmentTable(tws, aux=grads, scalars=scal)
    per, tot = ops.qloss_multi(table, 5.0, 5e-4)
    per = per.cpu().numpy()
    running = None
    for i, w in enumerate(ws):
        if w.size == 0:
            assert np.isnan(per[i])
            continue
        want = oracle.sum64(oracle.deriv_fwd(w, 5.0, 5e-4)) / w.size
        assert abs(per[i] - want) <= 1e-6 * abs(want), (i, per[i], want)
    nz = [i for i, w in enumerate(ws) if w.size]
    # NaN from the empty tensor propagates to the total, like torch
    assert np.isnan(tot.item())
    table2 = ops.SegmentTable([tws[i] for i in nz], aux=[grads[i] for i in nz], scalars=[scal[i] for i in nz])
    per2, tot2 = ops.qloss_multi(table2, 5.0, 5e-4)
    acc = np.float32(0)
    for j, v in enumerate(per2.cpu().numpy()):
        acc = v if j == 0 else np.float32(acc + v)
    # the means summed in the launch (as integers, order-free) agree with the reference's fp32 running sum in table
    # order to fp32 rounding; the two-launch entry point reproduces that running sum bit for bit (test_inlaunch_loss_gpu)
    assert abs(tot2.item() - float(acc)) <= 1e-6 * abs(float(acc))
    # gradient: overwrite, then accumulate on top
    ops.qloss_bwd_multi(table2, 5.0, 5e-4, accumulate=False)
    for i in nz:
        gfill = np.full(ws[i].size, scal[i], np.float32)
        assert_same(grads[i], oracle.deriv_bwd(ws[i], gfill, 5.0, 5e-4), f"qloss bwd {i}", atol=np.inf)
    ops.qloss_bwd_multi(table2, 5.0, 5e-4, accumulate=True)
    for i in nz:
        gfill = np.full(ws[i].size, scal[i], np.float32)
        one = oracle.deriv_bwd(ws[i], gfill, 5.0, 5e-4)
        assert_same(grads[i], one + one, f"qloss bwd acc {i}", atol=np.inf)
    ops.clamp_multi_(table2, -1.0, 1.0)
    for i in nz:
        assert_same(tws[i], oracle.clamp(ws[i], -1.0, 1.0), f"clamp multi {i}", atol=np.inf)


def test_full_size_properties(cuda, oracle):
    """The 64 Mi-element workload of the headline metric: properties that do not need the oracle
    at full size, plus an oracle check on a strided sample."""
    from tmq_amd import ops
    n = 1 << 26
    g0 = torch.Generator(device="cpu").manual_seed(1)
    w = (2 * torch.rand(n, generator=g0) - 1)
    m = torch.rand(n, generator=torch.Generator().manual_seed(2)) < 0.10
    lvl = torch.randint(-1, 2, (n,), generator=torch.Generator().manual_seed(3)).float()
    off = 0.04 * torch.rand(n, generator=torch.Generator().manual_seed(4)) - 0.02
    w[m] = (lvl + off)[m]
    g = torch.randn(n, generator=torch.Generator().manual_seed(5))
    tw, tg = w.to(cuda), g.to(cuda)
    d, gl = 4.72, float(np.float32(1.0) / np.float32(n))
    y, dw, wc, loss = ops.softstep_fused(tw, tg, d, 5.0, 5e-4, gl, -1.0, 1.0)
    # (1) fused == unfused kernels, bit for bit
    assert torch.equal(y, ops.fwd_softstep(tw, d))
    t1 = ops.bwd_softstep(tw, d, 1.0, tg)
    t2 = ops.bwd_softstep_derivative(tw, 5.0, 5e-4, torch.full_like(tw, gl))
    assert torch.equal(dw, t1 + t2)
    # (2) loss sum == fp64 sum of the integrand tensor
    q = ops.fwd_softstep_derivative(tw, 5.0, 5e-4)
    ref = q.double().sum().item()
    assert abs(loss.item() - ref) <= 1e-7 * abs(ref)
    # (3) clamp: idempotent, in range, identity inside the range
    assert wc.min().item() >= -1.0 and wc.max().item() <= 1.0
    inside = tw.abs() <= 1.0
    assert torch.equal(wc[inside], tw[inside])
    wc2 = wc.clone(); ops.clamp_(wc2, -1.0, 1.0)
    assert torch.equal(wc2, wc)
    # (4) staircase invariants: S maps [k, k+1) into [k, k+1], slope >= 0
    fl = torch.floor(tw)
    assert torch.all(y >= fl - 1.2e-7) and torch.all(y <= fl + 1 + 1.2e-7)
    assert torch.all(ops.bwd_softstep(tw, d, 1.0, torch.ones_like(tw)) >= 0)
    # (5) oracle on a strided sample of 1 Mi elements
    idx = torch.arange(0, n, 64)
    ws, gs = w[idx].numpy(), g[idx].numpy()
    oy, odw, owc, _ = oracle.fused(ws, gs, d, 5.0, 5e-4, gl, -1.0, 1.0)
    assert_same(y[idx.to(cuda)], oy, "sample y")
    assert_same(dw[idx.to(cuda)], odw, "sample dw")
    assert_same(wc[idx.to(cuda)], owc, "sample clamp")


@pytest.mark.parametrize("d", HARDNESS)
def test_ternarize_over_every_float_in_range(cuda, oracle, d):
    """Every fp32 value in [-1.02, 1.02] (2 x 1 065 520 989 bit patterns, both zeros included): ternarising
    through the soft staircase (tmq/tmq.py:284-295 with map, 328-338) is expected to equal plain
    round-half-even of the weight -- map is monotone and fixes k and k + 1/2 -- but the reference computes
    it through map's own fp32 op order. Wherever the two differ in value, the kernel must agree with
    the CPU restatement of that op order bit for bit; the test reports how often that happens, and how
    often only the sign of a zero differs (map's arithmetic does not keep it)."""
    from tmq_amd import ops
    top = int(np.float32(1.02).view(np.uint32))                 # 0x3F828F5C
    chunk = 1 << 26
    differ = signs = 0
    for base in range(0, top + 1, chunk):
        n = min(chunk, top + 1 - base)
        bits = torch.arange(base, base + n, dtype=torch.int64, device=cuda).to(torch.int32)
        for sign in (0, -(1 << 31)):
            w = (bits | sign).view(torch.float32) if sign else bits.view(torch.float32)
            t = w.clone()
            ops.ternarize_(t, d)
            r = torch.round(w)
            bad = (t != r).nonzero().flatten()                       # by value: -0.0 == +0.0
            signs += int((t.view(torch.int32) != r.view(torch.int32)).sum().item()) - bad.numel()
            if bad.numel():
                differ += bad.numel()
                sel = bad[:100000]
                wm = w[sel].cpu().numpy()
                assert np.array_equal(t[sel].cpu().numpy().view(np.uint32), oracle.ternarize(wm, d).view(np.uint32))
    # a sample of the whole range against the oracle as well (the mismatch set may be empty)
    g = torch.Generator(device=cuda).manual_seed(int(d * 1000))
    sample = torch.randint(0, top + 1, (1 << 20,), device=cuda, generator=g, dtype=torch.int64).to(torch.int32)
    sample[::2] |= -(1 << 31)
    ws = sample.view(torch.float32)
    ts = ws.clone()
    ops.ternarize_(ts, d)
    assert np.array_equal(ts.cpu().numpy().view(np.uint32), oracle.ternarize(ws.cpu().numpy(), d).view(np.uint32))
    print(f"hardness {d}: ternarise differs from round-half-even in value on {differ} of {2 * (top + 1)} inputs "
          f"and only in the sign of a zero on {signs}")
