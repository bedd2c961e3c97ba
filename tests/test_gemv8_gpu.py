"""One fp16 activation row with K a multiple of 256 (2048 .. 16384) runs on the 8-bit matrix instructions:
weights as fp8 +-2, the activation vector as four exact bf8 terms. Checked against an fp64 product of the
expanded weights (not the library), through every epilogue, ragged N, every K the kernel takes, and on the
inputs where its one numerical difference from an fp32 sum (the instruction's internal alignment window over
32 products) would show. On normally distributed activations that difference is a few 1e-6 of the largest output
(the fp16 kernels: below 1e-6); the bar for this path is 1e-3.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _ternary(rng, N, K, p0=0.5):
    u = rng.random((N, K))
    return np.where(u < (1 - p0) / 2, 1.0, np.where(u < 1 - p0, -1.0, 0.0)).astype(np.float32)


def _rel_err(got, want):
    want = np.asarray(want, np.float64)
    got = np.asarray(got, np.float64)
    return np.max(np.abs(got - want)) / max(1e-30, np.max(np.abs(want)))


def _layer(cuda, oracle, rng, N, K, p0=0.5):
    from tmq_amd import ops
    W = _ternary(rng, N, K, p0)
    words = oracle.pack(W)
    return W, ops.NativeWeights(torch.from_numpy(words.view(np.int32)).to(cuda), N)


# every multiple of 2048, and block counts that do not deal out evenly over the wavefronts of a channel block
# (9, 20, 27, 33, 43, 54 and 63 blocks of 256: a wavefront without a block in the last round multiplies by zero)
@pytest.mark.parametrize("K", [2048 * i for i in range(1, 9)] + [2304, 5120, 6912, 8448, 11008, 13824, 16128])
@pytest.mark.parametrize("N", [16, 1000, 4100])
def test_every_reduction_length_and_ragged_channels(cuda, oracle, K, N):
    from tmq_amd import ops
    rng = np.random.default_rng(K + N)
    W, nw = _layer(cuda, oracle, rng, N, K)
    x = rng.standard_normal((1, K)).astype(np.float16)
    y = ops.ternary_linear(torch.from_numpy(x).to(cuda), nw)
    ref = x.astype(np.float64) @ W.astype(np.float64).T
    assert y.shape == (1, N) and y.dtype == torch.float32
    assert _rel_err(y.cpu().numpy(), ref) <= 1e-5
    assert torch.equal(ops.ternary_linear(torch.from_numpy(x).to(cuda), nw), y)   # run to run identical
    # the reference's binding name on the compact words, a one-dimensional vector
    words = torch.from_numpy(oracle.pack(W).view(np.int32)).to(cuda)
    v = ops.ternary_mvm_cuda(torch.from_numpy(x[0]).to(cuda), words, N)
    assert torch.equal(v.reshape(1, N), y)


@pytest.mark.parametrize("y16", [False, True])
def test_epilogues(cuda, oracle, y16):
    from tmq_amd import ops
    K, N = 4096, 1000
    rng = np.random.default_rng(77)
    W, nw = _layer(cuda, oracle, rng, N, K)
    x = rng.standard_normal((1, K)).astype(np.float16)
    scale = (0.01 + 0.02 * rng.random(N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    res = rng.standard_normal((1, N)).astype(np.float16 if y16 else np.float32)
    acc = x.astype(np.float64) @ W.astype(np.float64).T
    t = lambda a: torch.from_numpy(a).to(cuda)
    odt = torch.float16 if y16 else torch.float32
    tol = 1e-3 if y16 else 1e-5
    y = ops.ternary_linear(t(x), nw, t(scale), t(bias), out_dtype=odt)
    assert y.dtype == odt
    assert _rel_err(y.float().cpu().numpy(), acc * scale + bias) <= tol
    y = ops.ternary_linear(t(x), nw, t(scale), None, residual=t(res), relu=True, out_dtype=odt)
    assert _rel_err(y.float().cpu().numpy(), np.maximum(acc * scale + res.astype(np.float64), 0)) <= tol
    y = ops.ternary_linear(t(x), nw, None, t(bias), relu=True, out_dtype=odt)
    assert _rel_err(y.float().cpu().numpy(), np.maximum(acc + bias, 0)) <= tol
    assert (y >= 0).all()


def test_exact_on_integers_and_on_every_fp16_mantissa(cuda, oracle):
    """Small integers: every product and every partial sum is an integer below 2^24, so the result is exact
    whatever the order. All 11 significant bits of the fp16 values must survive the four-term split: values
    (1024 + m) for every m reach the last bit."""
    from tmq_amd import ops
    K, N = 2048, 256
    rng = np.random.default_rng(3)
    W, nw = _layer(cuda, oracle, rng, N, K)
    x = rng.integers(-8, 9, size=(1, K)).astype(np.float16)
    y = ops.ternary_linear(torch.from_numpy(x).to(cuda), nw)
    assert np.array_equal(y.cpu().numpy().astype(np.float64), x.astype(np.float64) @ W.astype(np.float64).T)
    m = (1024 + (np.arange(K) % 1024)).astype(np.float16) * np.where(rng.random(K) < .5, -1, 1).astype(np.float16)
    y = ops.ternary_linear(torch.from_numpy(m[None]).to(cuda), nw)
    assert np.array_equal(y.cpu().numpy().astype(np.float64), m[None].astype(np.float64) @ W.astype(np.float64).T)
    # subnormal fp16 values: integers times 2^-24, so again exact whatever the order
    tiny = (rng.integers(-1023, 1024, size=(1, K)).astype(np.float64) * 2.0 ** -24).astype(np.float16)
    y = ops.ternary_linear(torch.from_numpy(tiny).to(cuda), nw)
    assert np.array_equal(y.cpu().numpy().astype(np.float64), tiny.astype(np.float64) @ W.astype(np.float64).T)
    # a layer whose activations are all of order 1e-3
    small = (rng.standard_normal((1, K)) * 1e-3).astype(np.float16)
    y = ops.ternary_linear(torch.from_numpy(small).to(cuda), nw)
    assert _rel_err(y.cpu().numpy(), small.astype(np.float64) @ W.astype(np.float64).T) <= 1e-5


def test_single_weight_selects_each_position(cuda, oracle):
    """A weight matrix with one nonzero per channel picks single activations: catches any mismatch between the
    byte order of the activation planes and the weight registers (a permuted k within a block)."""
    from tmq_amd import ops
    K, N = 2048, 2048
    W = np.zeros((N, K), np.float32)
    rng = np.random.default_rng(4)
    sign = np.where(rng.random(N) < .5, -1.0, 1.0).astype(np.float32)
    W[np.arange(N), np.arange(N)] = sign
    nw = ops.NativeWeights(torch.from_numpy(oracle.pack(W).view(np.int32)).to(cuda), N)
    x = rng.standard_normal((1, K)).astype(np.float16)
    y = ops.ternary_linear(torch.from_numpy(x).to(cuda), nw)
    assert np.array_equal(y.cpu().numpy()[0], x[0].astype(np.float32) * sign)


def test_every_finite_fp16_value_passes_through_exactly(cuda, oracle):
    """The activation vector reaches the 8-bit instruction as four scaled bf8 terms. With the identity as weights
    the output must be the input, bit for bit, for each of the 63488 finite fp16 values (subnormals included)."""
    from tmq_amd import ops
    K = N = 4096
    nw = ops.NativeWeights(torch.from_numpy(oracle.pack(np.eye(N, dtype=np.float32)).view(np.int32)).to(cuda), N)
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    vals = bits.view(np.float16).copy()
    vals[~np.isfinite(vals)] = 0
    perm = np.random.default_rng(8).permutation(65536)          # neighbours of unrelated magnitude
    vals = vals[perm]
    for c in range(65536 // K):
        x = vals[c * K:(c + 1) * K][None]
        y = ops.ternary_linear(torch.from_numpy(x).to(cuda), nw).cpu().numpy()
        assert np.array_equal(y, x.astype(np.float32)), c                  # by value: -0 comes back as +0


def test_wide_dynamic_range_within_the_stated_tolerance(cuda, oracle):
    """The 8-bit instruction aligns its 32 products to the largest before adding: next to 65504, values of order
    one lose their low bits. The loss is bounded by ~2^-17 of the largest product per instruction -- far inside
    the 1e-3 bar, and asserted here at 2e-4 of the largest output."""
    from tmq_amd import ops
    K, N = 4096, 512
    rng = np.random.default_rng(5)
    W, nw = _layer(cuda, oracle, rng, N, K)
    x = rng.standard_normal((1, K)).astype(np.float16)
    x[0, ::32] = np.float16(65504.0) * np.where(rng.random(K // 32) < .5, -1, 1)
    x[0, 1::32] = (rng.standard_normal(K // 32) * 1e-4).astype(np.float16)
    y = ops.ternary_linear(torch.from_numpy(x).to(cuda), nw)
    ref = x.astype(np.float64) @ W.astype(np.float64).T
    assert _rel_err(y.cpu().numpy(), ref) <= 2e-4
    # ten orders of magnitude apart, elementwise random
    x = (rng.standard_normal((1, K)) * 10.0 ** rng.integers(-6, 4, size=(1, K))).astype(np.float16)
    y = ops.ternary_linear(torch.from_numpy(x).to(cuda), nw)
    assert _rel_err(y.cpu().numpy(), x.astype(np.float64) @ W.astype(np.float64).T) <= 2e-4


def test_agrees_with_the_fp16_kernels_on_neighbouring_shapes(cuda, oracle):
    """M = 5 (fp16 weight-stream kernel) on copies of the row, and an unaligned view of the row (skinny
    kernel), give the same numbers to fp32 rounding."""
    from tmq_amd import ops
    K, N = 8192, 1024
    rng = np.random.default_rng(6)
    W, nw = _layer(cuda, oracle, rng, N, K)
    buf = torch.from_numpy(rng.standard_normal(K + 8).astype(np.float16)).to(cuda)
    x = buf[:K].clone()[None]
    y1 = ops.ternary_linear(x, nw)
    y2 = ops.ternary_linear(torch.cat([x] * 5), nw)
    assert torch.equal(y2[0], y2[4])
    assert _rel_err(y1.cpu().numpy(), y2[:1].cpu().numpy()) <= 1e-5
    buf[1:K + 1] = x[0]
    y3 = ops.ternary_linear(buf[1:K + 1][None], nw)                     # 2-byte aligned: not the 8-bit kernel
    assert _rel_err(y1.cpu().numpy(), y3.cpu().numpy()) <= 1e-5


@pytest.mark.parametrize("K", [256, 512, 1024, 1792, 2048, 4096, 6144, 8192, 2304, 5120, 6912, 8448, 11008, 12288, 13824, 16128, 16384])
def test_fp32_row_runs_as_two_fp16_halves(cuda, oracle, K):
    """One fp32 row (the reference's GEMV convention) up to K = 16384: hi = fp16(x), lo = fp16(x - hi), each as four
    bf8 terms in eight activation columns (beyond 8192 in workgroups of sixteen wavefronts). 22 significant bits of
    every value reach the product."""
    from tmq_amd import ops
    N = 1000
    rng = np.random.default_rng(K)
    W, nw = _layer(cuda, oracle, rng, N, K)
    x = rng.standard_normal((1, K)).astype(np.float32)
    scale = (0.5 + rng.random(N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    t = lambda a: torch.from_numpy(a).to(cuda)
    y = ops.ternary_linear(t(x), nw, t(scale), t(bias))
    ref = (x.astype(np.float64) @ W.astype(np.float64).T) * scale + bias
    assert y.dtype == torch.float32 and _rel_err(y.cpu().numpy(), ref) <= 1e-5
    # far better than a single fp16 rounding of the row would be
    y16 = ops.ternary_linear(t(x).half(), nw, t(scale), t(bias))
    assert _rel_err(y.cpu().numpy(), ref) < 0.1 * _rel_err(y16.cpu().numpy(), ref)
    # the reference's binding name, every rank it takes
    words = t(oracle.pack(W).view(np.int32))
    for shape in ((K,), (1, K), (1, 1, K)):
        v = ops.ternary_mvm_cuda(t(x.reshape(shape)), words, N)
        assert tuple(v.shape) == shape[:-1] + (N,)
        assert _rel_err(v.cpu().numpy().reshape(1, N), x.astype(np.float64) @ W.astype(np.float64).T) <= 1e-5
    # residual + ReLU, fp16 output
    res = rng.standard_normal((1, N)).astype(np.float16)
    y3 = ops.ternary_linear(t(x), nw, t(scale), t(bias), residual=t(res), relu=True, out_dtype=torch.float16)
    assert _rel_err(y3.float().cpu().numpy(), np.maximum(ref + res.astype(np.float64), 0)) <= 1e-3


@pytest.mark.parametrize("K", [2048, 2816, 4096, 6912, 8192, 8448, 11008, 16384])
def test_wide_layers(cuda, oracle, K):
    """1025 channel blocks (ragged): several channel blocks per workgroup, for an fp16 row and for an fp32 row."""
    from tmq_amd import ops
    N = 16400
    rng = np.random.default_rng(K)
    W = torch.from_numpy(rng.integers(-1, 2, size=(N, K), dtype=np.int8))
    words = torch.from_numpy(oracle.pack(W.numpy().astype(np.float32)).view(np.int32)).to(cuda)
    nw = ops.NativeWeights(words, N)
    Wd = W.to(cuda).double()
    for dt, tol in ((np.float16, 1e-5), (np.float32, 1e-5)):
        x = torch.from_numpy(rng.standard_normal((1, K)).astype(dt)).to(cuda)
        scale = torch.from_numpy((0.5 + rng.random(N)).astype(np.float32)).to(cuda)
        bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(cuda)
        y = ops.ternary_linear(x, nw, scale, bias)
        ref = (x.double() @ Wd.t()) * scale.double() + bias.double()
        err = ((y.double() - ref).abs().max() / ref.abs().max()).item()
        assert err <= tol, (K, dt, err)
        assert torch.equal(ops.ternary_linear(x, nw, scale, bias), y)
        if dt == np.float16:                # planes prepared beforehand: the same geometry, the same values
            assert torch.equal(ops.ternary_linear_planes(ops.gemv8_prepare(x), nw, scale, bias), y)


@pytest.mark.parametrize("K", [6144, 8448, 11008, 12288, 16384])
def test_two_long_rows_against_wide_layers(cuda, oracle, K):
    """Two fp16 rows of more than 8192 indices against 16384 channels or more: eight planes on the sixteen-wavefront
    workgroups (and 6144 indices, whose 24 weight blocks deal out evenly over eight wavefronts: the same kernel at any width). Rows of different magnitude stay apart, every row equals its own single-row launch bit for bit, every
    finite fp16 value passes an identity layer, and a narrower layer (the weight-stream kernel) agrees."""
    from tmq_amd import ops
    N = 16400
    rng = np.random.default_rng(K + 2)
    W = torch.from_numpy(rng.integers(-1, 2, size=(N, K), dtype=np.int8))
    nw = ops.NativeWeights(torch.from_numpy(oracle.pack(W.numpy().astype(np.float32)).view(np.int32)).to(cuda), N)
    Wd = W.to(cuda).double()
    x = rng.standard_normal((2, K)).astype(np.float16)
    x[1] *= np.float16(37.0)
    x = torch.from_numpy(x).to(cuda)
    scale = torch.from_numpy((0.5 + rng.random(N)).astype(np.float32)).to(cuda)
    bias = torch.from_numpy(rng.standard_normal(N).astype(np.float32)).to(cuda)
    y = ops.ternary_linear(x, nw, scale, bias)
    ref = (x.double() @ Wd.t()) * scale.double() + bias.double()
    for m in range(2):
        err = ((y[m].double() - ref[m]).abs().max() / ref[m].abs().max()).item()
        assert err <= 1e-5, (K, m, err)
        single = ops.ternary_linear(x[m:m + 1], nw, scale, bias)[0]
        if K > 8192:                         # the same geometry as the single row: the same sums in the same order
            assert torch.equal(single, y[m]), (K, m)
        else:                                # (a single row of 6144 indices splits its blocks over four wavefronts, two rows over eight)
            assert ((single.double() - y[m].double()).abs().max() / ref[m].abs().max()).item() <= 2e-6, (K, m)
    res = torch.from_numpy(rng.standard_normal((2, N)).astype(np.float16)).to(cuda)
    y2 = ops.ternary_linear(x, nw, scale, bias, residual=res, relu=True, out_dtype=torch.float16)
    ref2 = torch.clamp_min(ref + res.double(), 0)
    assert ((y2.double() - ref2).abs().max() / ref2.abs().max()).item() <= 1e-3
    narrow = ops.NativeWeights(torch.from_numpy(oracle.pack(W[:4100].numpy().astype(np.float32)).view(np.int32)).to(cuda), 4100)
    yn = ops.ternary_linear(x, narrow, scale[:4100], bias[:4100])
    assert ((yn.double() - y[:, :4100].double()).abs().max() / ref.abs().max()).item() <= 1e-5
    if K == 16384:
        vals = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16).copy()
        vals[~np.isfinite(vals)] = 0
        vals = vals[np.random.default_rng(8).permutation(65536)]
        eye = ops.NativeWeights(torch.from_numpy(oracle.pack(np.eye(K, dtype=np.float32)).view(np.int32)).to(cuda), K)
        for c in (0, 2):
            xv = vals[c * K:(c + 2) * K].reshape(2, K)
            yv = ops.ternary_linear(torch.from_numpy(xv).to(cuda), eye)
            assert np.array_equal(yv.cpu().numpy(), xv.astype(np.float32)), c


@pytest.mark.parametrize("K", [256, 2048, 16384])
def test_fp32_row_passes_22_bit_values_through_exactly(cuda, oracle, K):
    """Identity weights: integers of up to 22 bits (and their power-of-two multiples, small and large) come back
    exactly -- both halves and all eight term columns are in place."""
    from tmq_amd import ops
    N = K
    nw = ops.NativeWeights(torch.from_numpy(oracle.pack(np.eye(N, dtype=np.float32)).view(np.int32)).to(cuda), N)
    rng = np.random.default_rng(9)
    ints = rng.integers(-(1 << 21), 1 << 21, size=(1, K)).astype(np.float32)
    for s in (1.0, 2.0 ** -30, 2.0 ** 40, 2.0 ** -120, 2.0 ** 100):    # the kernel scales the row itself
        x = (ints * np.float32(s)).astype(np.float32)
        x[0, :4] = [0.0, -0.0, np.float32(s), -np.float32(s)]
        y = ops.ternary_linear(torch.from_numpy(x).to(cuda), nw).cpu().numpy()
        assert np.array_equal(y, x), s


def test_hip_graph_replays_match_eager(cuda, oracle):
    """The GEMV captured into a HIP graph (K = 16384: the launch that opts in to more than 64 KiB of LDS; an fp32
    row: the kernel that scales inside) gives the eager result on every replay, with eager work and
    synchronisations between the replays."""
    from tmq_amd import ops
    rng = np.random.default_rng(11)
    for K, N, dt in ((16384, 520, torch.float16), (4096, 1000, torch.float32), (11008, 300, torch.float16)):
        W, nw = _layer(cuda, oracle, rng, N, K)
        x = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float32)).to(cuda).to(dt)
        eager = ops.ternary_linear(x, nw).clone()
        torch.cuda.synchronize()
        graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
        with torch.cuda.stream(side):
            y = torch.empty(1, N, device=cuda)
            with torch.cuda.graph(graph, stream=side):
                y.copy_(ops.ternary_linear(x, nw))
        for rep in range(3):
            y.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, eager), (K, rep)
            x2 = torch.randn_like(x)                               # eager work on the same weights in between
            ops.ternary_linear(x2, nw)
            torch.cuda.synchronize()


# ---- two to four rows: row m's four term planes ride in activation columns 4 m .. 4 m + 3 -----------------------
@pytest.mark.parametrize("M,K", [(2, 2048), (2, 4096), (2, 2304), (3, 2048), (4, 2048), (2, 8192), (4, 4096), (2, 6144), (2, 5120), (2, 7168)])
@pytest.mark.parametrize("N", [16, 1000, 4100])
def test_few_rows_on_the_8bit_instruction(cuda, oracle, M, K, N):
    from tmq_amd import ops
    rng = np.random.default_rng(100 * M + K + N)
    W, nw = _layer(cuda, oracle, rng, N, K)
    x = rng.standard_normal((M, K)).astype(np.float16)
    x[M - 1] *= np.float16(37.0)                                  # rows of different magnitude must not mix
    t = lambda a: torch.from_numpy(a).to(cuda)
    y = ops.ternary_linear(t(x), nw)
    ref = x.astype(np.float64) @ W.astype(np.float64).T
    assert y.shape == (M, N)
    for m in range(M):
        assert _rel_err(y[m].cpu().numpy(), ref[m]) <= 1e-5, m
    # two rows of up to 4096 indices run on the 8-bit kernel like the single row (three and four take the fp16 weight
    # stream): every row equals the single-row launch of that row, bit for bit -- same instruction, same order
    if M == 2 and K <= 4096:
        for m in range(M):
            assert torch.equal(ops.ternary_linear(t(x[m:m + 1]), nw)[0], y[m]), m
    scale = (0.01 + 0.02 * rng.random(N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    res = rng.standard_normal((M, N)).astype(np.float16)
    y2 = ops.ternary_linear(t(x), nw, t(scale), t(bias), residual=t(res), relu=True, out_dtype=torch.float16)
    assert _rel_err(y2.float().cpu().numpy(), np.maximum(ref * scale + bias + res.astype(np.float64), 0)) <= 1e-3


def test_few_rows_pass_every_finite_fp16_value_through(cuda, oracle):
    """Identity weights, up to four rows at once: every finite fp16 value comes back exactly in its own row, from the
    kernel that splits the rows itself (K = 2048) and from prepared planes (K = 4096)."""
    from tmq_amd import ops
    vals = np.arange(65536, dtype=np.uint32).astype(np.uint16).view(np.float16).copy()
    vals[~np.isfinite(vals)] = 0
    vals = vals[np.random.default_rng(8).permutation(65536)]
    for K, prepared in ((2048, False), (4096, True)):
        nw = ops.NativeWeights(torch.from_numpy(oracle.pack(np.eye(K, dtype=np.float32)).view(np.int32)).to(cuda), K)
        for M in (2, 3, 4):
            for c in range(0, 65536 // K - M + 1, M):
                x = vals[c * K:(c + M) * K].reshape(M, K)
                tx = torch.from_numpy(x).to(cuda)
                y = ops.ternary_linear_planes(ops.gemv8_prepare(tx), nw) if prepared else ops.ternary_linear(tx, nw)
                assert np.array_equal(y.cpu().numpy(), x.astype(np.float32)), (K, M, c)
    # exact on integers whatever the order of summation
    rng = np.random.default_rng(12)
    W, nw2 = _layer(cuda, oracle, rng, 520, 4096)
    xi = rng.integers(-8, 9, size=(4, 4096)).astype(np.float16)
    y = ops.ternary_linear(torch.from_numpy(xi).to(cuda), nw2).cpu().numpy()
    assert np.array_equal(y.astype(np.float64), xi.astype(np.float64) @ W.astype(np.float64).T)


# ---- the term planes made once (tmq_gemv8_prepare) and multiplied with several layers ---------------------------
@pytest.mark.parametrize("M,K", [(1, 2048), (1, 4096), (1, 11008), (1, 16384), (2, 8192), (2, 6912), (3, 4096), (4, 4096),
                                 (4, 2304)])
def test_prepared_planes_give_the_plain_call_s_values(cuda, oracle, M, K):
    from tmq_amd import ops
    rng = np.random.default_rng(M * 1000 + K)
    N = 1000
    W, nw = _layer(cuda, oracle, rng, N, K)
    W2, nw2 = _layer(cuda, oracle, rng, 272, K)
    x = rng.standard_normal((M, K)).astype(np.float16)
    t = lambda a: torch.from_numpy(a).to(cuda)
    assert ops.gemv8_planes_supported(M, K)
    planes = ops.gemv8_prepare(t(x))
    ref = x.astype(np.float64) @ W.astype(np.float64).T
    y = ops.ternary_linear_planes(planes, nw)
    assert y.shape == (M, N) and _rel_err(y.cpu().numpy(), ref) <= 1e-5
    for m in range(M):                                             # same bits as the single-row kernel that splits in place
        assert torch.equal(ops.ternary_linear(t(x[m:m + 1]), nw)[0], y[m]), m
    y2 = ops.ternary_linear_planes(planes, nw2)                     # the same planes against another layer
    assert _rel_err(y2.cpu().numpy(), x.astype(np.float64) @ W2.astype(np.float64).T) <= 1e-5
    scale = (0.01 + 0.02 * rng.random(N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    res = rng.standard_normal((M, N)).astype(np.float32)
    y3 = ops.ternary_linear_planes(planes, nw, t(scale), t(bias), residual=t(res), relu=True)
    assert _rel_err(y3.cpu().numpy(), np.maximum(ref * scale + bias + res, 0)) <= 1e-5


def test_prepared_planes_limits_and_graph_replay(cuda, oracle):
    from tmq_amd import ops
    assert not ops.gemv8_planes_supported(5, 4096) and not ops.gemv8_planes_supported(4, 8192)
    assert not ops.gemv8_planes_supported(2, 16384)
    assert not ops.gemv8_planes_supported(1, 1024) and not ops.gemv8_planes_supported(1, 4100)
    with pytest.raises(RuntimeError):
        ops.gemv8_prepare(torch.zeros(5, 4096, dtype=torch.float16, device=cuda))
    rng = np.random.default_rng(13)
    K, N = 16384, 520
    W, nw = _layer(cuda, oracle, rng, N, K)
    x = torch.from_numpy(rng.standard_normal((1, K)).astype(np.float16)).to(cuda)
    eager = ops.ternary_linear_planes(ops.gemv8_prepare(x), nw).clone()
    torch.cuda.synchronize()
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    with torch.cuda.stream(side):
        y = torch.empty(1, N, device=cuda)
        with torch.cuda.graph(graph, stream=side):
            y.copy_(ops.ternary_linear_planes(ops.gemv8_prepare(x), nw))
    for rep in range(3):
        y.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), rep
        ops.ternary_linear(torch.randn_like(x), nw)
        torch.cuda.synchronize()
