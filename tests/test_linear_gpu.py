"""GPU parity of the ternary linear kernels (through the C ABI) vs the CPU oracle.

Bar: relative error <= 1e-3 against an fp64-accumulated product on the exactly expanded weights
(the stated tolerance for this path); in practice the fp32-accumulated MFMA result is ~1e-6.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
RTOL = 1e-3


def _ternary(rng, N, K, p0=0.5):
    u = rng.random((N, K))
    return np.where(u < (1 - p0) / 2, 1.0, np.where(u < 1 - p0, -1.0, 0.0)).astype(np.float32)


def _rel_err(got, want):
    want = np.asarray(want, np.float64)
    got = np.asarray(got, np.float64)
    return np.max(np.abs(got - want)) / max(1e-30, np.max(np.abs(want)))


SHAPES = [  # (M, K, N)
    (1, 32, 16), (1, 256, 16), (1, 4096, 64), (1, 147, 64), (1, 512, 102), (3, 40, 17), (16, 512, 256),
    (17, 300, 50), (33, 1000, 130), (64, 576, 64), (64, 512, 102), (48, 2304, 128), (1, 7, 5),
    (100, 256, 48), (130, 147, 64), (256, 512, 96),
]


@pytest.mark.parametrize("M,K,N", SHAPES)
def test_linear_fp16_matches_oracle(cuda, oracle, M, K, N):
    from tmq_amd import ops
    rng = np.random.default_rng(M * 7 + K * 3 + N)
    W = _ternary(rng, N, K)
    words = oracle.pack(W)
    x = rng.standard_normal((M, K)).astype(np.float16)
    scale = (0.5 + rng.random(N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    tw = torch.from_numpy(words.view(np.int32)).to(cuda)
    nw = ops.NativeWeights(tw, N)
    tx = torch.from_numpy(x).to(cuda)
    y = ops.ternary_linear(tx, nw, torch.from_numpy(scale).to(cuda), torch.from_numpy(bias).to(cuda))
    want = oracle.gemm(x.astype(np.float32), words, N, scale, bias)
    assert y.shape == (M, N) and y.dtype == torch.float32
    assert _rel_err(y.cpu().numpy(), want) <= RTOL
    # what fp32 accumulation actually delivers; a single row with K a multiple of 256 from 2048 on runs on the 8-bit matrix
    # instructions, whose 32-product adder rounds a little more coarsely
    tight = 1e-5 if (M == 1 and K % 256 == 0 and K >= 2048) else 2e-6
    assert _rel_err(y.cpu().numpy(), want) <= tight
    y0 = ops.ternary_linear(tx, nw)                          # no scale / bias
    assert _rel_err(y0.cpu().numpy(), oracle.gemm(x.astype(np.float32), words, N)) <= tight
    # the textbook routine on expanded weights
    ref = x.astype(np.float64) @ W.astype(np.float64).T
    assert _rel_err(y0.cpu().numpy(), ref) <= tight


@pytest.mark.parametrize("M,K,N", [(1, 4096, 4096), (16, 4096, 4096), (5, 300, 70), (64, 1024, 256), (200, 512, 64),
                                   (2, 2048, 1000), (3, 4096, 70), (4, 2304, 520), (1, 16384, 4100), (5, 2048, 200), (8, 4096, 1000), (7, 16384, 4096)])
def test_linear_fp32_activations(cuda, oracle, M, K, N):
    """fp32 activations (the reference's calling convention) keep fp32-level accuracy."""
    from tmq_amd import ops
    rng = np.random.default_rng(K + N + M)
    W = _ternary(rng, N, K)
    words = oracle.pack(W)
    x = rng.standard_normal((M, K)).astype(np.float32)
    tw = torch.from_numpy(words.view(np.int32)).to(cuda)
    y = ops.ternary_mmm_cuda(torch.from_numpy(x).to(cuda), tw, N)
    ref = x.astype(np.float64) @ W.astype(np.float64).T
    assert _rel_err(y.cpu().numpy(), ref) <= 5e-6
    if M == 1:
        for shape in ((K,), (1, K), (1, 1, K), (1, 1, 1, K)):
            v = ops.ternary_mvm_cuda(torch.from_numpy(x.reshape(shape)).to(cuda), tw, N)
            assert tuple(v.shape) == shape[:-1] + (N,)
            assert _rel_err(v.cpu().numpy().reshape(1, N), ref) <= 5e-6


def test_split_f32_terms(cuda):
    """hi = fp16(x), lo = fp16(x - hi), bit for bit, on aligned, ragged and unaligned buffers."""
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(5)
    base = torch.randn(1 << 16, device=cuda, generator=g) * torch.pow(10.0, torch.randint(-6, 4, (1 << 16,), device=cuda, generator=g).float())
    base[:8] = torch.tensor([0.0, -0.0, 65504.0, -65504.0, 1e-8, 70000.0, 1.0 + 2.0 ** -12, -3.0], device=cuda)
    for x in (base, base[:4099], base[1:2050], base[:5]):
        hi, lo = ops.split_f32(x)
        want_hi = x.half()
        want_lo = (x - want_hi.float()).half()
        assert torch.equal(hi.view(torch.int16), want_hi.view(torch.int16))
        assert torch.equal(lo.view(torch.int16), want_lo.view(torch.int16))
    fin = torch.isfinite(hi.float())
    x = base[:5]
    assert torch.all((hi.float() + lo.float() - x).abs()[fin] <= x.abs()[fin] * 2.0 ** -21 + 1e-7)


@pytest.mark.parametrize("M,K,N", [(1024, 1024, 4096), (600, 4096, 2048), (10, 8192, 8192), (5, 16384, 8192)])
def test_linear_fp32_many_rows(cuda, M, K, N):
    """Many fp32 rows run as two passes of the fp16 kernels over the two fp16 terms of the activations:
    fp32-level accuracy against the fp64 product, with every epilogue option."""
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(M + K)
    W = torch.randint(-1, 2, (N, K), dtype=torch.int8, device=cuda, generator=g)
    nw = ops.NativeWeights(ops.compactify_ternary(W), N)
    x = torch.randn(M, K, device=cuda, generator=g)
    scale = 0.5 + torch.rand(N, device=cuda, generator=g)
    bias = torch.randn(N, device=cuda, generator=g)
    res = torch.randn(M, N, device=cuda, generator=g)
    ref = x.double() @ W.double().T
    y = ops.ternary_linear(x, nw)
    assert ((y.double() - ref).abs().max() / ref.abs().max()).item() <= 5e-6
    y2 = ops.ternary_linear(x, nw, scale, bias, residual=res, relu=True)
    ref2 = torch.relu(ref * scale.double() + bias.double() + res.double())
    assert ((y2.double() - ref2).abs().max() / ref2.abs().max()).item() <= 5e-6
    # the fp16 product of the same activations is three orders of magnitude coarser
    y16 = ops.ternary_linear(x.half(), nw)
    assert ((y16.double() - ref).abs().max() / ref.abs().max()).item() > 5e-5
    # integers: exact
    xi = torch.randint(-8, 9, (M, K), device=cuda, generator=g).float()
    assert torch.equal(ops.ternary_linear(xi, nw), xi @ W.float().T)


def test_exactness_on_integers(cuda, oracle):
    """With small-integer activations every product and partial sum is exact in fp32, so the
    result must equal the integer matrix product bit for bit, whatever the summation order."""
    from tmq_amd import ops
    rng = np.random.default_rng(3)
    for (M, K, N) in [(1, 4096, 256), (16, 1024, 48), (64, 147, 64), (300, 512, 32)]:
        W = _ternary(rng, N, K)
        x = rng.integers(-8, 9, (M, K)).astype(np.float16)
        words = oracle.pack(W)
        nw = ops.NativeWeights(torch.from_numpy(words.view(np.int32)).to(cuda), N)
        y = ops.ternary_linear(torch.from_numpy(x).to(cuda), nw).cpu().numpy()
        ref = (x.astype(np.int64) @ W.astype(np.int64).T).astype(np.float32)
        assert np.array_equal(y, ref)


WIDE = [  # (M, K, N, fp32 activations): wide layers take the register-blocked variants of the skinny kernel
    (1, 1024, 8192, False), (3, 520, 8200, False), (1, 16384, 16384, False), (1, 16640, 16400, False),
    (7, 16384, 16464, True), (16, 4096, 16384, False), (2, 33000, 16384, False), (1, 4096, 8192, True),
]


MID = [  # batches between the skinny kernel and the big-tile kernel, both activation types
    (65, 4096, 4096, False), (256, 4096, 4096, False), (256, 4096, 4096, True), (128, 4096, 4096, False),
    (100, 1000, 4100, False), (777, 2304, 520, False), (300, 4096, 96, True), (1024, 1024, 1024, False),
    (2048, 512, 4096, False), (96, 8192, 2048, True), (65, 264, 40, False), (513, 4096, 1000, True),
    # the big-tile kernel at the full benchmark shape and around its tile-choice boundaries
    (4096, 4096, 4096, False), (1024, 4096, 4096, False), (2048, 4096, 4096, False), (3000, 2112, 1000, False),
    (40, 512, 102, False), (64, 512, 102, True), (33, 256, 4096, False),
    # 2 .. 16 rows with whole blocks and at most two per wavefront: private activation windows
    (3, 256, 70, False), (5, 1024, 1000, False), (15, 4096, 4096, False), (16, 4096, 4096, False), (2, 2048, 8192, False),
    (4, 8192, 1024, False), (16, 8192, 1024, False), (9, 768, 48, False), (16, 2048, 8192, False),
    # 64 x 128 split-reduction tiles (chosen where they save a pass over the CUs), ragged N included
    (512, 4096, 4096, False), (384, 1024, 4100, False), (256, 8192, 8192, False),
    # ... with pair-granular weights two pairs ahead (the weight blocks do not deal out evenly over four wavefronts):
    # 18, 19 / 20 and 6 / 7 pairs per wavefront, i.e. every tail of the three-slot ring; ragged M and N
    (512, 4608, 4096, False), (500, 4928, 4100, False), (512, 1600, 4096, False),
    # 32 x 32 and 16 x 32 split-reduction tiles (few rows: smaller tiles keep every CU busy), ragged shapes included
    (17, 4096, 4096, False), (64, 4096, 4096, True), (96, 2048, 2048, False), (128, 8192, 1024, False),
    (192, 8192, 1024, False), (50, 1000, 1001, False), (31, 192, 4100, True), (20, 64, 33, False),
]


STREAM = [  # at most 16 fp16 rows, K a multiple of 256 and >= 2048: every geometry of the weight-stream kernel
    (1, 2048, 70, False), (2, 4096, 1000, False), (3, 2304, 520, False), (4, 2048, 8200, False), (4, 2560, 4096, False),
    (5, 4096, 12300, False), (7, 2048, 8200, False), (8, 3072, 4100, False), (9, 4096, 12304, False), (12, 2048, 8192, False),
    (16, 16384, 4096, False), (13, 2304, 48, False), (6, 8192, 28672, False), (1, 28672, 8192, False),
    # 9 .. 16 rows with odd block counts per wavefront: every drain of the static pipeline
    (12, 6144, 520, False), (16, 7168, 100, False), (10, 5120, 8200, False), (9, 12800, 64, False),
    # fp32 rows on the small tiles of the register-staged split-reduction kernel
    (17, 4096, 4096, True), (64, 4096, 1024, True), (100, 2048, 1000, True),
    # a few fp32 rows: the fp32 form of the weight-stream kernel
    (4, 2048, 8200, True), (2, 8192, 1024, True), (3, 2560, 40, True), (1, 2048, 16, True), (8, 2048, 8200, True), (6, 4096, 100, True), (16, 4096, 1000, True), (11, 2304, 8200, True), (13, 6144, 64, True),
]


@pytest.mark.parametrize("M,K,N,x32", WIDE + MID + STREAM)
def test_wide_layers_exact_on_integers(cuda, M, K, N, x32):
    """Small-integer activations, power-of-two scales and integer biases: every intermediate is
    exact in fp32, so the output must equal the integer matrix product bit for bit. The expected
    value comes from an fp32 library matmul on the expanded weights (exact for the same reason)."""
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(M + K + N)
    W = torch.randint(-1, 2, (N, K), dtype=torch.int8, device=cuda, generator=g)
    x = torch.randint(-8, 9, (M, K), device=cuda, generator=g).float()
    scale = torch.pow(2.0, torch.randint(-2, 3, (N,), device=cuda, generator=g).float())
    bias = torch.randint(-50, 51, (N,), device=cuda, generator=g).float()
    nw = ops.NativeWeights(ops.compactify_ternary(W), N)
    y = ops.ternary_linear(x if x32 else x.half(), nw, scale, bias)
    ref = (x @ W.float().T) * scale + bias
    assert torch.equal(y, ref)
    # one hot rows pick single weights: catches any permutation between channel blocks
    e = torch.zeros(2, K, device=cuda)
    e[0, K - 1] = 1.0
    e[1, K // 2 + 3] = 1.0
    ye = ops.ternary_linear(e.half(), nw)
    assert torch.equal(ye, torch.stack([W[:, K - 1], W[:, K // 2 + 3]]).float())


def test_code_11_decodes_to_zero_and_linearity(cuda, oracle):
    from tmq_amd import ops
    rng = np.random.default_rng(5)
    K, N, M = 512, 64, 8
    W = _ternary(rng, N, K)
    words = oracle.pack(W)
    bad = words.copy()
    bad[::7, ::2] |= (((bad[::7, ::2] >> 1) | bad[::7, ::2]) & 0x55555555 ^ 0x55555555) * 3   # turn 00 codes into 11
    x = rng.standard_normal((M, K)).astype(np.float16)
    tx = torch.from_numpy(x).to(cuda)
    y = ops.ternary_linear(tx, ops.NativeWeights(torch.from_numpy(words.view(np.int32)).to(cuda), N))
    yb = ops.ternary_linear(tx, ops.NativeWeights(torch.from_numpy(bad.view(np.int32)).to(cuda), N))
    assert torch.equal(y, yb)
    # linearity in x (exactly, for power-of-two factors)
    y2 = ops.ternary_linear(tx * 2, ops.NativeWeights(torch.from_numpy(words.view(np.int32)).to(cuda), N))
    assert torch.equal(y2, y * 2)


def test_reference_binding_checks(cuda):
    from tmq_amd import ops
    w = torch.zeros(32, 4, dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError):
        ops.ternary_mmm_cuda(torch.zeros(2, 32), w, 64)                       # CPU lhs
    with pytest.raises(RuntimeError):
        ops.ternary_mmm_cuda(torch.zeros(2, 32, device=cuda), w, 65)          # width check (tmq_cuda.cu:489)
    with pytest.raises(RuntimeError):
        ops.ternary_mmm_cuda(torch.zeros(2, 32, device=cuda), w, 48)          # width check (tmq_cuda.cu:490)
    with pytest.raises(RuntimeError):
        ops.ternary_mvm_cuda(torch.zeros(2, 32, device=cuda), w, 64)          # batch > 1 (tmq_cuda.cu:584)
    with pytest.raises(RuntimeError):
        ops.ternary_mmm_cuda(torch.zeros(2, 31, device=cuda), w, 64)          # K mismatch
    assert tuple(ops.ternary_mmm_cuda(torch.zeros(32, device=cuda), w, 64).shape) == (1, 64)
    assert tuple(ops.ternary_mmm_cuda(torch.zeros(1, 3, 5, 32, device=cuda), w, 64).shape) == (1, 3, 5, 64)
