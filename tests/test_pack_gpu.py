"""GPU parity of 2-bit pack / unpack (through the C ABI) vs the CPU oracle: bit-exact."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SHAPES_2D = [(1, 1), (16, 1), (17, 3), (6, 5), (102, 512), (64, 147), (256, 64), (4096, 256), (300, 1000), (33, 65),
             (64, 4608), (520, 260), (48, 1024), (1, 256), (4100, 300), (130, 2052)]   # K >= 256, K % 4 == 0: the 256-k tiles
SHAPES_4D = [(64, 3, 7, 7), (128, 64, 3, 3), (102, 16, 1, 1), (20, 5, 3, 2)]


def _ternary(rng, shape, p0=0.5):
    u = rng.random(shape)
    return np.where(u < (1 - p0) / 2, 1.0, np.where(u < 1 - p0, -1.0, 0.0)).astype(np.float32)


@pytest.mark.parametrize("shape", SHAPES_2D)
def test_pack_matrix_all_dtypes(cuda, oracle, shape):
    from tmq_amd import ops
    rng = np.random.default_rng(shape[0] * 1000 + shape[1])
    w = _ternary(rng, shape)
    want = oracle.pack(w)
    for dt, tdt in ((np.float32, torch.float32), (np.int32, torch.int32), (np.int8, torch.int8)):
        got = ops.compactify_ternary(torch.from_numpy(w.astype(dt)).to(cuda))
        assert got.dtype == torch.int32 and tuple(got.shape) == (shape[1], (shape[0] + 15) // 16)
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want), dt
    # CPU tensor in -> CPU tensor out (the reference's calling convention)
    got = ops.compactify_ternary(torch.from_numpy(w))
    assert not got.is_cuda and np.array_equal(got.numpy().view(np.uint32), want)
    # unpack is the true inverse
    back = ops.expand_ternary(torch.from_numpy(want.view(np.int32)).to(cuda), list(shape))
    assert np.array_equal(back.cpu().numpy(), w)
    assert np.array_equal(oracle.unpack(want, shape[0], shape[1]), w)


@pytest.mark.parametrize("shape", SHAPES_4D)
def test_pack_conv_kernel(cuda, oracle, shape):
    from tmq_amd import ops
    rng = np.random.default_rng(sum(shape))
    w = _ternary(rng, shape)
    N = shape[0]
    K = shape[1] * shape[2] * shape[3]
    want = oracle.pack(w.reshape(N, K))
    got = ops.compactify_ternary(torch.from_numpy(w).to(cuda))
    assert tuple(got.shape) == (shape[1], shape[2], shape[3], (N + 15) // 16)
    assert np.array_equal(got.cpu().numpy().view(np.uint32).reshape(K, -1), want)
    back = ops.expand_ternary(got, list(shape))
    assert np.array_equal(back.cpu().numpy(), w)


def test_rounding_and_clamping_of_float_input(cuda, oracle):
    from tmq_amd import ops
    v = np.array([0.5, -0.5, 0.49999997, -0.49999997, 1.5, -1.5, 2.5, -2.5, 0.0, -0.0, 1e-30, 7.0, -7.0, 3e9, -3e9,
                  np.inf, -np.inf, np.nan, 2147483520.0, 2147483648.0, 0.50000006, 1e38], dtype=np.float32)
    for K, col in ((3, 1), (256, 77), (516, 515)):            # the scalar tiles and the 256-k tiles
        w = np.zeros((32, K), dtype=np.float32)
        w[:v.size, col] = v
        want = oracle.pack(w)
        got = ops.compactify_ternary(torch.from_numpy(w).to(cuda)).cpu().numpy().view(np.uint32)
        assert np.array_equal(got, want), K
    iv = np.array([0, 1, -1, 2, -2, 127, -128, 5, -5], dtype=np.int8)
    wi = np.zeros((16, 2), dtype=np.int8); wi[:iv.size, 0] = iv
    assert np.array_equal(ops.compactify_ternary(torch.from_numpy(wi).to(cuda)).cpu().numpy().view(np.uint32),
                          oracle.pack(wi))
    i32 = np.array([0, 1, -1, 2 ** 31 - 1, -2 ** 31, 70000, -70000], dtype=np.int32)
    w32 = np.zeros((16, 2), dtype=np.int32); w32[:i32.size, 1] = i32
    assert np.array_equal(ops.compactify_ternary(torch.from_numpy(w32).to(cuda)).cpu().numpy().view(np.uint32),
                          oracle.pack(w32))


def test_unpack_decodes_code_11_as_zero(cuda, oracle):
    from tmq_amd import ops
    words = np.array([[0xFFFFFFFF, 0x6C000001]], dtype=np.uint32)     # 1 row (k), 2 words -> N = 32
    got = ops.expand_ternary(torch.from_numpy(words.view(np.int32)).to(cuda), [32, 1]).cpu().numpy()
    assert np.array_equal(got, oracle.unpack(words, 32, 1, host_rule=0))
    assert np.all(got[:16] == 0)


def test_full_size_roundtrip(cuda):
    """4096 x 4096 (the linear-layer configuration): pack -> unpack -> pack is the identity."""
    from tmq_amd import ops
    g = torch.Generator().manual_seed(10)
    u = torch.rand(4096, 4096, generator=g)
    w = torch.where(u < .25, 1.0, torch.where(u < .5, -1.0, 0.0)).to(cuda)
    p = ops.compactify_ternary(w)
    assert tuple(p.shape) == (4096, 256)
    assert torch.equal(ops.expand_ternary(p, [4096, 4096]), w)
    assert torch.equal(ops.compactify_ternary(ops.expand_ternary(p, [4096, 4096])), p)
    # popcount identity: number of non-zero codes equals number of non-zero weights
    codes = torch.stack([(p >> (30 - 2 * j)) & 3 for j in range(16)], -1)
    assert int((codes != 0).sum()) == int((w != 0).sum()) and int((codes == 3).sum()) == 0


def test_errors(cuda):
    from tmq_amd import ops
    with pytest.raises(RuntimeError):
        ops.compactify_ternary(torch.zeros(4, 4, 4, device=cuda))
    with pytest.raises(RuntimeError):
        ops.compactify_ternary(torch.zeros(4, device=cuda))
    with pytest.raises(ValueError):
        ops.compactify_ternary(torch.zeros(4, 4, device=cuda, dtype=torch.float64))
    with pytest.raises(RuntimeError):
        ops.expand_ternary(torch.zeros(4, 1, device=cuda, dtype=torch.int32), [16, 5])
