"""The PyTorch extension (tmq_amd/tmq_hip_ext, the reference's twelve binding names over the C ABI)
must agree bit for bit with the ctypes binding that the rest of the suite checks against the oracle,
and raise the reference's error classes."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ext():
    from tmq_amd import tmq_hip_ext
    return tmq_hip_ext


def test_softstep_family_matches_ctypes_binding(cuda, ext):
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(1)
    w = (torch.rand(100003, device=cuda, generator=g) * 2.1 - 1.05).view(-1)
    grad = torch.randn(100003, device=cuda, generator=g)
    for d in (0.1, 3.0004, 6.0):
        assert torch.equal(ext.fwd_softstep(w, d), ops.fwd_softstep(w, d))
        assert torch.equal(ext.bwd_softstep(w, d, 1.0, grad), ops.bwd_softstep(w, d, 1.0, grad))
        assert torch.equal(ext.fwd_softstep_derivative(w, 5.0, 5e-4), ops.fwd_softstep_derivative(w, 5.0, 5e-4))
        assert torch.equal(ext.bwd_softstep_derivative(w, 5.0, 5e-4, grad), ops.bwd_softstep_derivative(w, 5.0, 5e-4, grad))
    # shape is kept, strided input is accepted
    w2 = w[:9000].view(90, 100)[:, ::2]
    assert ext.fwd_softstep(w2, 1.0).shape == w2.shape
    assert torch.equal(ext.fwd_softstep(w2, 1.0), ops.fwd_softstep(w2.contiguous(), 1.0))
    with pytest.raises(RuntimeError):
        ext.fwd_softstep(w.cpu(), 1.0)
    with pytest.raises(ValueError):                     # fp16 "Not implemented yet" (tmq_cuda.cu:759)
        ext.fwd_softstep(w.half(), 1.0)


def test_pack_codec_round_trip_and_oracle(cuda, ext, oracle):
    from tmq_amd import ops
    rng = np.random.default_rng(4)
    for shape in [(102, 512), (64, 3, 7, 7), (33, 65)]:
        u = rng.random(shape)
        w = np.where(u < .25, 1.0, np.where(u < .5, -1.0, 0.0)).astype(np.float32)
        tw = torch.from_numpy(w)
        words = ext.compactify_ternary(tw)                       # CPU in -> CPU out
        assert not words.is_cuda and words.dtype == torch.int32
        N, K = shape[0], int(np.prod(shape[1:]))
        assert np.array_equal(words.numpy().view(np.uint32).reshape(K, -1), oracle.pack(w.reshape(N, K)))
        assert torch.equal(ext.compactify_ternary(tw.to(cuda)).cpu(), words)
        assert torch.equal(ext.expand_ternary(words, list(shape), False), tw)
        stream = ext.compress_ternary(words, list(shape), True)
        assert torch.equal(stream, ops.compress_ternary(words, list(shape), True))
        assert torch.equal(ext.compress_ternary(tw, list(shape), False), stream)
        assert torch.equal(ext.decompress_ternary(stream, list(shape)), words)
        assert torch.equal(ext.expand_ternary(stream, list(shape), True), tw)
    with pytest.raises(ValueError):
        ext.compactify_ternary(torch.zeros(4, 4, dtype=torch.float64))
    with pytest.raises(RuntimeError):
        ext.decompress_ternary(torch.zeros(5, dtype=torch.int8), [4, 4])


def test_ternary_products_match_ctypes_binding(cuda, ext):
    from tmq_amd import ops
    g = torch.Generator(device=cuda).manual_seed(2)
    for (M, K, N) in [(1, 4096, 4096), (7, 512, 102), (300, 4096, 96), (64, 2304, 512), (1024, 2048, 2048)]:
        W = torch.randint(-1, 2, (N, K), device=cuda, generator=g).float()
        words = ext.compactify_ternary(W)
        x = torch.randn(M, K, device=cuda, generator=g)
        for xx in (x, x.half()):
            y = ext.ternary_mmm_cuda(xx, words, N)
            assert torch.equal(y, ops.ternary_mmm_cuda(xx, words, N))
            assert y.shape == (M, N) and y.dtype == torch.float32
        if M == 1:
            v = ext.ternary_mvm_cuda(x.view(K), words, N)
            assert v.shape == (N,) and torch.equal(v, ops.ternary_mvm_cuda(x.view(K), words, N))
        # a second call hits the cached native layout
        assert torch.equal(ext.ternary_mmm_cuda(x, words, N), ops.ternary_mmm_cuda(x, words, N))
    w = torch.zeros(32, 4, dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError):
        ext.ternary_mmm_cuda(torch.zeros(2, 32), w, 64)                       # CPU lhs
    with pytest.raises(RuntimeError):
        ext.ternary_mmm_cuda(torch.zeros(2, 32, device=cuda), w, 65)          # width check (tmq_cuda.cu:489)
    with pytest.raises(RuntimeError):
        ext.ternary_mvm_cuda(torch.zeros(2, 32, device=cuda), w, 64)          # batch > 1 (tmq_cuda.cu:584)
    with pytest.raises(RuntimeError):
        ext.ternary_dwconv_cuda(torch.zeros(1, device=cuda), w, 3, 3, 4)
    assert tuple(ext.ternary_mmm_cuda(torch.zeros(32, device=cuda), w, 64).shape) == (1, 64)
    assert tuple(ext.ternary_mmm_cuda(torch.zeros(1, 3, 5, 32, device=cuda), w, 64).shape) == (1, 3, 5, 64)
