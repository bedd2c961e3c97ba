"""Pins the oracle's pack / unpack / range coder, and the shipped host codec, on the CPU.

Sources of truth, strongest first: (1) golden vectors written by the reference's own host code
compiled from its sources (tests/golden/native_golden.npz, made by tests/golden/make_native_golden.py);
(2) the same compiled reference, live, where oracle/_ref exists (the build container only);
(3) hand-computed words of the format; (4) brute force and round trips.
"""
import ctypes
import importlib.util
import os

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = np.load(os.path.join(ROOT, "tests", "golden", "native_golden.npz"))
REF_SO = os.path.join(ROOT, "oracle", "_ref", "tmq_native.so")


def _ref():
    if not os.path.exists(REF_SO):
        pytest.skip("oracle/_ref not built (no reference tree here)")
    spec = importlib.util.spec_from_file_location("tmq_native", REF_SO)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _u32(a):
    return np.ascontiguousarray(a).view(np.uint32)


def test_hand_computed_words(oracle):
    assert oracle.pack(np.ones((16, 1), np.float32))[0, 0] == 0x55555555
    assert oracle.pack(-np.ones((16, 1), np.float32))[0, 0] == 0xAAAAAAAA
    w = np.zeros((16, 1), np.float32); w[0], w[1], w[15] = 1, -1, 1
    assert oracle.pack(w)[0, 0] == 0x60000001
    assert oracle.pack(np.ones((6, 1), np.float32))[0, 0] == 0x55500000        # ragged tail is zero-filled
    # transposed layout: word (k, q) holds W[16q + j][k]
    w = np.zeros((32, 3), np.float32); w[17, 2] = -1
    p = oracle.pack(w)
    assert p.shape == (3, 2) and p[2, 1] == (2 << 28) and np.count_nonzero(p) == 1


def test_all_byte_patterns_round_trip(oracle):
    # every sequence of 4 ternary values at each of the 4 byte positions of a word
    vals = np.array([0, 1, -1], np.float32)
    for pos in range(4):
        for code in range(81):
            d = [(code // 3 ** i) % 3 for i in range(4)]
            w = np.zeros((16, 1), np.float32)
            w[4 * pos:4 * pos + 4, 0] = vals[d]
            word = int(oracle.pack(w)[0, 0])
            want = 0
            for j in range(16):
                c = {0.0: 0, 1.0: 1, -1.0: 2}[float(w[j, 0])]
                want |= c << (30 - 2 * j)
            assert word == want
            assert np.array_equal(oracle.unpack(np.array([[word]], np.uint32), 16, 1), w)


@pytest.mark.parametrize("N", list(range(1, 18)) + [102])
def test_ragged_rows(oracle, N):
    rng = np.random.default_rng(N)
    w = rng.integers(-1, 2, (N, 5)).astype(np.float32)
    p = oracle.pack(w)
    assert p.shape == (5, (N + 15) // 16)
    assert np.array_equal(oracle.unpack(p, N, 5), w)
    if N % 16:
        assert np.all(p[:, -1] & np.uint32((1 << (2 * (16 - N % 16))) - 1) == 0)   # padding bits are zero


def test_oracle_matches_golden_pack_and_expand(oracle):
    n = int(GOLD["ncases"])
    for i in range(n):
        w = GOLD[f"w{i}"]
        N = w.shape[0]
        K = w.size // N
        words = oracle.pack(w.reshape(N, K))
        assert np.array_equal(words.reshape(-1), _u32(GOLD[f"compact{i}"]).reshape(-1)), i
        if w.ndim == 4:
            assert np.array_equal(oracle.unpack(words, N, K).reshape(w.shape), GOLD[f"expand{i}"]), i
            assert np.array_equal(GOLD[f"expand{i}"], w)
        else:
            # the reference's 2-D expander reads the words with rows and columns swapped; the oracle
            # keeps that routine for documentation and it must reproduce the reference's output,
            # while the true inverse reproduces the original weights.
            got = oracle.unpack_ref2d_as_written(words, w.shape[0], w.shape[1])
            if f"expand{i}" in GOLD:
                assert np.array_equal(got, GOLD[f"expand{i}"]), i
                assert not np.array_equal(got, w)          # ... and it is not the inverse
            else:
                assert got is None                          # the reference would read out of bounds
            assert np.array_equal(oracle.unpack(words, N, K), w), i
    assert np.array_equal(oracle.pack(GOLD["round_in"]).reshape(-1), _u32(GOLD["round_compact"]).reshape(-1))
    assert np.array_equal(oracle.pack(GOLD["i8_in"]).reshape(-1), _u32(GOLD["i8_compact"]).reshape(-1))
    assert np.array_equal(oracle.pack(GOLD["i32_in"]).reshape(-1), _u32(GOLD["i32_compact"]).reshape(-1))


def _shape_rows_cols(w):
    cols = w.shape[0]
    rows = w.size // cols
    return rows, cols


def test_oracle_codec_matches_golden_streams(oracle):
    for i in range(int(GOLD["ncases"])):
        w = GOLD[f"w{i}"]
        rows, cols = _shape_rows_cols(w)
        words = _u32(GOLD[f"compact{i}"]).reshape(rows, -1)
        stream = oracle.compress(words, rows, cols)
        assert np.array_equal(stream, GOLD[f"stream{i}"].view(np.uint8)), i
        assert np.array_equal(oracle.decompress(GOLD[f"stream{i}"].view(np.uint8), rows, cols), words), i


def _lib_compress(words, rows, cols):
    from tmq_amd import _capi
    lib = _capi.load()
    words = np.ascontiguousarray(words, np.uint32)
    cap = lib.tmq_compress_bound(rows, cols)
    buf = np.zeros(cap, np.uint8)
    size = ctypes.c_size_t(0)
    rc = lib.tmq_compress_ternary(words.ctypes.data_as(ctypes.c_void_p), rows, cols, buf.ctypes.data_as(ctypes.c_void_p),
                                  cap, ctypes.byref(size))
    return rc, buf[:size.value].copy()


def _lib_decompress(stream, rows, cols):
    from tmq_amd import _capi
    lib = _capi.load()
    stream = np.ascontiguousarray(stream, np.uint8)
    out = np.zeros((rows, (cols + 15) // 16), np.uint32)
    rc = lib.tmq_decompress_ternary(stream.ctypes.data_as(ctypes.c_void_p), stream.size,
                                    out.ctypes.data_as(ctypes.c_void_p), rows, cols)
    return rc, out


def test_shipped_codec_matches_golden_streams():
    for i in range(int(GOLD["ncases"])):
        w = GOLD[f"w{i}"]
        rows, cols = _shape_rows_cols(w)
        words = _u32(GOLD[f"compact{i}"]).reshape(rows, -1)
        rc, stream = _lib_compress(words, rows, cols)
        assert rc == 0
        assert np.array_equal(stream, GOLD[f"stream{i}"].view(np.uint8)), i
        rc, back = _lib_decompress(stream, rows, cols)
        assert rc == 0 and np.array_equal(back, words), i


@pytest.mark.parametrize("p0", [0.0, 0.2, 0.5, 0.9, 0.995])
@pytest.mark.parametrize("shape", [(1, 1), (16, 16), (300, 70), (102, 512), (4096, 64)])
def test_codec_round_trip_and_agreement(oracle, p0, shape):
    rng = np.random.default_rng(int(p0 * 1000) + shape[0])
    u = rng.random(shape)
    w = np.where(u < (1 - p0) / 2, 1.0, np.where(u < 1 - p0, -1.0, 0.0)).astype(np.float32)
    words = oracle.pack(w)                           # [K][ceil(N/16)]
    rows, cols = shape[1], shape[0]
    so = oracle.compress(words, rows, cols)
    rc, sl = _lib_compress(words, rows, cols)
    assert rc == 0 and np.array_equal(so, sl)
    assert np.array_equal(oracle.decompress(so, rows, cols), words)
    rc, back = _lib_decompress(sl, rows, cols)
    assert rc == 0 and np.array_equal(back, words)
    # header fields
    assert int.from_bytes(so[:8].tobytes(), "big") == rows * cols
    assert int.from_bytes(so[16:20].tobytes(), "big") == so.size
    assert int.from_bytes(so[8:16].tobytes(), "big") == 8 * (so.size - 26 - 1) and so[-1] == 0


def test_codec_size_is_near_entropy(oracle):
    rng = np.random.default_rng(0)
    u = rng.random((1024, 1024))
    w = np.where(u < .25, 1.0, np.where(u < .5, -1.0, 0.0)).astype(np.float32)
    s = oracle.compress(oracle.pack(w), 1024, 1024)
    bits_per_weight = 8.0 * s.size / w.size
    assert 1.49 < bits_per_weight < 1.52          # entropy of (.25, .5, .25) is 1.5 bit


def test_codec_rejects_bad_input(oracle):
    from tmq_amd import _capi
    words = np.array([[0xC0000000]], np.uint32)     # code 11
    with pytest.raises(ValueError):
        oracle.compress(words, 1, 16)
    rc, _ = _lib_compress(words, 1, 16)
    assert rc == -5
    rc, _ = _lib_decompress(np.zeros(10, np.uint8), 1, 16)
    assert rc == -5
    good = oracle.compress(np.array([[0x55555555]], np.uint32), 1, 16)
    rc, _ = _lib_decompress(good, 2, 16)            # symbol count in the header does not match the shape
    assert rc == -5


def test_live_reference_agrees_when_built(oracle):
    ref = _ref()
    rng = np.random.default_rng(99)
    for shape in [(40, 33), (102, 512), (16, 9, 3, 3), (130, 4, 5, 1)]:
        w = rng.integers(-1, 2, shape).astype(np.float32)
        N = shape[0]
        K = w.size // N
        compact = ref.compactify_ternary(torch.from_numpy(w))
        words = oracle.pack(w.reshape(N, K))
        assert np.array_equal(_u32(compact.numpy()).reshape(-1), words.reshape(-1))
        stream = ref.compress_ternary(torch.from_numpy(w), list(shape), False).numpy().view(np.uint8)
        assert np.array_equal(oracle.compress(words, K, N), stream)
        rc, sl = _lib_compress(words, K, N)
        assert rc == 0 and np.array_equal(sl, stream)
        back = ref.decompress_ternary(torch.from_numpy(sl.view(np.int8)), list(shape)).numpy()
        assert np.array_equal(_u32(back).reshape(-1), words.reshape(-1))
    for dt in (np.int32, np.int8):
        w = rng.integers(-3, 4, (50, 21)).astype(dt)
        assert np.array_equal(_u32(ref.compactify_ternary(torch.from_numpy(w)).numpy()).reshape(-1),
                              oracle.pack(w).reshape(-1))


def test_library_exports_every_declared_symbol():
    import re
    from tmq_amd import _capi
    lib = _capi.load()
    header = open(os.path.join(ROOT, "include", "tmq_hip.h")).read()
    declared = set(re.findall(r"\b(tmq_[a-z0-9_]+)\s*\(", header))
    declared -= {"tmq_status", "tmq_segment", "tmq_conv_shape", "tmq_epilogue"}
    assert declared, "no declarations found"
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in include/tmq_hip.h but not exported"
        assert name in _capi.SIGNATURES, f"{name} has no ctypes prototype"
    assert lib.tmq_version() >= 100
    assert lib.tmq_status_string(-5).decode().startswith("malformed")


def test_torch_extension_exports_the_reference_names():
    """tmq/tmq_cuda.cu:800-809 and tmq/tmq_native.cpp:550-555: the twelve names tmq.py imports."""
    from tmq_amd import tmq_hip_ext as ext
    for name in ("fwd_softstep", "bwd_softstep", "fwd_softstep_derivative", "bwd_softstep_derivative",
                 "ternary_mmm_cuda", "ternary_mvm_cuda", "ternary_dwconv_cuda", "ternary_dwconvtrans_cuda",
                 "compactify_ternary", "compress_ternary", "decompress_ternary", "expand_ternary"):
        assert callable(getattr(ext, name)), name
    # the host codec needs no GPU: a stream written by the reference's coder decodes to the same words
    g = np.load(os.path.join(ROOT, "tests", "golden", "native_golden.npz"))
    for i in range(3):
        w, compact, stream = g[f"w{i}"], g[f"compact{i}"], g[f"stream{i}"]
        words = ext.decompress_ternary(torch.from_numpy(stream.view(np.int8).copy()), list(w.shape)).numpy()
        assert words.shape == compact.shape and np.array_equal(_u32(words), _u32(compact))
        assert np.array_equal(ext.compress_ternary(torch.from_numpy(compact.view(np.int32).copy()), list(w.shape), True).numpy().view(np.uint8),
                              stream.view(np.uint8))


def test_oracle_depthwise_patches_is_the_textbook_sum(oracle):
    """y[p][c] = sum_t x[p][t][c] T[c][t] against numpy's einsum on the unpacked weights, ragged C."""
    rng = np.random.default_rng(9)
    for (P, T, C) in [(5, 9, 16), (3, 4, 5), (11, 25, 40), (2, 1, 1)]:
        u = rng.random((C, T))
        W = np.where(u < .25, 1.0, np.where(u < .5, -1.0, 0.0)).astype(np.float32)
        words = oracle.pack(W)                                   # [T][ceil(C/16)]
        x = rng.standard_normal((P, T, C)).astype(np.float32)
        want = np.einsum("ptc,ct->pc", x.astype(np.float64), W.astype(np.float64))
        assert np.allclose(oracle.dwconv_patches(x, words), want, rtol=0, atol=1e-12)


def test_oracle_transposed_depthwise_columns_are_the_outer_product(oracle):
    """y[b][c T + t][p] = x[b][p][c] * T[c][t] against numpy on the unpacked weights (bit for bit: the
    products are exact), ragged C, several batch entries."""
    rng = np.random.default_rng(10)
    for (B, P, T, C) in [(1, 5, 9, 16), (2, 3, 4, 5), (3, 11, 6, 40), (1, 1, 1, 1)]:
        u = rng.random((C, T))
        W = np.where(u < .25, 1.0, np.where(u < .5, -1.0, 0.0)).astype(np.float32)
        words = oracle.pack(W)
        x = rng.standard_normal((B, P, C)).astype(np.float32)
        want = (x.transpose(0, 2, 1)[:, :, None, :] * W[None, :, :, None]).reshape(B, C * T, P)
        assert np.array_equal(oracle.dwconvtrans_cols(x, words, T).view(np.uint32), want.view(np.uint32))


def test_pixel_index_division_constants():
    """The convolution / pooling kernels divide an output pixel's index by image extents with a multiply-high
    by host-computed constants. Host-only check of those constants against integer division: every divisor up
    to 4096 and a few large ones, on multiples of the divisor and their neighbours, both ends of the 31-bit
    range and random dividends."""
    import ctypes
    from tmq_amd import _capi
    lib = _capi.load()
    rng = np.random.default_rng(3)
    big = np.uint64(2 ** 31 - 1)
    for d in list(range(1, 4097)) + [65535, 65536, 65537, 1000003, 2 ** 30, 2 ** 30 + 1, 2 ** 31 - 1]:
        k = rng.integers(0, int(big) // d + 1, 300, dtype=np.uint64)
        mult = k * np.uint64(d)
        n = np.concatenate([mult, mult + np.uint64(d - 1), np.maximum(mult, 1) - 1,
                            rng.integers(0, 2 ** 31, 300, dtype=np.uint64),
                            np.array([0, 1, d - 1, d, min(d + 1, int(big)), int(big), int(big) - 1], dtype=np.uint64)])
        n = np.minimum(n, big).astype(np.uint32)
        bad = lib.tmq_selfcheck_fastdiv(d, n.ctypes.data_as(ctypes.c_void_p), n.size)
        assert bad == 0, f"divisor {d}: {bad} wrong quotients"
    assert lib.tmq_selfcheck_fastdiv(0, n.ctypes.data_as(ctypes.c_void_p), 1) == -1
