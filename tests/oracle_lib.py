"""numpy front end of the CPU oracle (oracle/libtmq_oracle.so). Test infrastructure only."""
import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
SO = os.path.join(ORACLE_DIR, "libtmq_oracle.so")

_lib = None
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
_sz, _dbl, _i64, _int, _flt = ctypes.c_size_t, ctypes.c_double, ctypes.c_int64, ctypes.c_int, ctypes.c_float


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(SO):
            subprocess.check_call(["make", "-C", ORACLE_DIR, "-s"])
        L = ctypes.CDLL(SO)
        L.tmq_oracle_consts.argtypes = [_dbl] + [ctypes.POINTER(_flt)] * 3
        L.tmq_oracle_softstep_fwd.argtypes = [_f32p, _f32p, _sz, _dbl]
        L.tmq_oracle_softstep_bwd.argtypes = [_f32p, _f32p, _f32p, _sz, _dbl, _dbl]
        L.tmq_oracle_deriv_fwd.argtypes = [_f32p, _f32p, _sz, _dbl, _dbl]
        L.tmq_oracle_deriv_bwd.argtypes = [_f32p, _f32p, _f32p, _sz, _dbl, _dbl]
        L.tmq_oracle_map.argtypes = [_f32p, _f32p, _sz, _dbl]
        L.tmq_oracle_dmap.argtypes = [_f32p, _f32p, _sz, _dbl]
        L.tmq_oracle_ternarize.argtypes = [_f32p, _f32p, _sz, _dbl]
        L.tmq_oracle_round.argtypes = [_f32p, _f32p, _sz]
        L.tmq_oracle_clamp.argtypes = [_f32p, _f32p, _sz, _dbl, _dbl]
        L.tmq_oracle_fused.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, ctypes.POINTER(_dbl), _sz, _dbl, _dbl,
                                       _dbl, _flt, _dbl, _dbl]
        L.tmq_oracle_sum64.argtypes = [_f32p, _sz]
        L.tmq_oracle_sum64.restype = _dbl
        L.tmq_oracle_pack.argtypes = [ctypes.c_void_p, _int, _i64, _i64, _u32p]
        L.tmq_oracle_unpack.argtypes = [_u32p, _i64, _i64, _f32p, _int]
        L.tmq_oracle_unpack_ref2d_as_written.argtypes = [_u32p, _i64, _i64, _i64, _f32p]
        L.tmq_oracle_unpack_ref2d_as_written.restype = _int
        L.tmq_oracle_gemm.argtypes = [_f32p, _i64, _i64, _u32p, _i64, ctypes.c_void_p, ctypes.c_void_p, _f64p]
        L.tmq_oracle_conv2d.argtypes = [_f32p] + [_i64] * 4 + [_u32p] + [_i64] * 9 + [ctypes.c_void_p,
                                                                                     ctypes.c_void_p, _f64p]
        L.tmq_oracle_dwconv_patches.argtypes = [_f32p, _i64, _i64, _i64, _u32p, _f64p]
        L.tmq_oracle_dwconvtrans_cols.argtypes = [_f32p, _i64, _i64, _i64, _i64, _u32p, _f32p]
        L.tmq_oracle_compress.argtypes = [_u32p, _i64, _i64, ctypes.POINTER(ctypes.POINTER(ctypes.c_uint8))]
        L.tmq_oracle_compress.restype = _i64
        L.tmq_oracle_free.argtypes = [ctypes.c_void_p]
        L.tmq_oracle_decompress.argtypes = [_u8p, _i64, _u32p, _i64, _i64]
        L.tmq_oracle_decompress.restype = _i64
        _lib = L
    return _lib


def _c(a, dt=np.float32):
    return np.ascontiguousarray(a, dtype=dt).reshape(-1)


def consts(d):
    a, b, c = _flt(), _flt(), _flt()
    lib().tmq_oracle_consts(d, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c))
    return np.float32(a.value), np.float32(b.value), np.float32(c.value)


def softstep_fwd(w, d):
    w = _c(w); y = np.empty_like(w); lib().tmq_oracle_softstep_fwd(w, y, w.size, d); return y


def softstep_bwd(w, g, d, scale=1.0):
    w = _c(w); g = _c(g); o = np.empty_like(w); lib().tmq_oracle_softstep_bwd(w, g, o, w.size, d, scale); return o


def deriv_fwd(w, d, strength):
    w = _c(w); o = np.empty_like(w); lib().tmq_oracle_deriv_fwd(w, o, w.size, d, strength); return o


def deriv_bwd(w, g, d, strength):
    w = _c(w); g = _c(g); o = np.empty_like(w); lib().tmq_oracle_deriv_bwd(w, g, o, w.size, d, strength); return o


def softstep_map(w, d):
    w = _c(w); o = np.empty_like(w); lib().tmq_oracle_map(w, o, w.size, d); return o


def softstep_dmap(w, d):
    w = _c(w); o = np.empty_like(w); lib().tmq_oracle_dmap(w, o, w.size, d); return o


def ternarize(w, d):
    w = _c(w); o = np.empty_like(w); lib().tmq_oracle_ternarize(w, o, w.size, d); return o


def round_half_even(w):
    w = _c(w); o = np.empty_like(w); lib().tmq_oracle_round(w, o, w.size); return o


def clamp(w, lo, hi):
    w = _c(w); o = np.empty_like(w); lib().tmq_oracle_clamp(w, o, w.size, lo, hi); return o


def fused(w, g, d, sharp, strength, gl, lo, hi):
    w = _c(w); g = _c(g)
    y, dw, wc = np.empty_like(w), np.empty_like(w), np.empty_like(w)
    s = _dbl(0.0)
    lib().tmq_oracle_fused(w, g, y, dw, wc, ctypes.byref(s), w.size, d, sharp, strength, gl, lo, hi)
    return y, dw, wc, s.value


def sum64(x):
    x = _c(x); return lib().tmq_oracle_sum64(x, x.size)


_DT = {np.dtype(np.float32): 0, np.dtype(np.int32): 1, np.dtype(np.int8): 2}


def pack(w2d):
    """W [N][K] (fp32 / int32 / int8) -> uint32 words [K][ceil(N/16)]."""
    w2d = np.ascontiguousarray(w2d)
    N, K = w2d.shape
    out = np.empty((K, (N + 15) // 16), dtype=np.uint32)
    lib().tmq_oracle_pack(w2d.ctypes.data_as(ctypes.c_void_p), _DT[w2d.dtype], N, K, out.reshape(-1))
    return out


def unpack(words, N, K, host_rule=0):
    words = np.ascontiguousarray(words, dtype=np.uint32)
    out = np.zeros((N, K), dtype=np.float32)
    lib().tmq_oracle_unpack(words.reshape(-1), N, K, out.reshape(-1), host_rule)
    return out


def unpack_ref2d_as_written(words, rows, cols):
    words = np.ascontiguousarray(words, dtype=np.uint32)
    out = np.zeros((rows, cols), dtype=np.float32)
    rc = lib().tmq_oracle_unpack_ref2d_as_written(words.reshape(-1), words.size, rows, cols, out.reshape(-1))
    return out if rc == 0 else None


def _opt(a):
    if a is None:
        return None, None
    a = _c(a)
    return a, a.ctypes.data_as(ctypes.c_void_p)


def gemm(x, words, N, scale=None, bias=None):
    """x [M][K] (any float dtype, taken exactly) x packed words [K][ceil(N/16)] -> fp64 [M][N]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    M, K = x.shape
    words = np.ascontiguousarray(words, dtype=np.uint32)
    y = np.empty((M, N), dtype=np.float64)
    s, sp = _opt(scale); b, bp = _opt(bias)
    lib().tmq_oracle_gemm(x.reshape(-1), M, K, words.reshape(-1), N, sp, bp, y.reshape(-1))
    return y


def conv2d(x, words, N, k, stride, pad, dil=(1, 1), scale=None, bias=None):
    """x NCHW -> fp64 NCHW."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    B, C, H, W = x.shape
    ky, kx = k; sy, sx = stride; py, px = pad; dy, dx = dil
    Ho = (H + 2 * py - dy * (ky - 1) - 1) // sy + 1
    Wo = (W + 2 * px - dx * (kx - 1) - 1) // sx + 1
    words = np.ascontiguousarray(words, dtype=np.uint32)
    y = np.empty((B, N, Ho, Wo), dtype=np.float64)
    s, sp = _opt(scale); b, bp = _opt(bias)
    lib().tmq_oracle_conv2d(x.reshape(-1), B, C, H, W, words.reshape(-1), N, ky, kx, sy, sx, py, px, dy, dx, sp, bp,
                            y.reshape(-1))
    return y


def dwconv_patches(x, words):
    """x [P][T][C] -> fp64 [P][C] (depthwise: one ternary filter of T taps per channel)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    P, T, C = x.shape
    words = np.ascontiguousarray(words, dtype=np.uint32)
    y = np.empty((P, C), dtype=np.float64)
    lib().tmq_oracle_dwconv_patches(x.reshape(-1), P, T, C, words.reshape(-1), y.reshape(-1))
    return y


def dwconvtrans_cols(x, words, taps):
    """x [B][P][C] fp32 -> fp32 [B][C*taps][P], y[b][c*taps + t][p] = x[b][p][c] * T[c][t]."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    B, P, C = x.shape
    words = np.ascontiguousarray(words, dtype=np.uint32)
    y = np.empty((B, C * taps, P), dtype=np.float32)
    lib().tmq_oracle_dwconvtrans_cols(x.reshape(-1), B, P, taps, C, words.reshape(-1), y.reshape(-1))
    return y


def compress(words, rows, columns):
    words = np.ascontiguousarray(words, dtype=np.uint32).reshape(-1)
    p = ctypes.POINTER(ctypes.c_uint8)()
    n = lib().tmq_oracle_compress(words, rows, columns, ctypes.byref(p))
    if n < 0:
        raise ValueError(f"oracle compress failed: {n}")
    out = np.ctypeslib.as_array(p, shape=(n,)).copy()
    lib().tmq_oracle_free(p)
    return out


def decompress(stream, rows, columns):
    stream = np.ascontiguousarray(stream, dtype=np.uint8)
    out = np.zeros((rows, (columns + 15) // 16), dtype=np.uint32)
    n = lib().tmq_oracle_decompress(stream, stream.size, out.reshape(-1), rows, columns)
    if n < 0:
        raise ValueError(f"oracle decompress failed: {n}")
    return out
