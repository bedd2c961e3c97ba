"""ctypes view of libtmq_hip.so -- the C ABI declared in include/tmq_hip.h.

torch is used only to own device memory and to name the current stream; every computation goes
through the shared library. There is no CPU or PyTorch fallback: if the library is missing or a
call fails, an exception is raised.
"""
import contextlib
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtmq_hip.so")

F32, I32, I8, F16 = 0, 1, 2, 3
_DTYPE_CODE = {torch.float32: F32, torch.int32: I32, torch.int8: I8, torch.float16: F16}


class TmqError(RuntimeError):
    """A libtmq_hip entry point returned a non-zero status."""


class Segment(ctypes.Structure):
    """tmq_segment of include/tmq_hip.h (32 bytes)."""
    _fields_ = [("ptr", ctypes.c_void_p), ("aux", ctypes.c_void_p), ("n", ctypes.c_uint64),
                ("block_begin", ctypes.c_uint32), ("scalar", ctypes.c_float)]


class StepTensor(ctypes.Structure):
    """tmq_step_tensor of include/tmq_hip.h (32 bytes)."""
    _fields_ = [("w", ctypes.c_void_p), ("g", ctypes.c_void_p), ("out", ctypes.c_void_p), ("n", ctypes.c_uint64)]


class ConvShape(ctypes.Structure):
    """tmq_conv_shape of include/tmq_hip.h."""
    _fields_ = [(k, ctypes.c_int32) for k in
                ("B", "C", "H", "W", "N", "ky", "kx", "sy", "sx", "py", "px", "dy", "dx", "py_end", "px_end")]


class OutputView(ctypes.Structure):
    """tmq_output_view of include/tmq_hip.h."""
    _fields_ = [("h0", ctypes.c_int32), ("w0", ctypes.c_int32), ("h_cnt", ctypes.c_int32), ("w_cnt", ctypes.c_int32),
                ("stride_b", ctypes.c_int64), ("stride_h", ctypes.c_int64), ("stride_w", ctypes.c_int64)]


class Epilogue(ctypes.Structure):
    """tmq_epilogue of include/tmq_hip.h."""
    _fields_ = [("scale", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("residual", ctypes.c_void_p),
                ("relu", ctypes.c_int32), ("y_dtype", ctypes.c_int32)]


_vp, _sz, _dbl, _i64, _int, _flt, _u32 = (ctypes.c_void_p, ctypes.c_size_t, ctypes.c_double, ctypes.c_int64,
                                           ctypes.c_int, ctypes.c_float, ctypes.c_uint32)

# name -> (restype, argtypes); every symbol include/tmq_hip.h declares.
SIGNATURES = {
    "tmq_version": (_int, []),
    "tmq_status_string": (ctypes.c_char_p, [_int]),
    "tmq_last_hip_error": (_int, []),
    "tmq_softstep_fwd": (_int, [_vp, _vp, _sz, _dbl, _vp]),
    "tmq_softstep_bwd": (_int, [_vp, _vp, _vp, _sz, _dbl, _dbl, _vp]),
    "tmq_softstep_deriv_fwd": (_int, [_vp, _vp, _sz, _dbl, _dbl, _vp]),
    "tmq_softstep_deriv_bwd": (_int, [_vp, _vp, _vp, _sz, _dbl, _dbl, _vp]),
    "tmq_softstep_map": (_int, [_vp, _vp, _sz, _dbl, _int, _vp]),
    "tmq_sigmoid_piece": (_int, [_vp, _vp, _sz, _int, _vp]),
    "tmq_clamp_inplace": (_int, [_vp, _sz, _dbl, _dbl, _vp]),
    "tmq_ternarize_inplace": (_int, [_vp, _sz, _dbl, _vp]),
    "tmq_softstep_fused_workspace_bytes": (_sz, [_sz]),
    "tmq_softstep_fused": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _dbl, _dbl, _dbl, _flt, _dbl, _dbl, _vp]),
    "tmq_softstep_fused_noalloc_max_elements": (_sz, []),
    "tmq_softstep_fused_noalloc": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _dbl, _dbl, _dbl, _flt, _dbl, _dbl, _vp]),
    "tmq_loss_state_bytes": (_sz, []),
    "tmq_softstep_fused_inlaunch": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _dbl, _dbl, _dbl, _flt, _dbl, _dbl, _vp]),
    "tmq_qloss_multi_inlaunch": (_int, [_vp, _int, _u32, _dbl, _dbl, _vp, _vp, _vp, _vp]),
    "tmq_selfcheck_division": (_int, [_dbl, _vp, _vp]),
    "tmq_probe_stream_read": (_int, [_vp, ctypes.c_size_t, _vp, _vp]),
    "tmq_split_f32": (_int, [_vp, _vp, _vp, _i64, _vp]),
    "tmq_split_f32_scaled": (_int, [_vp, _vp, _vp, _vp, _i64, _vp]),
    "tmq_f32_prescale_workspace_bytes": (_sz, [_i64]),
    "tmq_f32_to_f16_prescaled_workspace_bytes": (_sz, [_i64]),
    "tmq_f32_to_f16_prescaled": (_int, [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _vp]),
    "tmq_f32_prescale": (_int, [_vp, _i64, _vp, _vp, _vp, _vp, _i64, _vp, _vp]),
    "tmq_selfcheck_fastdiv": (_i64, [_u32, _vp, _i64]),
    "tmq_fp32_rows_prefer_split": (_int, [_i64, _i64, _i64]),
    "tmq_fp32_rows_self_scaled": (_int, [_vp, _i64, _i64]),
    "tmq_fp32_rows_self_scaled_for": (_int, [_vp, _i64, _i64, _i64]),
    "tmq_multi_plan": (_int, [ctypes.POINTER(Segment), _int, ctypes.POINTER(_u32)]),
    "tmq_qloss_multi_workspace_bytes": (_sz, [_u32]),
    "tmq_qloss_multi": (_int, [_vp, _int, _u32, _dbl, _dbl, _vp, _vp, _vp, _vp]),
    "tmq_qloss_bwd_multi": (_int, [_vp, _int, _u32, _dbl, _dbl, _vp, _int, _vp]),
    "tmq_clamp_multi": (_int, [_vp, _int, _u32, _dbl, _dbl, _vp]),
    "tmq_softstep_multi_workspace_bytes": (_sz, [ctypes.POINTER(StepTensor), _int]),
    "tmq_softstep_fwd_multi": (_int, [ctypes.POINTER(StepTensor), _int, _dbl, _dbl, _dbl, _vp, _vp, _vp, _vp]),
    "tmq_softstep_fwd_multi_inlaunch": (_int, [ctypes.POINTER(StepTensor), _int, _dbl, _dbl, _dbl, _vp, _vp, _vp, _vp]),
    "tmq_softstep_bwd_multi": (_int, [ctypes.POINTER(StepTensor), _int, _dbl, _dbl, _dbl, _vp, _vp]),
    "tmq_pack_ternary": (_int, [_vp, _int, _i64, _i64, _vp, _vp]),
    "tmq_unpack_ternary": (_int, [_vp, _i64, _i64, _vp, _vp]),
    "tmq_native_weight_bytes": (_sz, [_i64, _i64]),
    "tmq_prepack_weights": (_int, [_vp, _i64, _i64, _i64, _i64, _vp, _vp]),
    "tmq_ternary_linear": (_int, [_vp, _int, _i64, _i64, _vp, _i64, _vp, _vp, _vp]),
    "tmq_conv2d_out_hw": (_int, [ctypes.POINTER(ConvShape), ctypes.POINTER(ctypes.c_int32),
                                 ctypes.POINTER(ctypes.c_int32)]),
    "tmq_avgpool_linear": (_int, [_vp, _i64, _i64, _i64, _vp, _i64, _vp, _vp, _vp]),
    "tmq_ternary_conv2d": (_int, [_vp, ctypes.POINTER(ConvShape), _vp, _vp, _vp, _vp]),
    "tmq_ternary_conv2d_view": (_int, [_vp, ctypes.POINTER(ConvShape), _vp, _vp, _vp, ctypes.POINTER(OutputView), _vp]),
    "tmq_ternary_conv2d_relu_maxpool": (_int, [_vp, ctypes.POINTER(ConvShape), _vp, _vp, _vp, _vp, _vp]),
    "tmq_ternary_conv2d_relu_maxpool_planar": (_int, [_vp, ctypes.c_int32, ctypes.POINTER(ConvShape), _vp, _vp, _vp, _vp, _vp]),
    "tmq_ternary_dwconv2d": (_int, [_vp, ctypes.POINTER(ConvShape), _vp, _vp, _vp, _vp]),
    "tmq_ternary_dwconv_patches": (_int, [_vp, _int, _i64, ctypes.c_int32, _i64, _vp, _vp, _vp]),
    "tmq_maxpool2d_nhwc": (_int, [_vp] + [ctypes.c_int32] * 10 + [_vp, _vp]),
    "tmq_avgpool_global_nhwc": (_int, [_vp, _i64, _i64, _i64, _vp, _int, _vp]),
    "tmq_ternary_linear_workspace_bytes": (_sz, [_int, _i64, _i64, _i64]),
    "tmq_ternary_linear_ws": (_int, [_vp, _int, _i64, _i64, _vp, _i64, _vp, _vp, _vp, _sz, _vp]),
    "tmq_gemv8_planes_bytes": (_sz, [_i64, _i64]),
    "tmq_gemv8_prepare": (_int, [_vp, _i64, _i64, _vp, _vp]),
    "tmq_ternary_linear_planes": (_int, [_vp, _i64, _i64, _vp, _i64, _vp, _vp, _vp]),
    "tmq_nchw_to_nhwc4": (_int, [_vp, _int, _i64, ctypes.c_int32, _i64, _i64, _vp, _vp]),
    "tmq_convtranspose2d_out_hw": (_int, [ctypes.POINTER(ConvShape), ctypes.c_int32, ctypes.c_int32,
                                          ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32)]),
    "tmq_ternary_dwconvtrans2d": (_int, [_vp, ctypes.POINTER(ConvShape), ctypes.c_int32, ctypes.c_int32, _vp, _vp, _vp, _vp]),
    "tmq_ternary_dwconvtrans_cols": (_int, [_vp, _i64, _i64, ctypes.c_int32, _i64, _vp, _vp, _vp]),
    "tmq_compress_bound": (_sz, [_i64, _i64]),
    "tmq_compress_ternary": (_int, [_vp, _i64, _i64, _vp, _sz, ctypes.POINTER(_sz)]),
    "tmq_decompress_ternary": (_int, [_vp, _sz, _vp, _i64, _i64]),
}

_lib = None


def load():
    """Load libtmq_hip.so once and attach the prototypes. Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C tmq_amd/csrc` (or __graft_entry__.build()). "
                "tmq_amd has no CPU or PyTorch fallback for its kernels.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


ERR_UNSUPPORTED = -2     # TMQ_ERR_UNSUPPORTED


def check(status, what):
    if status != 0:
        lib = load()
        msg = lib.tmq_status_string(status).decode()
        extra = f" (hipError {lib.tmq_last_hip_error()})" if status == -3 else ""
        raise TmqError(f"{what}: {msg}{extra}")


def ptr(t):
    """Device (or host) address of a tensor, None for a missing optional tensor."""
    return None if t is None else ctypes.c_void_p(t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_current_device = getattr(torch._C, "_cuda_getDevice", None)
_STAY = contextlib.nullcontext()


def on_device(device):
    """Context in which `device` (a tensor's .device) is the current one: nothing to do, and nothing to pay, when it
    already is -- the usual case."""
    if _current_device is not None and device.index == _current_device():
        return _STAY
    return torch.cuda.device(device)


def stream_of(t):
    """The current HIP stream of the tensor's device, as the void* the ABI expects. (The raw handle where this
    PyTorch has the accessor: building a torch.cuda.Stream object per call costs ~4 us, more than a small kernel.)"""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(t.device.index))
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def dtype_code(t):
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise ValueError("Cannot handle the supplied data-type") from None


def require_gpu(t, name="tensor"):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def require_gpu_dense(t, name="tensor"):
    """On the GPU and dense in memory (contiguous in the default or the channels_last format)."""
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU")
    if not (t.is_contiguous() or (t.dim() == 4 and t.is_contiguous(memory_format=torch.channels_last))):
        raise RuntimeError(f"{name} must be dense in memory")
