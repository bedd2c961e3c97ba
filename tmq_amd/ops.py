"""Operator layer: the native-binding names of the reference (tmq_cuda / tmq_native), same
argument order and error behaviour, implemented on libtmq_hip through its C ABI.

Reference bindings: tmq/tmq_cuda.cu:800-809 and tmq/tmq_native.cpp:550-555. Every function
returns a newly allocated tensor owned by the caller and never mutates its inputs, like the
reference. Additive entry points (fused pass, multi-tensor forms, in-place clamp/ternarise, GPU
pack/unpack) follow below the drop-in ones.
"""
import ctypes

import torch

from . import _capi
from ._capi import check, ptr, stream_of


def _lib():
    return _capi.load()


def _f32_cuda(t, name):
    # tmq/tmq_cuda.cu:691-707: device check first, then the dtype ladder.
    if not t.is_cuda:
        raise RuntimeError(f"{name}: expected a tensor on the GPU")
    if t.dtype == torch.float16:
        raise ValueError("Not implemented yet")
    if t.dtype != torch.float32:
        raise ValueError("Expected either a float16 or a float32 tensor as input/output")
    return t if t.is_contiguous() else t.contiguous()


# ---- drop-in: soft-step family -------------------------------------------------------------
def fwd_softstep(weights: torch.Tensor, digamma: float) -> torch.Tensor:
    """Forward mapping for the soft-step function (tmq/tmq_cuda.cu:740-764)."""
    w = _f32_cuda(weights, "fwd_softstep")
    out = torch.empty_like(w)
    with _capi.on_device(w.device):
        check(_lib().tmq_softstep_fwd(ptr(w), ptr(out), w.numel(), float(digamma), stream_of(w)), "fwd_softstep")
    return out.view(weights.shape)


def bwd_softstep(weights: torch.Tensor, digamma: float, scale: float, grad: torch.Tensor) -> torch.Tensor:
    """Backward mapping incl. gradient multiplication (tmq/tmq_cuda.cu:768-794)."""
    w = _f32_cuda(weights, "bwd_softstep")
    if not grad.is_cuda:
        raise RuntimeError("bwd_softstep: expected a gradient on the GPU")
    if grad.dtype != w.dtype or grad.numel() != w.numel():
        raise RuntimeError("bwd_softstep: gradient must match the weights in dtype and size")
    g = grad if grad.is_contiguous() else grad.contiguous()
    out = torch.empty_like(w)
    with _capi.on_device(w.device):
        check(_lib().tmq_softstep_bwd(ptr(w), ptr(g), ptr(out), w.numel(), float(digamma), float(scale),
                                      stream_of(w)), "bwd_softstep")
    return out.view(weights.shape)


def fwd_softstep_derivative(weights: torch.Tensor, digamma: float, strength: float) -> torch.Tensor:
    """Forward mapping for the derivative of the soft-step function (tmq/tmq_cuda.cu:690-709)."""
    w = _f32_cuda(weights, "fwd_softstep_derivative")
    out = torch.empty_like(w)
    with _capi.on_device(w.device):
        check(_lib().tmq_softstep_deriv_fwd(ptr(w), ptr(out), w.numel(), float(digamma), float(strength),
                                            stream_of(w)), "fwd_softstep_derivative")
    return out.view(weights.shape)


def bwd_softstep_derivative(weights: torch.Tensor, digamma: float, scale: float, grad: torch.Tensor) -> torch.Tensor:
    """Backward mapping for the derivative (tmq/tmq_cuda.cu:713-735); `scale` is the strength."""
    w = _f32_cuda(weights, "bwd_softstep_derivative")
    if not grad.is_cuda:
        raise RuntimeError("bwd_softstep_derivative: expected a gradient on the GPU")
    if grad.dtype != w.dtype or grad.numel() != w.numel():
        raise RuntimeError("bwd_softstep_derivative: gradient must match the weights in dtype and size")
    g = grad if grad.is_contiguous() else grad.contiguous()
    out = torch.empty_like(w)
    with _capi.on_device(w.device):
        check(_lib().tmq_softstep_deriv_bwd(ptr(w), ptr(g), ptr(out), w.numel(), float(digamma), float(scale),
                                            stream_of(w)), "bwd_softstep_derivative")
    return out.view(weights.shape)


# ---- additive: in-place clamp / ternarise, fused pass -----------------------------------------
def clamp_(weights: torch.Tensor, lo: float, hi: float) -> torch.Tensor:
    """In-place clamp of an fp32 GPU tensor (value-equivalent to tmq/tmq.py:696, 879)."""
    _capi.require_gpu(weights, "weights")
    if weights.dtype != torch.float32:
        raise ValueError("clamp_: fp32 only")
    with _capi.on_device(weights.device):
        check(_lib().tmq_clamp_inplace(ptr(weights), weights.numel(), float(lo), float(hi), stream_of(weights)),
              "clamp_")
    return weights


def ternarize_(weights: torch.Tensor, digamma: float = 0.0) -> torch.Tensor:
    """In place: round_half_even(SoftStep.map(w; digamma)) (tmq/tmq.py:293-295); digamma <= 0
    gives plain round_half_even (tmq/tmq.py:603, 886, 1109)."""
    _capi.require_gpu(weights, "weights")
    if weights.dtype != torch.float32:
        raise ValueError("ternarize_: fp32 only")
    with _capi.on_device(weights.device):
        check(_lib().tmq_ternarize_inplace(ptr(weights), weights.numel(), float(digamma), stream_of(weights)),
              "ternarize_")
    return weights


_loss_states = {}


def loss_state(device):
    """The accumulator cells of the loss reductions that finish inside their launch (tmq_*_inlaunch): one small
    zero-filled buffer per device and stream, made on first use. Every launch leaves it zero, so it is never
    cleared again; launches on one stream are ordered, so they can share it."""
    device = torch.device(device)
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream(device).cuda_stream)
    st = _loss_states.get(key)
    if st is None:
        st = _loss_states[key] = torch.zeros(_lib().tmq_loss_state_bytes(), dtype=torch.uint8, device=device)
    return st


def softstep_fused(weights, grad, digamma, sharpness, strength, gl, lo, hi, *, want_y=True, want_dw=True,
                   want_clamp=True, want_loss=True, clamp_inplace=False, out=None, in_launch=False):
    """One pass: y = S(w), dw = g*S'(w) + gl*Q'(w), wc = clamp(w), loss_sum = sum q(w).

    Returns (y, dw, wc, loss_sum) with None for outputs not requested; loss_sum is a 1-element
    fp64 tensor. `out` may carry preallocated (y, dw, wc, loss_sum, workspace) to keep
    allocations out of a timed loop. in_launch: the loss sum is finished by the pass itself (fixed-point
    atomics, no finalisation launch, no workspace)."""
    _capi.require_gpu(weights, "weights")
    w = weights
    n = w.numel()
    lib = _lib()
    if out is not None:
        y, dw, wc, loss, ws = out
    else:
        y = torch.empty_like(w) if want_y else None
        dw = torch.empty_like(w) if want_dw else None
        wc = (w if clamp_inplace else torch.empty_like(w)) if want_clamp else None
        loss = torch.empty(1, dtype=torch.float64, device=w.device) if want_loss else None
        ws = torch.empty(lib.tmq_softstep_fused_workspace_bytes(n), dtype=torch.uint8, device=w.device) \
            if want_loss and not in_launch else None
    if dw is not None:
        _capi.require_gpu(grad, "grad")
        if grad.numel() != n or grad.dtype != torch.float32:
            raise RuntimeError("softstep_fused: gradient must match the weights")
    if in_launch and loss is not None and n:
        with _capi.on_device(w.device):
            status = lib.tmq_softstep_fused_inlaunch(ptr(w), ptr(grad) if dw is not None else None, ptr(y), ptr(dw), ptr(wc),
                                                     ptr(loss), ptr(loss_state(w.device)), n, float(digamma), float(sharpness),
                                                     float(strength), ctypes.c_float(gl), float(lo), float(hi), stream_of(w))
        if status != _capi.ERR_UNSUPPORTED:
            check(status, "softstep_fused_inlaunch")
            return y, dw, wc, loss
        if ws is None:
            ws = torch.empty(lib.tmq_softstep_fused_workspace_bytes(n), dtype=torch.uint8, device=w.device)
    with _capi.on_device(w.device):
        check(lib.tmq_softstep_fused(ptr(w), ptr(grad) if dw is not None else None, ptr(y), ptr(dw), ptr(wc),
                                     ptr(loss), ptr(ws), n, float(digamma), float(sharpness), float(strength),
                                     ctypes.c_float(gl), float(lo), float(hi), stream_of(w)), "softstep_fused")
    return y, dw, wc, loss


# ---- additive: multi-tensor forms ----------------------------------------------------------------
class SegmentTable:
    """Device-resident table of (weight, aux, n, scalar) for the multi-tensor launches. Build it
    once per set of tensors; rebuild when a tensor is reallocated."""

    def __init__(self, tensors, aux=None, scalars=None):
        lib = _lib()
        self.nseg = len(tensors)
        if self.nseg == 0:
            raise ValueError("SegmentTable: no tensors")
        dev = tensors[0].device
        arr = (_capi.Segment * self.nseg)()
        for i, t in enumerate(tensors):
            _capi.require_gpu(t, "segment tensor")
            if t.dtype != torch.float32 or t.device != dev:
                raise ValueError("SegmentTable: fp32 tensors on one device only")
            a = aux[i] if aux is not None else None
            if a is not None:
                _capi.require_gpu(a, "segment aux tensor")
                if a.numel() != t.numel() or a.dtype != torch.float32:
                    raise ValueError("SegmentTable: aux must match its tensor")
            arr[i].ptr = t.data_ptr()
            arr[i].aux = a.data_ptr() if a is not None else None
            arr[i].n = t.numel()
            arr[i].scalar = float(scalars[i]) if scalars is not None else 0.0
        total = ctypes.c_uint32(0)
        check(lib.tmq_multi_plan(arr, self.nseg, ctypes.byref(total)), "tmq_multi_plan")
        self.total_blocks = total.value
        self.key = tuple((t.data_ptr(), t.numel()) for t in tensors) + \
            tuple(a.data_ptr() if a is not None else 0 for a in (aux or []))
        host = torch.frombuffer(bytearray(bytes(arr)), dtype=torch.uint8)
        self.device = dev
        self.table = host.to(dev)
        self.workspace = torch.empty(lib.tmq_qloss_multi_workspace_bytes(self.total_blocks), dtype=torch.uint8,
                                     device=dev)
        self._keep = (list(tensors), list(aux) if aux is not None else None)


def qloss_multi(table: SegmentTable, sharpness: float, strength: float):
    """(per_tensor_means [nseg] fp32, total [1] fp32): one launch that finishes its own sums, or one launch + an ordered
    finalisation launch beyond that form's limits."""
    per = torch.empty(table.nseg, dtype=torch.float32, device=table.device)
    tot = torch.empty(1, dtype=torch.float32, device=table.device)
    with _capi.on_device(table.device):
        # finished inside the launch where the shape allows (up to 64 tensors, 2^18 blocks), else two launches
        status = _lib().tmq_qloss_multi_inlaunch(ptr(table.table), table.nseg, table.total_blocks, float(sharpness),
                                                 float(strength), ptr(per), ptr(tot), ptr(loss_state(table.device)),
                                                 stream_of(table.table)) if table.total_blocks else _capi.ERR_UNSUPPORTED
        if status != _capi.ERR_UNSUPPORTED:
            check(status, "qloss_multi_inlaunch")
            return per, tot
        check(_lib().tmq_qloss_multi(ptr(table.table), table.nseg, table.total_blocks, float(sharpness),
                                     float(strength), ptr(per), ptr(tot), ptr(table.workspace),
                                     stream_of(table.table)), "qloss_multi")
    return per, tot


def qloss_bwd_multi(table: SegmentTable, sharpness: float, strength: float, accumulate: bool, upstream=None):
    """aux_l (=|+=) s_l * Q'(w_l) for every segment, one launch; s_l = upstream / n_l when a device
    scalar `upstream` (fp32, 1 element) is given, else the table's per-tensor scalar."""
    if upstream is not None:
        _capi.require_gpu(upstream, "upstream")
        if upstream.dtype != torch.float32 or upstream.numel() != 1:
            raise RuntimeError("qloss_bwd_multi: upstream must be one fp32 value")
    with _capi.on_device(table.device):
        check(_lib().tmq_qloss_bwd_multi(ptr(table.table), table.nseg, table.total_blocks, float(sharpness),
                                         float(strength), ptr(upstream), int(bool(accumulate)),
                                         stream_of(table.table)), "qloss_bwd_multi")


def _carve(flat, offsets, like):
    """Tensors of the shapes of `like` on the storage of one flat buffer (not views of one another)."""
    out = []
    for off, t in zip(offsets, like):
        out.append(torch.empty(0, dtype=flat.dtype, device=flat.device).set_(flat.untyped_storage(), off, t.shape))
    return out


def _flat_offsets(tensors):
    """Element offsets of the tensors in one flat buffer, each starting on a 256-byte boundary."""
    offs, total = [], 0
    for t in tensors:
        offs.append(total)
        total += (t.numel() + 63) // 64 * 64
    return offs, total


def _step_weights(weights, name):
    if not weights:
        raise ValueError(f"{name}: no tensors")
    dev = weights[0].device
    ws = []
    for w in weights:
        w = _f32_cuda(w.detach(), name)
        if w.device != dev:
            raise RuntimeError(f"{name}: all tensors must live on one device")
        ws.append(w)
    return ws, dev


def softstep_fwd_all(weights, digamma: float, want_loss: bool = False, sharpness: float = 5.0, strength: float = 0.0):
    """y_l = S(w_l; digamma) for a list of fp32 GPU tensors in one launch (SoftStep.forward of every
    layer of a model, tmq/tmq.py:404-419) and, with want_loss, the total quantization loss
    sum_l mean(q(w_l; sharpness, strength)) (tmq/tmq.py:298-310) from the same pass over the weights.
    Returns (list of y, 0-dim fp32 loss or None)."""
    ws, dev = _step_weights(weights, "softstep_fwd_all")
    offs, total = _flat_offsets(ws)
    flat = torch.empty(total, dtype=torch.float32, device=dev)
    ys = _carve(flat, offs, ws)
    arr = (_capi.StepTensor * len(ws))()
    for i, (w, y) in enumerate(zip(ws, ys)):
        arr[i].w, arr[i].g, arr[i].out, arr[i].n = w.data_ptr(), None, y.data_ptr(), w.numel()
    lib = _lib()
    loss = wsp = None
    if want_loss:
        loss = torch.empty((), dtype=torch.float32, device=dev)
        # the loss finished inside the launch where the shape allows (up to 64 tensors of up to 2^18 blocks)
        with _capi.on_device(dev):
            status = lib.tmq_softstep_fwd_multi_inlaunch(arr, len(ws), float(digamma), float(sharpness), float(strength), None,
                                                         ptr(loss), ptr(loss_state(dev)), stream_of(flat))
        if status != _capi.ERR_UNSUPPORTED:
            check(status, "softstep_fwd_all")
            return ys, loss
        wsp = torch.empty(lib.tmq_softstep_multi_workspace_bytes(arr, len(ws)), dtype=torch.uint8, device=dev)
    with _capi.on_device(dev):
        check(lib.tmq_softstep_fwd_multi(arr, len(ws), float(digamma), float(sharpness), float(strength), None, ptr(loss),
                                         ptr(wsp), stream_of(flat)), "softstep_fwd_all")
    return ys, loss


def softstep_bwd_all(weights, grads, loss_upstream, digamma: float, sharpness: float = 5.0, strength: float = 0.0):
    """dw_l = g_l * S'(w_l; digamma) + (u / n_l) * Q'(w_l; sharpness, strength) for a list of tensors in
    one launch: the weight gradients of a whole step (tmq/tmq.py:422-438, 475-493 plus autograd's sum of
    the two). grads[l] may be None (no gradient reached y_l), loss_upstream (one fp32 GPU value u, the
    gradient arriving at the total quantization loss) may be None; a tensor that gets neither term
    yields None."""
    ws, dev = _step_weights(weights, "softstep_bwd_all")
    if len(grads) != len(ws):
        raise ValueError("softstep_bwd_all: one gradient (or None) per tensor")
    if loss_upstream is not None:
        _capi.require_gpu(loss_upstream, "loss_upstream")
        if loss_upstream.numel() != 1:
            raise RuntimeError("softstep_bwd_all: loss_upstream must be one value")
        loss_upstream = loss_upstream.detach().to(torch.float32).contiguous()
    live = [i for i in range(len(ws)) if grads[i] is not None or loss_upstream is not None]
    out = [None] * len(ws)
    if not live:
        return out
    offs, total = _flat_offsets([ws[i] for i in live])
    flat = torch.empty(total, dtype=torch.float32, device=dev)
    dws = _carve(flat, offs, [ws[i] for i in live])
    arr = (_capi.StepTensor * len(live))()
    keep = []
    for k, i in enumerate(live):
        g = grads[i]
        if g is not None:
            if not g.is_cuda or g.dtype != torch.float32 or g.numel() != ws[i].numel():
                raise RuntimeError("softstep_bwd_all: a gradient must match its weights in device, dtype and size")
            g = g.detach()
            g = g if g.is_contiguous() else g.contiguous()
            keep.append(g)
        arr[k].w, arr[k].g, arr[k].out, arr[k].n = ws[i].data_ptr(), (g.data_ptr() if g is not None else None), \
            dws[k].data_ptr(), ws[i].numel()
        out[i] = dws[k]
    with _capi.on_device(dev):
        check(_lib().tmq_softstep_bwd_multi(arr, len(live), float(digamma), float(sharpness), float(strength),
                                            ptr(loss_upstream), stream_of(flat)), "softstep_bwd_all")
    return out


def softstep_map(weights: torch.Tensor, digamma: float, derivative: bool = False) -> torch.Tensor:
    """SoftStep.map / SoftStep.dmap (tmq/tmq.py:328-350) on an fp32 GPU tensor."""
    w = _f32_cuda(weights, "softstep_map")
    out = torch.empty_like(w)
    with _capi.on_device(w.device):
        check(_lib().tmq_softstep_map(ptr(w), ptr(out), w.numel(), float(digamma), int(bool(derivative)),
                                      stream_of(w)), "softstep_map")
    return out.view(weights.shape)


def sigmoid_piece(x: torch.Tensor, order: int) -> torch.Tensor:
    """SoftStep.sigmoid (order 0), dsigmoid (1), d2sigmoid (2) of an fp32 GPU tensor (tmq/tmq.py:353-381)."""
    v = _f32_cuda(x, "sigmoid_piece")
    out = torch.empty_like(v)
    with _capi.on_device(v.device):
        check(_lib().tmq_sigmoid_piece(ptr(v), ptr(out), v.numel(), int(order), stream_of(v)), "sigmoid_piece")
    return out.view(x.shape)


def clamp_multi_(table: SegmentTable, lo: float, hi: float):
    """In-place clamp of every segment's weight tensor, one launch."""
    with _capi.on_device(table.device):
        check(_lib().tmq_clamp_multi(ptr(table.table), table.nseg, table.total_blocks, float(lo), float(hi),
                                     stream_of(table.table)), "clamp_multi_")


# ---- drop-in: 2-bit packing (tmq_native) ---------------------------------------------------------
def _gpu_device():
    if not torch.cuda.is_available():
        raise RuntimeError("tmq_amd needs a GPU: its pack/unpack kernels have no CPU fallback")
    return torch.device("cuda", torch.cuda.current_device())


def compactify_ternary(input: torch.Tensor) -> torch.Tensor:
    """Encode a ternary weight tensor into 16 elements per 32-bit word (tmq/tmq_native.cpp:418-425).

    [out, in] -> int32 [in, ceil(out/16)]; [out, in, ky, kx] -> int32 [in, ky, kx, ceil(out/16)].
    fp32 / int32 / int8 input. The reference accepts CPU tensors only; here a CPU tensor is staged
    through the GPU and the result returned on the CPU, a GPU tensor is packed in place on its
    device."""
    if input.dim() > 2 and input.dim() != 4:
        raise RuntimeError("compactify_ternary: expected a tensor with at most 2 or exactly 4 dimensions")
    if input.dim() < 2:
        raise RuntimeError("compactify_ternary: expected at least 2 dimensions")
    if input.dtype not in (torch.float32, torch.int32, torch.int8):
        raise ValueError("Cannot handle the supplied data-type")
    on_cpu = not input.is_cuda
    src = input.to(_gpu_device()) if on_cpu else input
    src = src.contiguous()
    N = src.shape[0]
    K = src.numel() // N if N else 0
    Q = (N + 15) // 16
    shape = (src.shape[1], Q) if src.dim() == 2 else (src.shape[1], src.shape[2], src.shape[3], Q)
    out = torch.empty(shape, dtype=torch.int32, device=src.device)
    with _capi.on_device(src.device):
        check(_lib().tmq_pack_ternary(ptr(src), _capi.dtype_code(src), N, K, ptr(out), stream_of(src)),
              "compactify_ternary")
    return out.cpu() if on_cpu else out


def expand_ternary(input: torch.Tensor, orig_shape, entropy_decode: bool = False) -> torch.Tensor:
    """Decode compact (or, with entropy_decode, range-coded) ternary weights to fp32 in the original
    shape (tmq/tmq_native.cpp:516-544). For 2-D tensors this is the true inverse of
    compactify_ternary (the reference decodes them with rows and columns swapped)."""
    orig_shape = [int(s) for s in orig_shape]
    if entropy_decode:
        input = decompress_ternary(input, orig_shape)
    if input.dtype != torch.int32:
        raise RuntimeError("expand_ternary: expected an int32 tensor")
    if len(orig_shape) not in (2, 4):
        raise ValueError("Shape needs to be of dim 2 or 4")
    on_cpu = not input.is_cuda
    src = (input.to(_gpu_device()) if on_cpu else input).contiguous()
    N = orig_shape[0]
    K = 1
    for s in orig_shape[1:]:
        K *= s
    if src.numel() != K * ((N + 15) // 16):
        raise RuntimeError("expand_ternary: packed tensor does not match the original shape")
    out = torch.empty(orig_shape, dtype=torch.float32, device=src.device)
    with _capi.on_device(src.device):
        check(_lib().tmq_unpack_ternary(ptr(src), N, K, ptr(out), stream_of(src)), "expand_ternary")
    return out.cpu() if on_cpu else out


def compress_ternary(input: torch.Tensor, orig_shape, from_compact: bool) -> torch.Tensor:
    """Range-code a ternary weight tensor (tmq/tmq_native.cpp:439-477). Returns a 1-D int8 CPU tensor.
    from_compact=True takes the int32 compact tensor, else fp32 weights (packed first)."""
    orig_shape = [int(s) for s in orig_shape]
    if from_compact:
        if input.dtype != torch.int32 or input.dim() not in (2, 4):
            raise RuntimeError("compress_ternary: expected a 2-D or 4-D int32 compact tensor")
        words = input
    else:
        if input.dtype != torch.float32:
            raise RuntimeError("compress_ternary: expected fp32 weights")
        words = compactify_ternary(input)
    words = words.detach().cpu().contiguous()
    columns = orig_shape[0]
    rows = words.numel() // ((columns + 15) // 16)
    lib = _lib()
    cap = lib.tmq_compress_bound(rows, columns)
    buf = torch.empty(cap, dtype=torch.int8)
    size = ctypes.c_size_t(0)
    check(lib.tmq_compress_ternary(ptr(words), rows, columns, ptr(buf), cap, ctypes.byref(size)), "compress_ternary")
    return buf[:size.value].clone()


def decompress_ternary(input: torch.Tensor, orig_shape) -> torch.Tensor:
    """Decode a range-coded stream into the int32 compact tensor (tmq/tmq_native.cpp:489-503)."""
    orig_shape = [int(s) for s in orig_shape]
    if input.is_cuda:
        raise RuntimeError("decompress_ternary: expected a CPU tensor")
    if input.dim() != 1 or input.dtype != torch.int8 or input.numel() < 26:
        raise RuntimeError("decompress_ternary: expected a 1-D int8 stream of at least 26 bytes")
    cols = orig_shape[0]
    qcols = (cols + 15) // 16
    if len(orig_shape) == 4:
        rows = orig_shape[1] * orig_shape[2] * orig_shape[3]
        out = torch.empty((orig_shape[1], orig_shape[2], orig_shape[3], qcols), dtype=torch.int32)
    else:
        rows = orig_shape[1]
        out = torch.empty((rows, qcols), dtype=torch.int32)
    src = input.contiguous()
    check(_lib().tmq_decompress_ternary(ptr(src), src.numel(), ptr(out), rows, cols), "decompress_ternary")
    return out


# ---- ternary inference ---------------------------------------------------------------------------------
class NativeWeights:
    """Kernel-native re-tiling of a compact weight tensor (still 2 bits per weight), built once
    per layer from the reference-format words; the compact tensor itself is left untouched."""

    def __init__(self, words: torch.Tensor, columns: int, conv_kernel=None):
        if words.dtype != torch.int32:
            raise RuntimeError("expected int32 compact weights")
        if not words.is_cuda:
            raise RuntimeError("expected compact weights on the GPU")
        w2 = words.reshape(-1, words.shape[-1]).contiguous()
        self.N = int(columns)
        self.K = int(w2.shape[0])
        q = w2.shape[1]
        if not (q * 16 >= self.N and q * 16 < self.N + 16):       # tmq/tmq_cuda.cu:489-490
            raise RuntimeError("compact weight width does not match the number of output columns")
        if conv_kernel is None:
            C, ky, kx = self.K, 1, 1
        else:
            ky, kx = conv_kernel
            if self.K % (ky * kx):
                raise RuntimeError("compact weight rows do not match the kernel size")
            C = self.K // (ky * kx)
        self.C, self.ky, self.kx = C, ky, kx
        lib = _lib()
        self.buf = torch.empty(lib.tmq_native_weight_bytes(self.N, self.K), dtype=torch.uint8, device=words.device)
        with _capi.on_device(words.device):
            check(lib.tmq_prepack_weights(ptr(w2), self.N, C, ky, kx, ptr(self.buf), stream_of(w2)), "prepack_weights")
        self.key = (words.data_ptr(), tuple(words.shape), words._version)


_native_cache = {}   # key -> (NativeWeights, compact tensor); insertion-ordered, least recently used first
_NATIVE_CACHE_SIZE = 64


def native_weights(words: torch.Tensor, columns: int, conv_kernel=None) -> NativeWeights:
    """NativeWeights for a compact tensor, cached across calls of the raw binding functions.

    The key is the storage address, shape and version counter of the compact tensor. The cache
    keeps a reference to that tensor, so its address cannot be handed to another tensor while the
    entry lives; entries are evicted least-recently-used. Compact tensors are expected to be immutable:
    a caller that passes `weight.data` (as the reference's layers do) hands over a tensor whose version
    counter never moves, so words overwritten in place at the same address are not noticed --
    clear_native_cache() after such a write."""
    key = (words.data_ptr(), tuple(words.shape), tuple(words.stride()), words._version, int(columns), conv_kernel,
           words.device.index)
    hit = _native_cache.pop(key, None)
    if hit is None:
        hit = (NativeWeights(words, columns, conv_kernel), words)
        while len(_native_cache) >= _NATIVE_CACHE_SIZE:
            _native_cache.pop(next(iter(_native_cache)))
    _native_cache[key] = hit
    return hit[0]


def clear_native_cache():
    """Forget every cached kernel-native weight buffer of the raw binding functions."""
    _native_cache.clear()


def _epilogue(nw, scale, bias, residual, relu, out_dtype, y):
    for t, name in ((scale, "scale"), (bias, "bias")):
        if t is not None:
            _capi.require_gpu(t, name)
            if t.dtype != torch.float32 or t.numel() != nw.N:
                raise RuntimeError(f"{name} must be fp32 with one entry per output channel")
    if out_dtype not in (torch.float32, torch.float16):
        raise RuntimeError("output dtype must be fp32 or fp16")
    if residual is not None:
        # (the stride of a dimension of size one says nothing about where the elements are)
        same_places = all(a == b for a, b, n in zip(residual.stride(), y.stride(), y.shape) if n > 1)
        if residual.dtype != out_dtype or residual.shape != y.shape or not same_places:
            raise RuntimeError("residual must match the output in shape, dtype and memory format")
    ep = _capi.Epilogue()
    ep.scale = scale.data_ptr() if scale is not None else None
    ep.bias = bias.data_ptr() if bias is not None else None
    ep.residual = residual.data_ptr() if residual is not None else None
    ep.relu = int(bool(relu))
    ep.y_dtype = _capi.F16 if out_dtype == torch.float16 else _capi.F32
    return ep


_fp32_prescale = True


def set_fp32_prescale(flag: bool) -> bool:
    """fp32 activations reach the fp16 MFMA kernels as fp16 terms. By default every fp32 tensor is first
    scaled by the power of two that puts its largest value into fp16's comfortable range (one extra small
    launch, exact, undone in the epilogue), so any magnitude works, as in the reference, which multiplies in
    fp32. A caller who knows its activations are of order 1 (max|x| <= 65504, nothing of interest below ~1e-4)
    can switch that off. (Most shapes take kernels that scale every row or group of rows themselves and the switch
    changes nothing for them; a thousand rows or more against at most 128 channels are the case where it pays: the
    kernel that splits fp32 values on the fly then reads the rows once, K = 4096, N = 16, M = 32768: 335 -> 128 us.)
    Returns the previous setting."""
    global _fp32_prescale
    prev, _fp32_prescale = _fp32_prescale, bool(flag)
    return prev


def f32_prescale(x: torch.Tensor, scale=None, channels: int = 0, want_copy: bool = False):
    """(prescale [2] = (s, 1 / s), s x or None, scale / s [channels] or None) for an fp32 GPU tensor: s is the
    power of two that brings max|x| into [1024, 2048). x must be dense (any memory format)."""
    _capi.require_gpu_dense(x, "activations")
    if x.dtype != torch.float32:
        raise RuntimeError("f32_prescale: expected fp32")
    lib = _lib()
    n = x.numel()
    ps = torch.empty(2, dtype=torch.float32, device=x.device)
    xs = torch.empty_like(x) if want_copy else None
    adj = torch.empty(channels, dtype=torch.float32, device=x.device) if channels else None
    if scale is not None and (scale.dtype != torch.float32 or scale.numel() != channels or not scale.is_cuda):
        raise RuntimeError("scale must be fp32 with one entry per output channel")
    wsb = lib.tmq_f32_prescale_workspace_bytes(n)
    ws = torch.empty(wsb, dtype=torch.uint8, device=x.device) if wsb else None
    with _capi.on_device(x.device):
        check(lib.tmq_f32_prescale(ptr(x), n, ptr(ps), ptr(xs), ptr(scale), ptr(adj), channels, ptr(ws), stream_of(x)),
              "f32_prescale")
    return ps, xs, adj


def split_f32(x: torch.Tensor, prescale=None, want_lo: bool = True):
    """(hi, lo) with hi = fp16(s x), lo = fp16(s x - hi): fp32 activations as two fp16 terms (s = prescale[0],
    1 without). lo is None with want_lo=False. The terms keep x's shape and memory format."""
    _capi.require_gpu_dense(x, "activations")
    if x.dtype != torch.float32:
        raise RuntimeError("split_f32: expected fp32")
    hi = torch.empty_like(x, dtype=torch.float16)
    lo = torch.empty_like(x, dtype=torch.float16) if want_lo else None
    with _capi.on_device(x.device):
        check(_lib().tmq_split_f32_scaled(ptr(x), ptr(prescale), ptr(hi), ptr(lo), x.numel(), stream_of(x)), "split_f32")
    return hi, lo


def f32_to_f16_prescaled(x: torch.Tensor, scale, channels: int):
    """One fp16 term of an fp32 activation tensor for the convolution kernels: (fp16 tensor of x's shape and
    memory format holding s x, scale / s) with the range prescale s, or (x.half(), scale) when the prescale
    is switched off."""
    if not _fp32_prescale or x.numel() == 0:      # nothing to scale in an empty batch
        return x.to(torch.float16), scale
    if not (x.is_contiguous() or x.is_contiguous(memory_format=torch.channels_last)):
        x = x.contiguous()
    _capi.require_gpu_dense(x, "activations")
    if scale is not None and (scale.dtype != torch.float32 or scale.numel() != channels or not scale.is_cuda):
        raise RuntimeError("scale must be fp32 with one entry per output channel")
    lib = _lib()
    n = x.numel()
    ps = torch.empty(2, dtype=torch.float32, device=x.device)
    hi = torch.empty_like(x, dtype=torch.float16)
    adj = torch.empty(channels, dtype=torch.float32, device=x.device) if channels else None
    ws = torch.empty(lib.tmq_f32_to_f16_prescaled_workspace_bytes(n), dtype=torch.uint8, device=x.device)
    with _capi.on_device(x.device):
        check(lib.tmq_f32_to_f16_prescaled(ptr(x), n, ptr(ps), ptr(hi), ptr(scale), ptr(adj), channels, ptr(ws), stream_of(x)),
              "f32_to_f16_prescaled")
    return hi, (adj if channels else scale)


def ternary_linear(x: torch.Tensor, nw: NativeWeights, scale=None, bias=None, residual=None, relu=False,
                   out_dtype=torch.float32) -> torch.Tensor:
    """y[..., n] = relu?(scale[n] * sum_k x[..., k] T[k][n] + bias[n] + residual); x fp16 or fp32."""
    _capi.require_gpu(x, "activations")
    if x.dtype not in (torch.float16, torch.float32):
        raise RuntimeError("ternary_linear: activations must be fp16 or fp32")
    if x.shape[-1] != nw.K:
        raise RuntimeError(f"ternary_linear: activations have {x.shape[-1]} features, weights expect {nw.K}")
    M = x.numel() // nw.K if nw.K else 0
    pairs = 0
    if (x.dtype == torch.float32 and 1 <= M <= 2 and x.is_contiguous()
            and _lib().tmq_fp32_rows_self_scaled_for(ptr(x), M, nw.K, nw.N)):
        pass            # one row (two over a small layer) the kernel scales itself, any magnitude: one launch
    elif (x.dtype == torch.float32 and M >= 1 and x.is_contiguous() and x.data_ptr() % 16 == 0
          and not (not _fp32_prescale and M >= 1024 and nw.N <= 128)
          and _lib().tmq_ternary_linear_workspace_bytes(_capi.F32, M, nw.K, nw.N)):
        # split once into fp16 row pairs in the workspace (a few rows: each scaled by its own power of two; from
        # seventeen: the whole tensor by one), then one pass of the fp16 kernels with the pairs added in the epilogue
        pairs = _lib().tmq_ternary_linear_workspace_bytes(_capi.F32, M, nw.K, nw.N)
    elif x.dtype == torch.float32 and M > 0:
        two_pass = (out_dtype == torch.float32 and (residual is None or residual.dtype == torch.float32)
                    and bool(_lib().tmq_fp32_rows_prefer_split(M, nw.K, nw.N)))
        ps = None
        if _fp32_prescale:
            if scale is not None:
                _capi.require_gpu(scale, "scale")
            # any magnitude: the tensor times a power of two, undone in the per-channel scale
            ps, xs, scale = f32_prescale(x, scale, nw.N, want_copy=not two_pass)
            x = x if two_pass else xs
        if two_pass:
            # many fp32 rows (or a few over a very large layer): two passes of the fp16 kernels over the two
            # fp16 terms of the activations beat the kernels that split them on the fly
            hi, lo = split_f32(x, ps)
            t = ternary_linear(hi, nw, scale, bias, residual, False, torch.float32)
            return ternary_linear(lo, nw, scale, None, t, relu, torch.float32)
    y = torch.empty(x.shape[:-1] + (nw.N,), dtype=out_dtype, device=x.device)
    ep = _epilogue(nw, scale, bias, residual, relu, out_dtype, y)
    lib = _lib()
    # shapes whose reduction pays to be cut across workgroups get a workspace for the partial sums, and rows of a
    # ragged length one for their copy padded to whole 64-index tiles
    wsb = pairs or (lib.tmq_ternary_linear_workspace_bytes(_capi.dtype_code(x), M, nw.K, nw.N)
                    if M > 16 and (M <= 32 or nw.K % 64) else 0)
    with _capi.on_device(x.device):
        if wsb:
            ws = torch.empty(wsb, dtype=torch.uint8, device=x.device)
            check(lib.tmq_ternary_linear_ws(ptr(x), _capi.dtype_code(x), M, nw.K, ptr(nw.buf), nw.N, ctypes.byref(ep), ptr(y),
                                            ptr(ws), wsb, stream_of(x)), "ternary_linear")
        else:
            check(lib.tmq_ternary_linear(ptr(x), _capi.dtype_code(x), M, nw.K, ptr(nw.buf), nw.N, ctypes.byref(ep),
                                         ptr(y), stream_of(x)), "ternary_linear")
    return y


class ActivationPlanes:
    """One to four fp16 activation rows in the operand form of the 8-bit GEMV (each value as four bf8 terms), made
    once by gemv8_prepare and multiplied with any number of layers by ternary_linear_planes."""

    def __init__(self, buf, rows, K, lead):
        self.buf, self.rows, self.K, self.lead = buf, rows, K, lead


def gemv8_planes_supported(rows: int, K: int) -> bool:
    """Whether gemv8_prepare / ternary_linear_planes take `rows` rows of K values (at most 4 rows, K a multiple of
    256 from 2048 to 16384, rows padded to 1 / 2 / 4 times K at most 16384)."""
    return _lib().tmq_gemv8_planes_bytes(int(rows), int(K)) > 0


def gemv8_prepare(x: torch.Tensor) -> ActivationPlanes:
    """The bf8 term planes of x (fp16 [..., K], at most four rows in all): one small launch; see ActivationPlanes."""
    _capi.require_gpu(x, "activations")
    if x.dtype != torch.float16:
        raise RuntimeError("gemv8_prepare: activations must be fp16")
    K = int(x.shape[-1])
    M = x.numel() // K if K else 0
    lib = _lib()
    nbytes = lib.tmq_gemv8_planes_bytes(M, K)
    if nbytes == 0:
        raise RuntimeError("gemv8_prepare: at most 4 rows of K = 2048 .. 16384 (a multiple of 256), rows x K <= 16384")
    buf = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    with _capi.on_device(x.device):
        check(lib.tmq_gemv8_prepare(ptr(x), M, K, ptr(buf), stream_of(x)), "gemv8_prepare")
    return ActivationPlanes(buf, M, K, tuple(x.shape[:-1]))


def ternary_linear_planes(planes: ActivationPlanes, nw: NativeWeights, scale=None, bias=None, residual=None, relu=False,
                          out_dtype=torch.float32) -> torch.Tensor:
    """ternary_linear on rows prepared by gemv8_prepare: same values, without the conversion every workgroup of the
    plain call repeats."""
    if planes.K != nw.K:
        raise RuntimeError(f"ternary_linear_planes: activations have {planes.K} features, weights expect {nw.K}")
    y = torch.empty(planes.lead + (nw.N,), dtype=out_dtype, device=planes.buf.device)
    ep = _epilogue(nw, scale, bias, residual, relu, out_dtype, y)
    with _capi.on_device(y.device):
        check(_lib().tmq_ternary_linear_planes(ptr(planes.buf), planes.rows, nw.K, ptr(nw.buf), nw.N, ctypes.byref(ep), ptr(y),
                                               stream_of(y)), "ternary_linear_planes")
    return y


def ternary_conv2d(x: torch.Tensor, nw: NativeWeights, stride=1, padding=0, dilation=1, scale=None, bias=None,
                   residual=None, relu=False, out_dtype=torch.float32) -> torch.Tensor:
    """Implicit-GEMM ternary convolution. x: fp16 [B, C, H, W] in channels_last memory (any other
    layout / fp32 is converted first); nw: NativeWeights built with conv_kernel=(ky, kx). Returns
    [B, N, Ho, Wo] in channels_last memory."""
    pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    (sy, sx), (py, px), (dy, dx) = pair(stride), pair(padding), pair(dilation)
    # padding may also be ((top, bottom), (left, right))
    (py, py_end), (px, px_end) = pair(py), pair(px)
    if not x.is_cuda or x.dim() != 4:
        raise RuntimeError("ternary_conv2d: expected a 4-D GPU tensor")
    if x.shape[1] != nw.C:
        raise RuntimeError(f"ternary_conv2d: input has {x.shape[1]} channels, weights expect {nw.C}")
    if x.dtype == torch.float32:
        x, scale = f32_to_f16_prescaled(x, scale, nw.N)
    if x.dtype != torch.float16 or not x.is_contiguous(memory_format=torch.channels_last):
        x = x.to(dtype=torch.float16, memory_format=torch.channels_last)
    B, C, H, W = x.shape
    shp = _capi.ConvShape(B, C, H, W, nw.N, nw.ky, nw.kx, sy, sx, py, px, dy, dx, py_end, px_end)
    ho, wo = ctypes.c_int32(0), ctypes.c_int32(0)
    lib = _lib()
    check(lib.tmq_conv2d_out_hw(ctypes.byref(shp), ctypes.byref(ho), ctypes.byref(wo)), "conv2d_out_hw")
    if ho.value <= 0 or wo.value <= 0:
        raise RuntimeError("ternary_conv2d: empty output")
    y = torch.empty((B, nw.N, ho.value, wo.value), dtype=out_dtype, device=x.device,
                    memory_format=torch.channels_last)
    ep = _epilogue(nw, scale, bias, residual, relu, out_dtype, y)
    if B == 0:
        return y
    with _capi.on_device(x.device):
        check(lib.tmq_ternary_conv2d(ptr(x), ctypes.byref(shp), ptr(nw.buf), ctypes.byref(ep), ptr(y), stream_of(x)),
              "ternary_conv2d")
    return y


def ternary_conv2d_into(out: torch.Tensor, x: torch.Tensor, nw: NativeWeights, stride=1, padding=0, dilation=1, scale=None,
                        bias=None, residual=None, relu=False, first=(0, 0)) -> torch.Tensor:
    """ternary_conv2d written straight into `out`, a strided view [B, N, h, w] of a channels_last tensor (fp16 or
    fp32, e.g. big[:, :, 1::2, 0::2]): output position (first[0] + i, first[1] + j) of the convolution goes to
    out[:, :, i, j]; positions of the convolution outside that h x w window are dropped. `residual`, when given, is a
    view with out's shape and strides. One launch, no temporary. x must already be fp16."""
    pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    (sy, sx), (py, px), (dy, dx) = pair(stride), pair(padding), pair(dilation)
    (py, py_end), (px, px_end) = pair(py), pair(px)
    if not x.is_cuda or x.dim() != 4 or out.dim() != 4 or out.device != x.device:
        raise RuntimeError("ternary_conv2d_into: expected 4-D GPU tensors on one device")
    if x.dtype != torch.float16:
        raise RuntimeError("ternary_conv2d_into: activations must be fp16")
    if x.shape[1] != nw.C:
        raise RuntimeError(f"ternary_conv2d_into: input has {x.shape[1]} channels, weights expect {nw.C}")
    if not x.is_contiguous(memory_format=torch.channels_last):
        x = x.contiguous(memory_format=torch.channels_last)
    B, C, H, W = x.shape
    N = nw.N
    sb_, sc_, sh_, sw_ = out.stride()
    if out.shape[0] != B or out.shape[1] != N or (N > 1 and sc_ != 1) or any(v % N for v in (sb_, sh_, sw_)):
        raise RuntimeError("ternary_conv2d_into: out must be a [B, N, h, w] view of a channels_last tensor with N channels")
    shp = _capi.ConvShape(B, C, H, W, N, nw.ky, nw.kx, sy, sx, py, px, dy, dx, py_end, px_end)
    ep = _epilogue(nw, scale, bias, residual, relu, out.dtype, out)
    view = _capi.OutputView(int(first[0]), int(first[1]), int(out.shape[2]), int(out.shape[3]), sb_ // N, sh_ // N, sw_ // N)
    if out.numel() == 0:
        return out
    with _capi.on_device(x.device):
        check(_lib().tmq_ternary_conv2d_view(ptr(x), ctypes.byref(shp), ptr(nw.buf), ctypes.byref(ep), ptr(out),
                                             ctypes.byref(view), stream_of(x)), "ternary_conv2d_view")
    return out


def ternary_conv2d_relu_maxpool(x: torch.Tensor, nw: NativeWeights, stride=1, padding=0, dilation=1, scale=None,
                                bias=None) -> torch.Tensor:
    """max_pool2d(relu(ternary_conv2d(x) * scale + bias), 3, 2, 1), the opening of a ResNet. Arguments as
    ternary_conv2d; the result is fp16 [B, N, Po, Pwo] in channels_last memory. Few-channel inputs with a short
    reduction (8, 16 or 32 channels, C * ky * kx <= 256, at most 64 output channels in groups of 8) take one
    kernel that never writes the convolution's output; everything else makes the two calls. Both give the same
    bits."""
    pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    (sy, sx), (py, px), (dy, dx) = pair(stride), pair(padding), pair(dilation)
    (py, py_end), (px, px_end) = pair(py), pair(px)
    if not x.is_cuda or x.dim() != 4:
        raise RuntimeError("ternary_conv2d_relu_maxpool: expected a 4-D GPU tensor")
    if x.shape[1] != nw.C:
        raise RuntimeError(f"ternary_conv2d_relu_maxpool: input has {x.shape[1]} channels, weights expect {nw.C}")
    if x.dtype == torch.float32:
        x, scale = f32_to_f16_prescaled(x, scale, nw.N)
    if x.dtype != torch.float16 or not x.is_contiguous(memory_format=torch.channels_last):
        x = x.to(dtype=torch.float16, memory_format=torch.channels_last)
    B, C, H, W = x.shape
    shp = _capi.ConvShape(B, C, H, W, nw.N, nw.ky, nw.kx, sy, sx, py, px, dy, dx, py_end, px_end)
    ho, wo = ctypes.c_int32(0), ctypes.c_int32(0)
    lib = _lib()
    check(lib.tmq_conv2d_out_hw(ctypes.byref(shp), ctypes.byref(ho), ctypes.byref(wo)), "conv2d_out_hw")
    if ho.value <= 0 or wo.value <= 0:
        raise RuntimeError("ternary_conv2d_relu_maxpool: empty output")
    y = torch.empty((B, nw.N, (ho.value - 1) // 2 + 1, (wo.value - 1) // 2 + 1), dtype=torch.float16, device=x.device,
                    memory_format=torch.channels_last)
    ep = _epilogue(nw, scale, bias, None, True, torch.float16, y)     # validates scale and bias
    if B == 0:
        return y
    with _capi.on_device(x.device):
        status = lib.tmq_ternary_conv2d_relu_maxpool(ptr(x), ctypes.byref(shp), ptr(nw.buf), ep.scale, ep.bias, ptr(y),
                                                     stream_of(x))
    if status == _capi.ERR_UNSUPPORTED:
        full = ternary_conv2d(x, nw, stride, padding, dilation, scale, bias, relu=True, out_dtype=torch.float16)
        return maxpool2d_nhwc(full, 3, 2, 1)
    check(status, "ternary_conv2d_relu_maxpool")
    return y


def ternary_conv2d_relu_maxpool_planar(x: torch.Tensor, nw: NativeWeights, stride=1, padding=0, dilation=1, scale=None,
                                       bias=None) -> torch.Tensor:
    """ternary_conv2d_relu_maxpool on the network's own input: x is NCHW fp16 [B, C <= 4, H, W] (W even), nw the weights of
    the convolution over 8-channel "super-pixels" (two neighbouring pixels x 4 channels) that stride, padding and dilation
    describe -- what nchw_to_nhwc4(x).view(B, H, W / 2, 8) would feed the other call, without that copy of the input.
    Same bits as the two-step form, which it falls back to where the one-kernel opening does not apply."""
    pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    (sy, sx), (py, px), (dy, dx) = pair(stride), pair(padding), pair(dilation)
    (py, py_end), (px, px_end) = pair(py), pair(px)
    if not x.is_cuda or x.dim() != 4 or x.shape[1] > 4 or x.shape[3] % 2 or nw.C != 8:
        raise RuntimeError("ternary_conv2d_relu_maxpool_planar: expected an NCHW GPU tensor of at most 4 channels and even "
                           "width, and weights over 8-channel super-pixels")

    def two_step():
        B, C, H, W = x.shape
        xs = nchw_to_nhwc4(x).view(B, H, W // 2, 8).permute(0, 3, 1, 2)      # [B, 8, H, W / 2], channels_last memory
        return ternary_conv2d_relu_maxpool(xs, nw, stride, padding, dilation, scale, bias)
    if x.dtype != torch.float16:
        return two_step()
    x = x.contiguous()
    B, C, H, W = x.shape
    shp = _capi.ConvShape(B, 8, H, W // 2, nw.N, nw.ky, nw.kx, sy, sx, py, px, dy, dx, py_end, px_end)
    ho, wo = ctypes.c_int32(0), ctypes.c_int32(0)
    lib = _lib()
    check(lib.tmq_conv2d_out_hw(ctypes.byref(shp), ctypes.byref(ho), ctypes.byref(wo)), "conv2d_out_hw")
    if ho.value <= 0 or wo.value <= 0:
        raise RuntimeError("ternary_conv2d_relu_maxpool_planar: empty output")
    y = torch.empty((B, nw.N, (ho.value - 1) // 2 + 1, (wo.value - 1) // 2 + 1), dtype=torch.float16, device=x.device,
                    memory_format=torch.channels_last)
    ep = _epilogue(nw, scale, bias, None, True, torch.float16, y)     # validates scale and bias
    if B == 0:
        return y
    with _capi.on_device(x.device):
        status = lib.tmq_ternary_conv2d_relu_maxpool_planar(ptr(x), C, ctypes.byref(shp), ptr(nw.buf), ep.scale, ep.bias, ptr(y),
                                                            stream_of(x))
    if status == _capi.ERR_UNSUPPORTED:
        return two_step()
    check(status, "ternary_conv2d_relu_maxpool_planar")
    return y


class _Channels:
    """What _epilogue needs to know about a depthwise layer: its channel count."""
    def __init__(self, n):
        self.N = n


def ternary_dwconv2d(x: torch.Tensor, words: torch.Tensor, kernel, stride=1, padding=0, dilation=1, scale=None,
                     bias=None, residual=None, relu=False, out_dtype=torch.float32) -> torch.Tensor:
    """Depthwise ternary convolution (groups == channels) straight from the compact words of a
    [C, 1, ky, kx] weight tensor (int32 [1, ky, kx, ceil(C/16)] as compactify_ternary returns them).
    x: fp16 [B, C, H, W] in channels_last memory (anything else is converted first); returns
    [B, C, Ho, Wo] in channels_last memory."""
    pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    (ky, kx), (sy, sx), (py, px), (dy, dx) = pair(kernel), pair(stride), pair(padding), pair(dilation)
    (py, py_end), (px, px_end) = pair(py), pair(px)
    if not x.is_cuda or x.dim() != 4:
        raise RuntimeError("ternary_dwconv2d: expected a 4-D GPU tensor")
    B, C, H, W = x.shape
    _capi.require_gpu(words, "words")
    if words.dtype != torch.int32 or words.numel() != ky * kx * ((C + 15) // 16):
        raise RuntimeError("ternary_dwconv2d: expected the int32 compact words of a [C, 1, ky, kx] weight tensor")
    if x.dtype == torch.float32:
        x, scale = f32_to_f16_prescaled(x, scale, C)
    if x.dtype != torch.float16 or not x.is_contiguous(memory_format=torch.channels_last):
        x = x.to(dtype=torch.float16, memory_format=torch.channels_last)
    words = words.contiguous()
    shp = _capi.ConvShape(B, C, H, W, C, ky, kx, sy, sx, py, px, dy, dx, py_end, px_end)
    ho, wo = ctypes.c_int32(0), ctypes.c_int32(0)
    lib = _lib()
    check(lib.tmq_conv2d_out_hw(ctypes.byref(shp), ctypes.byref(ho), ctypes.byref(wo)), "conv2d_out_hw")
    if ho.value <= 0 or wo.value <= 0:
        raise RuntimeError("ternary_dwconv2d: empty output")
    y = torch.empty((B, C, ho.value, wo.value), dtype=out_dtype, device=x.device, memory_format=torch.channels_last)
    ep = _epilogue(_Channels(C), scale, bias, residual, relu, out_dtype, y)
    if B == 0:
        return y
    with _capi.on_device(x.device):
        check(lib.tmq_ternary_dwconv2d(ptr(x), ctypes.byref(shp), ptr(words), ctypes.byref(ep), ptr(y), stream_of(x)),
              "ternary_dwconv2d")
    return y


def ternary_dwconv_cuda(input: torch.Tensor, weights: torch.Tensor, kx: int, ky: int, channels: int) -> torch.Tensor:
    """The reference's binding (tmq/tmq_cuda.cu:607-642, caller tmq/tmq.py:849-853): input is the
    unfolded tensor [..., positions, ky * kx * channels] (tap-major, channel fastest), weights the
    compact words of the [channels, 1, ky, kx] kernel; returns [..., positions, channels] fp32 with
    out[p][c] = sum_t input[p][t * channels + c] * T[c][t]."""
    if not input.is_cuda or not weights.is_cuda:
        raise RuntimeError("ternary_dwconv_cuda: expected tensors on the GPU")
    if input.dtype not in (torch.float32, torch.float16):
        raise RuntimeError("ternary_dwconv_cuda: expected fp32 (or fp16) input")
    taps = int(kx) * int(ky)
    if weights.dtype != torch.int32 or weights.numel() != taps * ((channels + 15) // 16):
        raise RuntimeError("ternary_dwconv_cuda: compact weights do not match kernel size and channels")
    if input.dim() < 2 or input.shape[-1] != taps * channels:
        raise RuntimeError("ternary_dwconv_cuda: the last dimension must be ky * kx * channels")
    x = input.contiguous()
    P = x.numel() // (taps * channels)
    y = torch.empty(tuple(input.shape[:-1]) + (channels,), dtype=torch.float32, device=x.device)
    with _capi.on_device(x.device):
        check(_lib().tmq_ternary_dwconv_patches(ptr(x), _capi.dtype_code(x), P, taps, channels, ptr(weights.contiguous()),
                                                ptr(y), stream_of(x)), "ternary_dwconv_cuda")
    return y


def ternary_dwconvtrans2d(x: torch.Tensor, words: torch.Tensor, kernel, stride=1, padding=0, output_padding=0, dilation=1,
                          scale=None, bias=None, residual=None, relu=False, out_dtype=torch.float32) -> torch.Tensor:
    """Depthwise transposed ternary convolution (groups == channels, one filter per channel) straight
    from the compact words of a [C, 1, ky, kx] weight tensor, gathered per output position -- no
    columns, no fold. x: fp16 [B, C, H, W] in channels_last memory (anything else is converted first);
    returns [B, C, Ho, Wo] in channels_last memory, extents by nn.ConvTranspose2d's formula."""
    pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    (ky, kx), (sy, sx), (py, px), (oy, ox), (dy, dx) = (pair(kernel), pair(stride), pair(padding), pair(output_padding),
                                                       pair(dilation))
    if not x.is_cuda or x.dim() != 4:
        raise RuntimeError("ternary_dwconvtrans2d: expected a 4-D GPU tensor")
    B, C, H, W = x.shape
    _capi.require_gpu(words, "words")
    if words.dtype != torch.int32 or words.numel() != ky * kx * ((C + 15) // 16):
        raise RuntimeError("ternary_dwconvtrans2d: expected the int32 compact words of a [C, 1, ky, kx] weight tensor")
    if x.dtype == torch.float32:
        x, scale = f32_to_f16_prescaled(x, scale, C)
    if x.dtype != torch.float16 or not x.is_contiguous(memory_format=torch.channels_last):
        x = x.to(dtype=torch.float16, memory_format=torch.channels_last)
    words = words.contiguous()
    shp = _capi.ConvShape(B, C, H, W, C, ky, kx, sy, sx, py, px, dy, dx, py, px)
    ho, wo = ctypes.c_int32(0), ctypes.c_int32(0)
    lib = _lib()
    check(lib.tmq_convtranspose2d_out_hw(ctypes.byref(shp), oy, ox, ctypes.byref(ho), ctypes.byref(wo)),
          "convtranspose2d_out_hw")
    y = torch.empty((B, C, ho.value, wo.value), dtype=out_dtype, device=x.device, memory_format=torch.channels_last)
    ep = _epilogue(_Channels(C), scale, bias, residual, relu, out_dtype, y)
    if B == 0:
        return y
    with _capi.on_device(x.device):
        check(lib.tmq_ternary_dwconvtrans2d(ptr(x), ctypes.byref(shp), oy, ox, ptr(words), ctypes.byref(ep), ptr(y),
                                            stream_of(x)), "ternary_dwconvtrans2d")
    return y


def ternary_dwconvtrans_cuda(input: torch.Tensor, weights: torch.Tensor, kx: int, ky: int) -> torch.Tensor:
    """The reference's binding (tmq/tmq_cuda.cu:645-686, caller tmq/tmq.py:1026-1029): input fp32
    [P, C], [B, P, C] or [B, 1, P, C]; weights the compact words of the [C, 1, ky, kx] kernel, shaped
    [1, *, *, ceil(C/16)]; returns fp32 [C*ky*kx, P], [B, C*ky*kx, P] or [B, 1, C*ky*kx, P] with
    out[c*taps + t][p] = input[p][c] * T[c][t], ready for F.fold. Every batch entry is computed and a
    4-D input gives the 4-D output (the reference's host fills entry 0 only and overwrites the 4-D
    result with a 2-D one, tmq/tmq_cuda.cu:677-682)."""
    if not input.is_cuda or not weights.is_cuda:
        raise RuntimeError("ternary_dwconvtrans_cuda: expected tensors on the GPU")
    if input.dtype != torch.float32:
        raise RuntimeError("ternary_dwconvtrans_cuda: expected fp32 input")
    if input.dim() not in (2, 3, 4) or (input.dim() == 4 and input.shape[1] != 1):
        raise RuntimeError("ternary_dwconvtrans_cuda: expected [P, C], [B, P, C] or [B, 1, P, C]")
    taps = int(kx) * int(ky)
    P, C = int(input.shape[-2]), int(input.shape[-1])
    B = int(input.shape[0]) if input.dim() > 2 else 1
    if weights.dtype != torch.int32 or weights.dim() != 4 or weights.shape[0] != 1 or \
            weights.shape[1] * weights.shape[2] != taps or weights.shape[3] != (C + 15) // 16:
        raise RuntimeError("ternary_dwconvtrans_cuda: compact weights do not match kernel size and channels")
    x = input.contiguous()
    y = torch.empty(tuple(input.shape[:-2]) + (C * taps, P), dtype=torch.float32, device=x.device)
    if y.numel():
        with _capi.on_device(x.device):
            check(_lib().tmq_ternary_dwconvtrans_cols(ptr(x), B, P, taps, C, ptr(weights.contiguous()), ptr(y), stream_of(x)),
                  "ternary_dwconvtrans_cuda")
    return y


def maxpool2d_nhwc(x: torch.Tensor, kernel, stride=None, padding=0) -> torch.Tensor:
    """nn.MaxPool2d(kernel, stride, padding) on an fp16 [B, C, H, W] tensor in channels_last memory
    (anything else is converted first); returns [B, C, Ho, Wo] fp16 in channels_last memory."""
    pair = lambda v: tuple(v) if isinstance(v, (tuple, list)) else (v, v)
    (ky, kx), (py, px) = pair(kernel), pair(padding)
    sy, sx = pair(stride) if stride is not None else (ky, kx)
    if not x.is_cuda or x.dim() != 4:
        raise RuntimeError("maxpool2d_nhwc: expected a 4-D GPU tensor")
    if x.dtype != torch.float16 or not x.is_contiguous(memory_format=torch.channels_last):
        x = x.to(dtype=torch.float16, memory_format=torch.channels_last)
    B, C, H, W = x.shape
    if 2 * py > ky or 2 * px > kx or H + 2 * py < ky or W + 2 * px < kx:
        raise RuntimeError("maxpool2d_nhwc: pad should be at most half of the kernel size and the window must fit")
    ho, wo = (H + 2 * py - ky) // sy + 1, (W + 2 * px - kx) // sx + 1
    y = torch.empty((B, C, ho, wo), dtype=torch.float16, device=x.device, memory_format=torch.channels_last)
    if y.numel() == 0:
        return y
    with _capi.on_device(x.device):
        check(_lib().tmq_maxpool2d_nhwc(ptr(x), B, C, H, W, ky, kx, sy, sx, py, px, ptr(y), stream_of(x)), "maxpool2d_nhwc")
    return y


def avgpool_global_nhwc(x: torch.Tensor, out_dtype=torch.float16) -> torch.Tensor:
    """Mean over H x W of an fp16 [B, C, H, W] tensor in channels_last memory -> [B, C]."""
    if not x.is_cuda or x.dim() != 4:
        raise RuntimeError("avgpool_global_nhwc: expected a 4-D GPU tensor")
    if x.dtype != torch.float16 or not x.is_contiguous(memory_format=torch.channels_last):
        x = x.to(dtype=torch.float16, memory_format=torch.channels_last)
    B, C, H, W = x.shape
    y = torch.empty((B, C), dtype=out_dtype, device=x.device)
    if y.numel() == 0:
        return y
    with _capi.on_device(x.device):
        check(_lib().tmq_avgpool_global_nhwc(ptr(x), B, H * W, C, ptr(y), _capi.dtype_code(y), stream_of(x)),
              "avgpool_global_nhwc")
    return y


def avgpool_linear(x: torch.Tensor, nw: NativeWeights, scale=None, bias=None, relu=False, out_dtype=torch.float32) -> torch.Tensor:
    """ternary_linear(avgpool_global_nhwc(x), nw, ...), a network's head: one launch when the feature map has at most 512
    channels in whole groups of 8, else the two calls. x: fp16 [B, C, H, W] in channels_last memory."""
    if not x.is_cuda or x.dim() != 4:
        raise RuntimeError("avgpool_linear: expected a 4-D GPU tensor")
    if x.dtype != torch.float16 or not x.is_contiguous(memory_format=torch.channels_last):
        x = x.to(dtype=torch.float16, memory_format=torch.channels_last)
    B, C, H, W = x.shape
    if C != nw.K:
        raise RuntimeError(f"avgpool_linear: feature map has {C} channels, weights expect {nw.K}")
    y = torch.empty((B, nw.N), dtype=out_dtype, device=x.device)
    ep = _epilogue(nw, scale, bias, None, relu, out_dtype, y)
    if y.numel() == 0:
        return y
    with _capi.on_device(x.device):
        status = _lib().tmq_avgpool_linear(ptr(x), B, H * W, C, ptr(nw.buf), nw.N, ctypes.byref(ep), ptr(y), stream_of(x))
    if status == _capi.ERR_UNSUPPORTED:
        return ternary_linear(avgpool_global_nhwc(x), nw, scale=scale, bias=bias, relu=relu, out_dtype=out_dtype)
    check(status, "avgpool_linear")
    return y


def nchw_to_nhwc4(x: torch.Tensor) -> torch.Tensor:
    """Contiguous NCHW network input (fp16 or fp32, at most 4 channels, W a multiple of 4) -> fp16
    [B, H, W, 4] with the missing channels zero."""
    if not x.is_cuda or x.dim() != 4 or x.dtype not in (torch.float16, torch.float32):
        raise RuntimeError("nchw_to_nhwc4: expected a 4-D fp16 / fp32 GPU tensor")
    x = x.contiguous()
    B, C, H, W = x.shape
    if C > 4 or W % 4:
        raise RuntimeError("nchw_to_nhwc4: at most 4 channels, width a multiple of 4")
    y = torch.empty((B, H, W, 4), dtype=torch.float16, device=x.device)
    if y.numel() == 0:
        return y
    with _capi.on_device(x.device):
        check(_lib().tmq_nchw_to_nhwc4(ptr(x), _capi.dtype_code(x), B, C, H, W, ptr(y), stream_of(x)), "nchw_to_nhwc4")
    return y


def _check_mm_args(lhs, weights, columns, name):
    # tmq/tmq_cuda.cu:480-490, 566-575
    if not lhs.is_cuda or not weights.is_cuda:
        raise RuntimeError(f"{name}: expected tensors on the GPU")
    if lhs.dtype not in (torch.float32, torch.float16):
        raise RuntimeError(f"{name}: expected fp32 (or fp16) activations")
    if weights.dim() != 2 or weights.dtype != torch.int32:
        raise RuntimeError(f"{name}: expected 2-D int32 compact weights")
    if not (weights.shape[1] * 16 >= columns and weights.shape[1] * 16 < columns + 16):
        raise RuntimeError(f"{name}: compact weight width does not match the number of columns")


def ternary_mmm_cuda(lhs: torch.Tensor, weights: torch.Tensor, columns: int) -> torch.Tensor:
    """Ternary weights matrix/matrix multiplication (tmq/tmq_cuda.cu:478-549): lhs of rank 1..4
    (rank 4 needs a leading 1), weights int32 [K][ceil(columns/16)]; returns lhs.dtype-agnostic fp32
    of shape lhs.shape[:-1] + (columns,) (rank 1 gives [1, columns], like the reference)."""
    _check_mm_args(lhs, weights, columns, "ternary_mmm_cuda")
    if lhs.dim() < 1 or lhs.dim() > 4:
        raise RuntimeError("ternary_mmm_cuda: expected an lhs of rank 1..4")
    if lhs.dim() == 4 and lhs.shape[0] != 1:
        raise RuntimeError("ternary_mmm_cuda: a rank-4 lhs needs a leading dimension of 1")
    x = lhs.contiguous()
    if x.dim() == 1:
        x = x.view(1, -1)
    return ternary_linear(x, native_weights(weights, columns))


def ternary_mvm_cuda(vector: torch.Tensor, weights: torch.Tensor, columns: int) -> torch.Tensor:
    """Ternary weights matrix/vector multiplication (tmq/tmq_cuda.cu:563-603); every leading
    dimension of `vector` must be 1, the result keeps the rank."""
    _check_mm_args(vector, weights, columns, "ternary_mvm_cuda")
    if vector.dim() < 1 or vector.dim() > 4 or any(s != 1 for s in vector.shape[:-1]):
        raise RuntimeError("ternary_mvm_cuda: expected a single vector (leading dimensions of 1)")
    return ternary_linear(vector.contiguous(), native_weights(weights, columns))


# ---- the PyTorch extension with the reference's binding names --------------------------------------------
# tmq_hip_ext (csrc/torch_ext.cpp, `make -C tmq_amd/csrc ext`) exposes the same twelve names as the
# reference's tmq_cuda / tmq_native modules over the same C ABI; tmq.py calls through it when it has
# been built and through the ctypes functions above otherwise. Either way the kernels are libtmq_hip's.
try:
    from . import tmq_hip_ext as ext
except ImportError:
    ext = None
