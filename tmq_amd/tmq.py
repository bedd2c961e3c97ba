"""TMQ's Python API on the MI355X-native kernels.

Same public surface as the reference's tmq/tmq.py -- QuantMode, TensorType,
QuantizationScheduleBuilder, QuantizationControl, SoftStep, SoftStepDerivative, TMQLayer, Linear,
Conv2d, ConvTranspose2d, quantize_weights, quantize_model, compressed_state_dict,
prepare_compressed_load, load_compressed_state_dict, expand_compact_layers -- with the same
argument meaning and error behaviour, so user code switches by changing the import.

What differs underneath:
  * every tensor-valued computation of the hot path (soft staircase forward / backward,
    quantization loss and its gradient, clamp, ternarisation, 2-bit packing, compact inference)
    runs in libtmq_hip on the GPU; there is no CPU implementation of that math here, and weights
    must live on the GPU (a clear error is raised otherwise);
  * QuantizationControl.quantization_loss() and .clamp() are single multi-tensor launches over
    all registered layers instead of per-layer Python loops, and clamp works in place;
  * compact inference takes any batch shape and runs convolutions as implicit GEMM.
Host-only logic (the hardness / penalty schedule, model surgery, state-dict metadata) is plain
Python as in the reference.
"""
import fnmatch
from enum import Enum

import torch
from torch import nn
from torch.autograd.function import Function

from . import ops
from ._capi import load as _load_native

# the reference's binding names: the C++ extension when built, else the ctypes binding (same C ABI)
_b = ops.ext if ops.ext is not None else ops

# The reference exposes these two flags (tmq/tmq.py:28-46). Here the single native library is
# mandatory: importing this module without it raises instead of degrading.
_load_native()
CUDA_EXT_AVAILABLE = True
NATIVE_EXT_AVAILABLE = True

_compact_out = torch.float32


def set_compact_output_dtype(dtype):
    """Output type of the compact (2-bit) forward of Linear / Conv2d: torch.float32 (the reference's
    behaviour, default) or torch.float16. With fp16 the convolutions hand fp16 channels_last tensors to
    whatever follows (BatchNorm, ReLU, pooling, the next compact layer, which then needs no input
    conversion), halving the activation traffic of an inference model. Returns the previous setting."""
    global _compact_out
    if dtype not in (torch.float32, torch.float16):
        raise ValueError("compact output dtype must be torch.float32 or torch.float16")
    prev, _compact_out = _compact_out, dtype
    return prev


class QuantMode(Enum):
    """Quantization modes (tmq/tmq.py:49-63); only TERNARY is implemented, as in the reference."""
    NONE = 0
    TERNARY = 1
    TWO_BIT = 2
    THREE_BIT = 3
    FOUR_BIT = 4
    FIVE_BIT = 5
    SIX_BIT = 6
    EIGHT_BIT = 8


class TensorType(Enum):
    """Storage type of a TMQ layer's weight tensor (tmq/tmq.py:65-72)."""
    FLOAT_32BIT = 0
    FLOAT_16BIT = 1
    COMPACT_TERNARY_32BIT = 2
    COMPRESSED_TERNARY_32BIT = 3


class QuantizationScheduleBuilder:
    """tmq/tmq.py:75-82"""

    @staticmethod
    def default_schedule(max_epochs: int):
        assert max_epochs >= 50, "Need at least 50 epochs for a default schedule"
        return tuple(int(max_epochs * f) for f in (0.3, 0.8, 0.875, 0.93)) + (max_epochs,)


def _require_gpu_weight(t, what):
    if not t.is_cuda:
        raise RuntimeError(f"tmq_amd: {what} needs its weights on the GPU (no CPU implementation is provided); "
                           "move the model with .to('cuda') first")


class QuantizationControl:
    """Controller for quantization-aware training (tmq/tmq.py:85-310): owns the registry of TMQ
    layers and the hardness (`digamma`) / penalty (`qpenalty`) schedule.

    epoch_knots: (reach digamma 3, reach digamma max and start the penalty ramp, reach the maximum
    penalty, stop cycling, total epochs)."""

    _WARMUP = 7          # tmq/tmq.py:117
    _CYCLE = 15          # tmq/tmq.py:141

    def __init__(self, epoch_knots=None, digamma_range=(0.1, 6), qpenalty_range=None, quant_mode=QuantMode.TERNARY,
                 post_scale=False, init_range=None, device="cpu"):
        assert epoch_knots is None or len(epoch_knots) == 5
        assert len(digamma_range) == 2, "Need to supply a start/end value for the digamma parameter of the softstep function"
        assert digamma_range[0] >= 0.05, "Initial digamma value must be >= 0.05"
        assert digamma_range[0] <= 1, "Initial digamma value must be <= 1"
        assert digamma_range[1] <= 20.0, "Final digamma value must be <= 20"
        assert digamma_range[1] >= 3, "Final digamma value must be >= 3"
        assert digamma_range[0] <= digamma_range[1], "Please supply a valid range for digamma"
        self._warmup_epochs = self._WARMUP
        if epoch_knots is not None:
            assert epoch_knots[0] >= self._warmup_epochs + 5, \
                "At least %d epochs required to reach halfway point" % (self._warmup_epochs + 5)
            self.max_epochs = epoch_knots[4]
        else:
            self.max_epochs = 0
        self.quantization = quant_mode
        self.epoch_knots = epoch_knots
        self.post_scale = post_scale
        self.digamma_start = max(0.05, digamma_range[0])
        self.digamma_end = max(3, digamma_range[1])
        self.digamma = self.digamma_start
        self.qpenalty = qpenalty_range[0] if qpenalty_range is not None else 0
        self.qpenalty_sharpness = 5.0
        self.inference_mode = self.max_epochs == 0
        self.device = device
        self._registry = {}
        self._last_cycle = -1
        self._digamma_cycle_start = 0
        self._digamma_cycle_end = 0
        self._cycle_len = self._CYCLE
        if quant_mode == QuantMode.TERNARY:
            self.clamp_values = (-1., 1.)
        else:
            bits = int(quant_mode.value)
            self.clamp_values = (-2 ** bits, (2 ** bits) - 1)
        self.init_range = init_range if init_range is not None else self.clamp_values
        if qpenalty_range is not None:
            assert len(qpenalty_range) == 2, "Quantization penalty needs to supply a range"
            self.qpenalty_range = qpenalty_range
        else:
            self.qpenalty_range = (0, 0)
        self._table = None            # cached multi-tensor segment table over the registered weights
        self._step = None             # soft weights of the current forward pass (_StepState)
        self._loss_wanted = False     # set by the first quantization_loss(): later passes fuse the loss

    # ---- schedule (host scalars only) -----------------------------------------------------------
    @staticmethod
    def _mix(lo_epoch, hi_epoch, epoch, start, end):
        t = min(1, max(0, (epoch - lo_epoch) / (hi_epoch - lo_epoch)))
        return t * end + (1 - t) * start

    def _segment(self, epoch):
        """Index of the knot interval an epoch falls into (0..4), tmq/tmq.py:176-181."""
        kn = self.epoch_knots
        if epoch >= kn[3]:
            return 4
        if epoch < kn[0]:
            return 0
        if epoch < kn[1]:
            return 1
        return 2 if epoch < kn[2] else 3

    def _ramp(self, seg, epoch):
        """The un-cycled hardness ramp: start -> 3 over [warm-up, knot 0], 3 -> end over
        [knot 0, knot 1], end afterwards (tmq/tmq.py:183-190)."""
        if seg >= 2:
            return self.digamma_end
        if seg == 0:
            return self._mix(self._warmup_epochs, self.epoch_knots[0], epoch, self.digamma_start, 3.0)
        return self._mix(self.epoch_knots[0], self.epoch_knots[1], epoch, 3.0, self.digamma_end)

    def step(self, epoch):
        """Advance the schedule; call once before every epoch, in order (the saw-tooth keeps state).

        Behaviour of tmq/tmq.py:160-240: nothing changes through the warm-up; from knot 3 on the
        hardness and the penalty sit at their final values; in between the hardness follows the
        ramp, except that every 15 epochs it restarts at 0.45 x the ramp (never below the start
        value) and climbs linearly to the ramp value 15 epochs ahead. The penalty ramps linearly
        between knots 2 and 3."""
        if self.epoch_knots is None:
            return
        if epoch >= self.epoch_knots[3]:
            self.qpenalty = self.qpenalty_range[1]
            self.digamma = self.digamma_end
            return
        if epoch <= self._warmup_epochs:
            return
        seg = self._segment(epoch)
        first_window = self._warmup_epochs + self._cycle_len
        in_cycle = self._last_cycle != -1
        if seg < 4 or in_cycle:
            ramp_now = self._ramp(seg, epoch)
            may_restart = not in_cycle and seg < 4 and (seg != 0 or epoch >= first_window)
            if may_restart:
                ahead = self._segment(epoch + self._cycle_len)
                if ahead < 4:
                    self._digamma_cycle_start = max(self.digamma_start, ramp_now * 0.45)
                    self._digamma_cycle_end = self._ramp(ahead, epoch + self._cycle_len)
                    self._last_cycle = epoch
                    self.digamma = self._digamma_cycle_start
            elif epoch < first_window:
                self.digamma = ramp_now
            elif epoch <= self._last_cycle + self._cycle_len:
                self.digamma = self._mix(self._last_cycle, self._last_cycle + self._cycle_len, epoch,
                                         self._digamma_cycle_start, self._digamma_cycle_end)
            else:
                self._last_cycle = -1
        else:
            self.digamma = self._ramp(seg, epoch)
        if seg >= 2:
            self.qpenalty = self._mix(self.epoch_knots[2], self.epoch_knots[3], epoch, self.qpenalty_range[0],
                                      self.qpenalty_range[1])

    # ---- registry -----------------------------------------------------------------------------------
    def inference(self):
        """Run all TMQ layers in inference mode (tmq/tmq.py:243-249)."""
        self.inference_mode = True

    def register_node(self, name, node):
        self._registry[name] = node
        self._table = None
        self._step = None

    def collect_grad_norms(self):
        return {name: node.weight.grad.norm() for name, node in self._registry.items()
                if node.weight.grad is not None}

    def _weights(self):
        return [node.weight for node in self._registry.values()]

    def _segment_table(self):
        """Multi-tensor table over the weights of every registered layer; rebuilt whenever a weight
        tensor has been reallocated."""
        ws = [w.data for w in self._weights()]
        for w in ws:
            _require_gpu_weight(w, "QuantizationControl")
            if w.dtype != torch.float32:
                raise ValueError("Expected either a float16 or a float32 tensor as input/output")
        key = tuple((w.data_ptr(), w.numel()) for w in ws)
        if self._table is None or self._table[0] != key:
            ws = [w if w.is_contiguous() else w.contiguous() for w in ws]
            self._table = (key, ops.SegmentTable(ws), ws)
        return self._table

    # ---- tensor work: one launch for all layers ------------------------------------------------------
    def clamp(self, slack=0):
        """Clamp the weights of all registered layers into the quantization range (+- slack), in
        place, in one launch (tmq/tmq.py:263-272 with 691-696 / 874-879)."""
        if not self._registry:
            return
        lo, hi = self.clamp_values[0] - slack, self.clamp_values[1] + slack
        _, table, _ = self._segment_table()
        ops.clamp_multi_(table, lo, hi)
        self._step = None

    def quantize(self):
        """Hard-quantize every registered layer: w <- round(SoftStep.map(w)) (tmq/tmq.py:284-295)."""
        for node in self._registry.values():
            w = node.weight.data
            _require_gpu_weight(w, "QuantizationControl.quantize")
            node.weight.data = ops.ternarize_(w.contiguous().clone(), self.digamma)
        self._step = None

    def quantization_loss(self, penalty=None):
        """Sum over layers of mean(SoftStepDerivative(w, sharpness, p)) (tmq/tmq.py:298-310). When the
        model's forward pass of this step has already produced it (same weights, same penalty), that
        value is returned and its gradient joins the soft-step backward in one launch; otherwise one
        multi-tensor launch forward, one backward. Returns None when no layer is registered."""
        if not self._registry:
            return None
        p = float(penalty if penalty is not None else self.qpenalty)
        self._loss_wanted = True
        st = self._step
        if (st is not None and st.loss is not None and not st.spent[0] and st.strength == p and st.sharpness == float(self.qpenalty_sharpness)
                and st.grad_mode == torch.is_grad_enabled() and st.covers(self._registry.values())):
            return st.loss
        return _QuantizationLossAll.apply(self, p, float(self.qpenalty_sharpness), *self._weights())

    # ---- soft weights of a forward pass: one launch for all layers ------------------------------------
    def _soft_weight_of(self, node):
        """S(weight) of a registered layer for the forward pass that is under way. The first layer that
        asks triggers one multi-tensor launch for every registered fp32 layer (and, once
        quantization_loss() has been used, for the loss as well); each layer's result is handed out
        once per pass, and a changed weight tensor, hardness or autograd mode starts a new pass.
        Returns None for a layer this controller cannot serve (then SoftStep.apply does it)."""
        st = self._step
        if st is not None and not st.spent[0] and id(node) in st.unserved:
            return None                    # no relaunch for the served layers on account of this one
        i = st.index.get(id(node)) if st is not None else None
        w = node.weight
        if (i is None or st.spent[0] or st.used[i] or st.versions[i] != w._version or st.ptrs[i] != w.data_ptr()
                or st.digamma != self.digamma or st.grad_mode != torch.is_grad_enabled()):
            st = self._step = _StepState.run(self)
            i = st.index.get(id(node)) if st is not None else None
            if i is None:
                return None
        st.used[i] = True
        return st.ys[i]


class _StepState:
    """Outputs of one multi-tensor soft-step forward launch and what they were computed from."""

    __slots__ = ("index", "nodes", "ptrs", "versions", "used", "ys", "loss", "digamma", "sharpness", "strength", "grad_mode",
                 "unserved", "spent")

    @classmethod
    def run(cls, ctrl):
        nodes, unserved, dev = [], set(), None
        for node in ctrl._registry.values():
            w = getattr(node, "weight", None)
            if w is None or node.compact or not w.is_cuda or w.dtype != torch.float32 or (dev is not None and w.device != dev):
                unserved.add(id(node))     # these go through SoftStep.apply on their own
                continue
            dev = w.device
            nodes.append(node)
        if not nodes:
            return None
        st = cls()
        st.nodes = nodes
        st.unserved = unserved
        # spent[0] is set by the autograd node's backward: the graph behind `ys` is freed then, so a layer that
        # did not take its result in that pass (a branch the forward skipped) must not be handed it in a later
        # one. A one-element list, so that the node holds the flag and not the state (no reference cycle
        # through `ys`, whose buffers are released by reference count).
        st.spent = [False]
        st.index = {id(n): i for i, n in enumerate(nodes)}
        weights = [n.weight for n in nodes]
        st.ptrs = [w.data_ptr() for w in weights]
        st.versions = [w._version for w in weights]
        st.used = [False] * len(nodes)
        st.digamma, st.sharpness, st.strength = ctrl.digamma, float(ctrl.qpenalty_sharpness), float(ctrl.qpenalty)
        st.grad_mode = torch.is_grad_enabled()
        want_loss = ctrl._loss_wanted
        outs = _SoftStepAll.apply(st.spent, st.digamma, want_loss, st.sharpness, st.strength, *weights)
        st.ys = outs[:len(nodes)]
        st.loss = outs[len(nodes)] if want_loss else None
        return st

    def covers(self, registered):
        """True when every registered layer took part and none of their weights changed since."""
        registered = list(registered)
        if len(registered) != len(self.nodes):
            return False
        for n, p, v in zip(self.nodes, self.ptrs, self.versions):
            w = n.weight
            if w.data_ptr() != p or w._version != v:
                return False
        return all(a is b for a, b in zip(registered, self.nodes))


class _SoftStepAll(Function):
    """(y_1 .. y_L [, loss]) = (S(w_1) .. S(w_L) [, sum_l mean q(w_l)]) as ONE autograd node: the forward
    is one multi-tensor launch and, because autograd runs a node only when the gradients of all its
    outputs are there, so is the backward, dw_l = g_l S'(w_l) + (g_loss / n_l) Q'(w_l) -- the two terms
    the reference computes in SoftStep.backward and SoftStepDerivative.backward per layer and lets autograd
    add (tmq/tmq.py:422-438, 475-493)."""

    @staticmethod
    def forward(ctx, spent, digamma, want_loss, sharpness, strength, *weights):
        ctx.args = (digamma, want_loss, sharpness, strength)
        ctx.spent = spent
        ctx.save_for_backward(*weights)
        ctx.set_materialize_grads(False)
        ys, loss = _b.softstep_fwd_all([w.data for w in weights], digamma, want_loss, sharpness, strength)
        return (*ys, loss) if want_loss else tuple(ys)

    @staticmethod
    def backward(ctx, *grads):
        digamma, want_loss, sharpness, strength = ctx.args
        ctx.spent[0] = True
        weights = ctx.saved_tensors
        L = len(weights)
        upstream = grads[L] if want_loss else None
        need = ctx.needs_input_grad[5:]
        live = [i for i in range(L) if need[i] and (grads[i] is not None or upstream is not None)]
        out = [None] * L
        if live:
            dws = _b.softstep_bwd_all([weights[i].data for i in live], [grads[i] for i in live], upstream, digamma,
                                      sharpness, strength)
            for i, dw in zip(live, dws):
                out[i] = dw
        return (None, None, None, None, None) + tuple(out)


class _QuantizationLossAll(Function):
    """total = sum_l mean_i q(w_l[i]); d total / d w_l = (g / n_l) * Q'(w_l) (tmq/tmq.py:456-493,
    698-699) for every registered layer at once, when the loss is asked for outside a forward pass."""

    @staticmethod
    def forward(ctx, ctrl, strength, sharpness, *weights):
        _, table, _ = ctrl._segment_table()
        ctx.strength, ctx.sharpness = strength, sharpness
        ctx.save_for_backward(*weights)
        _, total = ops.qloss_multi(table, sharpness, strength)
        return total.reshape(())

    @staticmethod
    def backward(ctx, grad_output):
        weights = ctx.saved_tensors
        need = ctx.needs_input_grad[3:]
        live = [i for i in range(len(weights)) if need[i]]
        out = [None] * len(weights)
        if live:
            dws = _b.softstep_bwd_all([weights[i].data for i in live], [None] * len(live), grad_output, 1.0,
                                      ctx.sharpness, ctx.strength)
            for i, dw in zip(live, dws):
                out[i] = dw
        return (None, None, None) + tuple(out)


class SoftStep(Function):
    """The differentiable staircase (tmq/tmq.py:315-438): y = sig(d frac(w) - d/2) / (2 sig(d/2)) +
    1/2 + floor(w), sig a clamped cubic-over-quadratic. Forward and backward are single HIP kernels
    with the fp32 arithmetic of the reference's CPU op chain."""

    @staticmethod
    @torch.no_grad()
    def map(weight: torch.Tensor, ctrl: QuantizationControl) -> torch.Tensor:
        """Soft-quantized image of a tensor, for logging and final ternarisation (tmq/tmq.py:328-338)."""
        assert ctrl, "Control instance is required"
        _require_gpu_weight(weight, "SoftStep.map")
        return ops.softstep_map(weight.data, ctrl.digamma, derivative=False)

    @staticmethod
    @torch.no_grad()
    def dmap(weight: torch.Tensor, ctrl: QuantizationControl) -> torch.Tensor:
        """Slope of the staircase at a tensor (tmq/tmq.py:341-350)."""
        assert ctrl, "Control instance is required"
        _require_gpu_weight(weight, "SoftStep.dmap")
        return ops.softstep_map(weight.data, ctrl.digamma, derivative=True)

    @staticmethod
    def sigmoid(input: torch.Tensor) -> torch.Tensor:
        """tmq/tmq.py:353-360"""
        _require_gpu_weight(input, "SoftStep.sigmoid")
        return ops.sigmoid_piece(input, 0)

    @staticmethod
    def dsigmoid(input: torch.Tensor) -> torch.Tensor:
        """tmq/tmq.py:363-370"""
        _require_gpu_weight(input, "SoftStep.dsigmoid")
        return ops.sigmoid_piece(input, 1)

    @staticmethod
    def d2sigmoid(input: torch.Tensor) -> torch.Tensor:
        """tmq/tmq.py:373-381"""
        _require_gpu_weight(input, "SoftStep.d2sigmoid")
        return ops.sigmoid_piece(input, 2)

    @staticmethod
    def scalar_sigmoid(input: float) -> float:
        """tmq/tmq.py:384-391"""
        x = min(3.0, max(-3.0, input))
        return x * (x * x + 27.0) / (27.0 + x * x * 9.0)

    @staticmethod
    def scalar_dsigmoid(input: float) -> float:
        """tmq/tmq.py:394-401"""
        x = min(3.0, max(-3.0, input))
        x2 = x * x
        return ((x2 - 9) * (x2 - 9)) / (9 * (3 + x2) * (3 + x2))

    @staticmethod
    def forward(ctx, weight, scale: float, ctrl: QuantizationControl):
        _require_gpu_weight(weight, "SoftStep")
        ctx.ctrl = ctrl
        ctx.scale = scale            # only scales the gradient (tmq/tmq.py:412)
        ctx.save_for_backward(weight)
        return _b.fwd_softstep(weight.data, ctrl.digamma)

    @staticmethod
    def backward(ctx, grad_output):
        weight = ctx.saved_tensors[0]
        return _b.bwd_softstep(weight.data, ctx.ctrl.digamma, ctx.scale, grad_output), None, None


class SoftStepDerivative(Function):
    """First derivative of the staircase as an autograd function -- the quantization-loss
    integrand (tmq/tmq.py:441-493)."""

    @staticmethod
    def forward(ctx, weight, digamma, strength):
        _require_gpu_weight(weight, "SoftStepDerivative")
        ctx.save_for_backward(weight)
        ctx.digamma = digamma
        ctx.strength = strength
        return _b.fwd_softstep_derivative(weight.data, digamma, strength)

    @staticmethod
    def backward(ctx, grad_output):
        weight = ctx.saved_tensors[0]
        return _b.bwd_softstep_derivative(weight.data, ctx.digamma, ctx.strength, grad_output), None, None


class TMQLayer:
    """Bookkeeping shared by the quantization-aware layers (tmq/tmq.py:496-570)."""

    _VARIANCE = {QuantMode.TERNARY: 2.0 / 3.0, QuantMode.TWO_BIT: (2 * 2 * 2 + 2 + 1) / 6.0,
                 QuantMode.THREE_BIT: (2 * 4 * 4 + 4 + 1) / 6.0, QuantMode.FOUR_BIT: (2 * 8 * 8 + 8 + 1) / 6.0,
                 QuantMode.FIVE_BIT: (2 * 16 * 16 + 16 + 1) / 6.0, QuantMode.SIX_BIT: (2 * 32 * 32 + 32 + 1) / 6.0,
                 QuantMode.EIGHT_BIT: (2 * 128 * 128 + 128 + 1) / 6.0}

    def __init__(self, ctrl=None, quant_mode=QuantMode.NONE, tensor_type=TensorType.FLOAT_32BIT, device=None):
        self._ctrl = ctrl
        self.quantization = quant_mode
        self.tensor_type = tensor_type
        self._device = device
        self.compact = False
        self.original_shape = None
        self.post_scale_imm = 1.0
        self.post_scale = None
        self.layer_name = None
        self._scale_dirty = True
        self._native = None          # cached kernel-native weights for compact inference
        self._scale_vec = None
        self._pair_epilogue = None   # scale / bias repeated for the pixel-pair form of a first layer
        self._fold = None            # (scale [N], bias [N]) of a BatchNorm folded into the compact epilogue

    def compact_inference_mode(self):
        self.training = False
        self.compact = True

    def quantization_loss(self, strength, sharpness):
        """mean(SoftStepDerivative(w, sharpness, strength)) (tmq/tmq.py:698-699, 889-891)."""
        return torch.mean(SoftStepDerivative.apply(self.weight, sharpness, strength))

    def quantize(self):
        """Round the fp32 weights to the nearest integers, half to even (tmq/tmq.py:599-603, 882-886)."""
        _require_gpu_weight(self.weight.data, "quantize")
        self.weight.data = ops.ternarize_(self.weight.data.contiguous().clone())

    @torch.no_grad()
    def clamp(self, limits=(-1., 1.)):
        """Clamp the weights (not the bias) in place (tmq/tmq.py:691-696, 874-879)."""
        _require_gpu_weight(self.weight.data, "clamp")
        if not self.weight.data.is_contiguous():
            self.weight.data = self.weight.data.contiguous()
        ops.clamp_(self.weight.data, limits[0], limits[1])

    def _update_scale(self):
        if self._scale_dirty and self.post_scale is not None:
            self.post_scale_imm = self.post_scale.item()
            self._scale_dirty = False

    def _variance_estimate(self) -> float:
        """Output variance of a unit-variance input under the layer's quantization levels
        (tmq/tmq.py:550-570)."""
        return self._VARIANCE.get(self.quantization, 1.0)

    def _soft_weight(self):
        ctrl = self._ctrl
        if ctrl is None or ctrl.inference_mode:
            return self.weight
        y = ctrl._soft_weight_of(self)
        return y if y is not None else SoftStep.apply(self.weight, 1.0, ctrl)

    def _weight_key(self, *extra):
        """Identity of the compact weight tensor for the cache of its kernel-native form: storage address,
        shape and the Parameter's version counter (weight.data has a counter of its own that never moves).
        In-place writes that bypass autograd's bookkeeping (weight.data.copy_(...)) are not seen: call
        invalidate_native() after them."""
        w = self.weight
        return (w.data_ptr(), tuple(w.shape), w._version) + extra

    def invalidate_native(self):
        """Drop the cached kernel-native form of the compact weights (rebuilt on the next forward)."""
        self._native = None

    def _native_weights(self, conv_kernel=None):
        key = self._weight_key()
        if self._native is None or self._native[0] != key:
            self._native = (key, ops.NativeWeights(self.weight.data, self.original_shape[0], conv_kernel))
        return self._native[1]

    def _epilogue_scale(self, n, device):
        """Per-channel scale vector carrying the scalar post-scale (None when it is 1)."""
        if self.post_scale_imm == 1.0:
            return None
        if self._scale_vec is None or self._scale_vec[0] != (self.post_scale_imm, n, device):
            self._scale_vec = ((self.post_scale_imm, n, device),
                               torch.full((n,), self.post_scale_imm, dtype=torch.float32, device=device))
        return self._scale_vec[1]

    def _epilogue(self, n, device):
        """(per-channel scale or None, bias or None) of the compact forward: the scalar post-scale and
        the layer's bias, then the affine map of a folded BatchNorm (fold_batchnorm) on top:
        bn(ps * acc + b) = (g * ps) * acc + (g * b + h)."""
        scale = self._epilogue_scale(n, device)
        bias = self.bias.data.float() if getattr(self, "bias", None) is not None else None
        if self._fold is None:
            return scale, bias
        g, h = self._fold
        if g.device != device:
            g, h = g.to(device), h.to(device)
            self._fold = (g, h)
        scale = g * self.post_scale_imm if self.post_scale_imm != 1.0 else g
        bias = h if bias is None else g * bias + h
        return scale, bias

    def _adopt_stored_weight(self, state_dict, prefix, local_metadata):
        """Shared tail of _load_from_state_dict (tmq/tmq.py:748-765, 956-973): interpret the
        tmq.* metadata written by compressed_state_dict."""
        if "tmq.quant" in local_metadata and "tmq.tensor_type" in local_metadata:
            self.tensor_type = TensorType(local_metadata["tmq.tensor_type"])
            self.original_shape = local_metadata["tmq.shape"]
            if self.tensor_type == TensorType.COMPRESSED_TERNARY_32BIT:
                stored = state_dict[prefix + "weight"]
                dev = self.weight.device
                self.weight = nn.Parameter(_b.decompress_ternary(stored.cpu(), self.original_shape).to(dev),
                                           requires_grad=False)
                self.tensor_type = TensorType.COMPACT_TERNARY_32BIT
                self.compact = True
            elif self.tensor_type == TensorType.COMPACT_TERNARY_32BIT:
                self.weight = nn.Parameter(state_dict[prefix + "weight"].to(self.weight.device), requires_grad=False)
                self.compact = True
            else:
                self.compact = False
            self.quantization = QuantMode(local_metadata["tmq.quant"])
            self.training = False if self.compact else self.training
            self._native = None
        else:
            self.compact = False


def _uniform_init(*shape):
    # U(-1, 1) drawn exactly like the reference (one torch.rand call on the CPU generator), so
    # seeded runs start from the same weights (tmq/tmq.py:723-725, 919-927).
    return 2.0 * (torch.rand(*shape) - 0.5)


class Linear(nn.Module, TMQLayer):
    """Quantization-aware drop-in for nn.Linear (tmq/tmq.py:573-765)."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None,
                 ctrl: QuantizationControl = None, quant_mode=QuantMode.NONE, post_scale=False):
        nn.Module.__init__(self)
        TMQLayer.__init__(self, ctrl, quant_mode, TensorType.FLOAT_32BIT, device)
        self.weight = nn.Parameter()
        self._in_features = in_features
        self._out_features = out_features
        self._init_weights(bias, device)
        self.original_shape = self.weight.shape
        self.post_scale_imm = 1.0 / (self._in_features * self._variance_estimate()) if post_scale else 1.0
        self.post_scale = nn.Parameter(torch.tensor(self.post_scale_imm), requires_grad=False)
        self.bn = None

    def __repr__(self):
        if len(self.original_shape) == 2:
            return "Linear(%d,%d) [tmq]" % tuple(self.original_shape) + " <%s>" % self.layer_name
        return "Linear(???) [tmq] <%s>" % self.layer_name

    def disable_bias(self):
        self.bias = None

    def implicit_bn(self):
        """Attach an internal BatchNorm1d that rescales the layer output (tmq/tmq.py:611-622)."""
        self.bn = nn.BatchNorm1d(self._out_features)

    def forward(self, x):
        """Training / fp32 path: F.linear on the soft-quantized weights; compact path when packed
        weights are loaded (tmq/tmq.py:637-659; the reference's debug dump of 624-635 is not kept)."""
        if self.compact:
            return self.compact_forward(x)
        assert self._ctrl or not self.training, "Quantization controller required for training"
        self._update_scale()
        w = self._soft_weight()
        if self.post_scale != 1.0:
            out = self.post_scale * nn.functional.linear(x, w, None)
            final = self.bias + out if self.bias is not None else out
        else:
            final = nn.functional.linear(x, w, self.bias)
        return self.bn(final) if self.bn is not None else final

    forward_wrap = forward

    @torch.no_grad()
    def compact_forward(self, x, residual=None, relu=False):
        """Inference straight from the 2-bit packed weights (tmq/tmq.py:662-688), any batch shape.
        residual / relu: added / applied in the kernel's epilogue (fuse_epilogues)."""
        assert self.training == False, "Compact inference is not supported in training mode"
        assert self.weight.data.dtype == torch.int32, "Compact inference requires 32-bit integer words"
        self._update_scale()
        if x.dim() == 4:
            assert x.shape[1] == 1, "Illegal shape supplied"
        nw = self._native_weights()
        xin = x if x.is_contiguous() else x.contiguous()
        scale, bias = self._epilogue(nw.N, x.device)
        if (residual is not None or relu) and self.bn is not None:
            raise RuntimeError("compact_forward: the layer's own BatchNorm comes between the product and the fused epilogue")
        if residual is not None:
            residual = residual.to(_compact_out).contiguous()
        out = ops.ternary_linear(xin, nw, scale=scale, bias=bias, residual=residual, relu=relu, out_dtype=_compact_out)
        return self.bn(out) if self.bn is not None else out

    @classmethod
    def from_linear(cls, source: nn.Linear, name: str, ctrl: QuantizationControl):
        assert ctrl, "Control instance is required"
        obj = cls(source.in_features, source.out_features, source.bias is not None, ctrl=ctrl,
                  device=source.weight.device, quant_mode=ctrl.quantization, post_scale=ctrl.post_scale)
        obj.layer_name = name
        ctrl.register_node(name, obj)
        return obj

    @torch.no_grad()
    def _init_weights(self, bias, device):
        if bias:
            self.bias = nn.Parameter(torch.zeros(self._out_features).to(device), requires_grad=True)
        else:
            self.bias = None
        self.weight = nn.Parameter(_uniform_init(self._out_features, self._in_features).to(device),
                                   requires_grad=True)

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                                      error_msgs)
        self._adopt_stored_weight(state_dict, prefix, local_metadata)


def _pair(v):
    return tuple(v) if isinstance(v, (tuple, list)) else (v, v)


def _phase_extent(r, s, p, n_out, n_in, geo):
    """One axis of one phase of a transposed convolution (ConvTranspose2d._phase_weights): the output
    positions o = s q + r - p inside [0, n_out) and the stride-1 convolution over the n_in input positions that
    computes them. geo = (taps, largest e, step of e). Returns (first output position, count, padding before,
    padding after, leading results to skip) or None when the phase has no output position."""
    taps, e_max, step = geo
    q_min = -((r - p) // s)                       # ceil((p - r) / s)
    q_max = (n_out - 1 + p - r) // s
    if q_max < q_min:
        return None
    count = q_max - q_min + 1
    first = s * q_min + r - p
    if taps == 0:
        return first, count, 0, 0, 0
    # result u of the convolution reads x[u - before + t step]; it stands for q = u + q_start with before = e_max - q_start
    q_start = min(q_min, e_max)                   # no negative padding: start earlier and skip
    before, skip = e_max - q_start, q_min - q_start
    after = max(0, (skip + count) - n_in - before + step * (taps - 1))
    return first, count, before, after, skip


class Conv2d(nn.Module, TMQLayer):
    """Quantization-aware drop-in for nn.Conv2d (tmq/tmq.py:769-973)."""

    _transposed = False

    def __init__(self, in_channels, out_channels, kernel, stride=1, padding=0, groups=1, dilation=1, bias=True,
                 device=None, ctrl=None, quant_mode=QuantMode.NONE, post_scale=False):
        nn.Module.__init__(self)
        TMQLayer.__init__(self, ctrl, quant_mode, TensorType.FLOAT_32BIT, device)
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel = kernel
        self.stride = stride
        self.padding = padding
        self.groups = groups
        self.dilation = dilation
        self._init_weights(bias, device)
        self.original_shape = self.weight.shape
        self.post_scale_imm = 1.0 / (self._fan_in * self._variance_estimate()) if post_scale else 1.0
        self.post_scale = nn.Parameter(torch.tensor(self.post_scale_imm), requires_grad=False)

    def __repr__(self):
        return "Conv2d(%d,%d,%d,%d) [tmq]" % tuple(self.original_shape) + " <%s>" % self.layer_name

    def to(self, *args, **kwargs):
        me = super().to(*args, **kwargs)
        me.post_scale_imm = me.post_scale.item()
        return me

    def _conv(self, x, w, bias):
        return nn.functional.conv2d(x, w, bias, self.stride, self.padding, dilation=self.dilation, groups=self.groups)

    def forward(self, x):
        """tmq/tmq.py:805-819"""
        if self.compact:
            return self.compact_forward(x)
        assert self._ctrl or not self.training, "Quantization controller required for training"
        self._update_scale()
        w = self._soft_weight()
        if self.post_scale != 1.0:
            out = self.post_scale * self._conv(x, w, None)
            return self.bias + out if self.bias is not None else out
        return self._conv(x, w, self.bias)

    @torch.no_grad()
    def compact_forward(self, x, residual=None, relu=False, pool=False):
        """Implicit-GEMM convolution from the packed weights (replaces the unfold / GEMM / fold
        sequence of tmq/tmq.py:822-871). Output extents follow PyTorch's formula. Returns fp32
        [B, N, Ho, Wo] (channels_last memory); a 3-D input gives a 3-D output.
        residual / relu: added / applied in the kernel's epilogue (fuse_epilogues). pool: a 3 x 3 / stride 2 /
        pad 1 max-pool follows the ReLU (fp16 output, no residual, groups == 1): one call, and for a network's
        first layer one kernel."""
        assert not self.training, "Compact inference is not supported in training mode"
        assert self.weight.data.dtype == torch.int32, "Compact inference requires 32-bit integer words"
        self._update_scale()
        if pool and not (relu and residual is None and self.groups == 1 and x.dim() == 4 and _compact_out == torch.float16):
            raise RuntimeError("compact_forward(pool=True) needs relu, no residual, groups == 1, a 4-D input and fp16 outputs")
        if x.dim() == 3:
            r3 = residual.unsqueeze(0) if residual is not None else None
            return self.compact_forward(x.unsqueeze(0), r3, relu).squeeze(0)
        if residual is not None and (residual.dtype != _compact_out or
                                     not residual.is_contiguous(memory_format=torch.channels_last)):
            residual = residual.to(dtype=_compact_out, memory_format=torch.channels_last)
        if x.dim() != 4:
            raise Exception("Expected a 3D tensor")
        assert self.groups == 1 or self.groups == self.original_shape[0], \
            "Grouped convolutions are only supported for group == channels"
        ky, kx = _pair(self.kernel)
        if self.groups != 1:
            # depthwise (tmq/tmq.py:849-853): the compact words are read as they are, no re-tiling
            if self.original_shape[1] != 1 or x.shape[1] != self.original_shape[0]:
                raise RuntimeError("depthwise compact inference needs one filter per input channel")
            scale, bias = self._epilogue(x.shape[1], x.device)
            return ops.ternary_dwconv2d(x, self.weight.data, (ky, kx), _pair(self.stride), _pair(self.padding),
                                        _pair(self.dilation), scale=scale, bias=bias, residual=residual, relu=relu,
                                        out_dtype=_compact_out)
        scale, bias = self._epilogue(int(self.original_shape[0]), x.device)
        sp = self._superpixel_plan(x)
        if sp is not None:
            # a network's first layer (at most 4 input channels, horizontal stride 2): two neighbouring
            # pixels of the 4-channel NHWC image are read as one pixel of 8 channels, see _superpixel_plan
            nw, kxs, pl, pr = sp
            B, C, H, W = x.shape
            if x.dtype == torch.float32:
                x, scale = ops.f32_to_f16_prescaled(x, scale, int(self.original_shape[0]))
            (sy, _), (py, _) = _pair(self.stride), _pair(self.padding)
            if pool:      # the one-kernel opening gathers the pixel pairs from the NCHW planes itself
                return ops.ternary_conv2d_relu_maxpool_planar(x, nw, (sy, 1), ((py, py), (pl, pr)), 1, scale=scale, bias=bias)
            xs = ops.nchw_to_nhwc4(x).view(B, H, W // 2, 8).permute(0, 3, 1, 2)
            return ops.ternary_conv2d(xs, nw, (sy, 1), ((py, py), (pl, pr)), 1, scale=scale, bias=bias,
                                      residual=residual, relu=relu, out_dtype=_compact_out)
        pp = self._pixelpair_plan(x)
        if pp is not None:
            # a first layer with at most 4 input channels and horizontal stride 1: pairs of input pixels are read as
            # one pixel of 8 channels and pairs of output pixels come out as one pixel of 2 N channels, see _pixelpair_plan
            nw, kxs, pl, pr, scale, bias = pp
            B, C, H, W = x.shape
            N = int(self.original_shape[0])
            if x.dtype == torch.float32:
                x, scale = ops.f32_to_f16_prescaled(x, scale, 2 * N)
            (sy, _), (py, _) = _pair(self.stride), _pair(self.padding)
            if x.is_contiguous():
                xs = ops.nchw_to_nhwc4(x).view(B, H, W // 2, 8).permute(0, 3, 1, 2)
            else:                         # 4 channels in channels-last memory are the pixel pairs already
                xs = x.permute(0, 2, 3, 1).view(B, H, W // 2, 8).permute(0, 3, 1, 2)
            if residual is not None:      # [B, N, Ho, Wo] in NHWC memory is [B, Ho, Wo / 2, 2 N]
                Ho, Wo = int(residual.shape[2]), int(residual.shape[3])
                residual = residual.permute(0, 2, 3, 1).view(B, Ho, Wo // 2, 2 * N).permute(0, 3, 1, 2)
            ys = ops.ternary_conv2d(xs, nw, (sy, 1), ((py, py), (pl, pr)), 1, scale=scale, bias=bias, residual=residual,
                                    relu=relu, out_dtype=_compact_out)
            Ho, Wh = int(ys.shape[2]), int(ys.shape[3])
            y = ys.permute(0, 2, 3, 1).view(B, Ho, 2 * Wh, N).permute(0, 3, 1, 2)
            return ops.maxpool2d_nhwc(y, 3, 2, 1) if pool else y      # the one-kernel opening is for horizontal stride 2
        nw = self._native_weights(conv_kernel=(ky, kx))
        if pool:
            return ops.ternary_conv2d_relu_maxpool(x, nw, _pair(self.stride), _pair(self.padding), _pair(self.dilation),
                                                   scale=scale, bias=bias)
        return ops.ternary_conv2d(x, nw, _pair(self.stride), _pair(self.padding), _pair(self.dilation), scale=scale,
                                  bias=bias, residual=residual, relu=relu, out_dtype=_compact_out)

    def _pixelpair_plan(self, x):
        """For a convolution with at most 4 input channels, horizontal stride 1, no dilation and an odd window
        width on a contiguous NCHW fp16 / fp32 input (a network's own input) of a width that is a multiple of 4:
        the equivalent convolution whose input pixels are pairs (2u, 2u + 1) of image pixels stored NHWC with 4
        channels (8 channels, the 16-byte loader applies) and whose output pixels are pairs (2u, 2u + 1) of
        output pixels (2 N channels: filter v' N + n produces column 2u + v' of filter n). Output column
        2u + v' reads image columns 2u + v' - px + j = 2 (u + t) + v, so pair tap t, channel 4 v + c of filter
        v' N + n carries the weight of (n, c, j = 2 t + v - v' + px). In memory [B, Ho, Wo / 2, 2 N] is
        [B, Ho, Wo, N]: the result needs no rearrangement. Returns (native weights, pair taps, pad left,
        pad right, scale or None, bias or None -- both repeated for the 2 N filters) or None when the layer
        does not qualify. Four channels in channels-last memory are pixel pairs as they lie (no repack launch); fewer
        channels in channels-last memory keep the generic loader."""
        N, C, ky, kx = (int(v) for v in self.original_shape)
        (sy, sx), (py, px), (dy, dx) = _pair(self.stride), _pair(self.padding), _pair(self.dilation)
        W = int(x.shape[-1])
        if C > 4 or x.shape[1] != C or sx != 1 or (dy, dx) != (1, 1) or W % 4 or kx % 2 == 0 or x.numel() == 0 or \
                x.dtype not in (torch.float16, torch.float32) or \
                not (x.is_contiguous() or (C == 4 and x.is_contiguous(memory_format=torch.channels_last))) or \
                isinstance(py, (tuple, list)) or isinstance(px, (tuple, list)):
            return None
        t_min, t_max = (-px) // 2, (kx - px) // 2
        kxs, pl = t_max - t_min + 1, -t_min
        wo = W + 2 * px - kx + 1
        pr = wo // 2 - 1 + kxs - W // 2 - pl
        if wo < 2 or wo % 2 or pr < 0:
            return None
        key = self._weight_key("pixelpair")
        if self._native is None or self._native[0] != key:
            full = ops.expand_ternary(self.weight.data, [N, C, ky, kx])
            wpp = torch.zeros((2 * N, 8, ky, kxs), dtype=full.dtype, device=full.device)
            for t in range(kxs):
                for v in range(2):
                    for vo in range(2):
                        j = 2 * (t + t_min) + v - vo + px
                        if 0 <= j < kx:
                            wpp[vo * N:(vo + 1) * N, 4 * v:4 * v + C, :, t] = full[:, :, :, j]
            self._native = (key, ops.NativeWeights(ops.compactify_ternary(wpp), 2 * N, (ky, kxs)))
        b = getattr(self, "bias", None)
        ekey = (self.post_scale_imm, id(self._fold), None if b is None else (b.data_ptr(), b._version), x.device)
        if self._pair_epilogue is None or self._pair_epilogue[0] != ekey:
            scale, bias = self._epilogue(N, x.device)
            # the folded pair is kept in the entry so that its id cannot be handed to a later one while the entry lives
            self._pair_epilogue = (ekey, None if scale is None else scale.repeat(2), None if bias is None else bias.repeat(2),
                                   self._fold)
        return self._native[1], kxs, pl, pr, self._pair_epilogue[1], self._pair_epilogue[2]

    def _superpixel_plan(self, x):
        """For a convolution with at most 4 input channels, horizontal stride 2 and no dilation on an
        NCHW fp16 / fp32 input of even width: the equivalent stride-1 convolution over "super-pixels"
        (pixels 2u and 2u + 1 of the image stored NHWC with 4 channels, read as one pixel of 8
        channels). Output column ow reads image columns 2 ow - px + j = 2 (ow + t) + v with
        t = floor((j - px) / 2), v = (j - px) mod 2, so super-pixel tap t, channel 4 v + c carries the
        weight of (c, j) and the taps t_min .. t_max replace the kx image taps: the reduction is
        ky * kxs * 8 long (224 for a 7 x 7 / 2 stem) where padding 3 channels to 8 would make it
        ky * kx * 8 (392), and the 16-byte loader applies instead of the scalar one.
        Returns (native weights, kxs, pad left, pad right) or None when the layer does not qualify."""
        N, C, ky, kx = (int(v) for v in self.original_shape)
        (sy, sx), (py, px), (dy, dx) = _pair(self.stride), _pair(self.padding), _pair(self.dilation)
        W = int(x.shape[-1])
        if C > 4 or x.shape[1] != C or sx != 2 or (dy, dx) != (1, 1) or W % 4 or x.dtype not in (torch.float16, torch.float32) or \
                isinstance(py, (tuple, list)) or isinstance(px, (tuple, list)):
            return None
        t_min, t_max = (-px) // 2, (kx - 1 - px) // 2
        kxs, pl = t_max - t_min + 1, -t_min
        wo = (W + 2 * px - kx) // 2 + 1
        pr = wo - 1 + kxs - W // 2 - pl
        if wo < 1 or pr < 0:
            return None
        w = self.weight.data
        key = self._weight_key("superpixel")
        if self._native is None or self._native[0] != key:
            full = ops.expand_ternary(w, [N, C, ky, kx])
            wsp = torch.zeros((N, 8, ky, kxs), dtype=full.dtype, device=full.device)
            for t in range(kxs):
                for v in range(2):
                    j = 2 * (t + t_min) + v + px
                    if 0 <= j < kx:
                        wsp[:, 4 * v:4 * v + C, :, t] = full[:, :, :, j]
            self._native = (key, ops.NativeWeights(ops.compactify_ternary(wsp), N, (ky, kxs)))
        return self._native[1], kxs, pl, pr

    @classmethod
    def from_conv2d(cls, source: nn.Conv2d, name: str, ctrl: QuantizationControl):
        assert ctrl, "Controller required"
        obj = cls(source.in_channels, source.out_channels, source.kernel_size, stride=source.stride,
                  padding=source.padding, groups=source.groups, dilation=source.dilation,
                  bias=source.bias is not None, device=source.weight.device, ctrl=ctrl,
                  quant_mode=ctrl.quantization, post_scale=ctrl.post_scale)
        obj.layer_name = name
        ctrl.register_node(name, obj)
        return obj

    def _weight_shape(self, ky, kx):
        return [self.out_channels, self.in_channels // self.groups, ky, kx]

    @torch.no_grad()
    def _init_weights(self, bias, device):
        ky, kx = _pair(self.kernel)
        self._fan_in = ky * kx * self.in_channels
        self._fan_out = ky * kx * self.out_channels
        self.weight = nn.Parameter(_uniform_init(self._weight_shape(ky, kx)).to(device), requires_grad=True)
        if bias:
            self.bias = nn.Parameter(torch.zeros(self.out_channels).to(device), requires_grad=True)
        else:
            self.bias = None

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                                      error_msgs)
        self._adopt_stored_weight(state_dict, prefix, local_metadata)


class ConvTranspose2d(Conv2d):
    """Quantization-aware drop-in for nn.ConvTranspose2d (tmq/tmq.py:978-1087), with working compact
    paths for groups == 1 (the reference's own cannot pass its shape checks) and groups == channels."""

    _transposed = True

    def __init__(self, in_channels, out_channels, kernel, stride=1, padding=0, output_padding=0, groups=1, bias=True,
                 dilation=1, device=None, ctrl=None, quant_mode=QuantMode.NONE, post_scale=False):
        super().__init__(in_channels, out_channels, kernel, stride, padding, groups, dilation, bias, device, ctrl,
                         quant_mode, post_scale)
        self.output_padding = output_padding

    def __repr__(self):
        return "ConvTranspose2d(%d,%d,%d,%d) [tmq] " % tuple(self.original_shape) + " <%s>" % self.layer_name

    def _conv(self, x, w, bias):
        # output_padding is honoured (the reference's forward drops it, tmq/tmq.py:989-1003, and then
        # disagrees with the nn.ConvTranspose2d it replaced)
        return nn.functional.conv_transpose2d(x, w, bias, self.stride, self.padding, self.output_padding,
                                              groups=self.groups, dilation=self.dilation)

    def _weight_shape(self, ky, kx):
        return [self.in_channels, self.out_channels // self.groups, ky, kx]

    @torch.no_grad()
    def compact_forward(self, x):
        """Transposed convolution from the packed weights, gathered: every phase of the output grid is an
        ordinary stride-1 ternary implicit-GEMM convolution with the sub-kernel of the taps that reach it
        (_phase_weights), written into its strided share of the output. No columns and no F.fold, the useful
        multiply-adds only (the reference's plan, tmq/tmq.py:1005-1038, is GEMM + F.fold over columns ky kx /
        (sy sx) times the size of the output, and its own shape checks reject its weight view). The compact
        tensor of a [Cin, Cout, ky, kx] kernel packs along Cin, the reduction index here, so the sub-kernels
        are unpacked and re-packed along Cout once per layer. groups == channels takes the depthwise kernel."""
        assert not self.training, "Compact inference is not supported in training mode"
        assert self.weight.data.dtype == torch.int32, "Compact inference requires 32-bit integer words"
        self._update_scale()
        if x.dim() == 3:
            return self.compact_forward(x.unsqueeze(0)).squeeze(0)
        cin, cout, ky, kx = (int(v) for v in self.original_shape)
        if self.groups != 1:
            # depthwise (tmq/tmq.py:1025-1029, columns + F.fold there): gathered per output position
            # straight from the compact words
            assert self.groups == cin, "Grouped transpose convolutions are only supported for channels == groupsize"
            if cout != 1 or x.shape[1] != cin:
                raise RuntimeError("depthwise transposed compact inference needs one filter per input channel")
            bias = self.bias.data.float() if self.bias is not None else None
            return ops.ternary_dwconvtrans2d(x, self.weight.data, (ky, kx), _pair(self.stride), _pair(self.padding),
                                             _pair(self.output_padding), _pair(self.dilation),
                                             scale=self._epilogue_scale(cin, x.device), bias=bias)
        B, C, H, W = x.shape
        sy, sx = _pair(self.stride)
        py, px = _pair(self.padding)
        oy, ox = _pair(self.output_padding)
        dy, dx = _pair(self.dilation)
        h_out = (H - 1) * sy - 2 * py + dy * (ky - 1) + 1 + oy
        w_out = (W - 1) * sx - 2 * px + dx * (kx - 1) + 1 + ox
        if C != cin or h_out <= 0 or w_out <= 0:
            raise RuntimeError("ConvTranspose2d.compact_forward: input does not match the layer")
        phases = self._phase_weights(cin, cout, ky, kx, sy, sx, dy, dx)
        scale = self._epilogue_scale(cout, x.device)
        bias = self.bias.data.float() if self.bias is not None else None
        if x.dtype == torch.float32:
            x, scale = ops.f32_to_f16_prescaled(x, scale, cout)     # once for all phases
        if x.dtype != torch.float16 or not x.is_contiguous(memory_format=torch.channels_last):
            x = x.to(dtype=torch.float16, memory_format=torch.channels_last)
        y = torch.empty((B, cout, h_out, w_out), dtype=_compact_out, device=x.device, memory_format=torch.channels_last)
        for (rh, rw), (nw, geo_h, geo_w) in phases.items():
            rows, cols = _phase_extent(rh, sy, py, h_out, H, geo_h), _phase_extent(rw, sx, px, w_out, W, geo_w)
            if rows is None or cols is None:
                continue                                             # no output position in this phase
            (o0, cnt_h, pt, pb, skip_h), (p0, cnt_w, pl, pr, skip_w) = rows, cols
            target = y[:, :, o0::sy, p0::sx]
            if nw is None:                                           # no tap reaches this phase: bias only
                target.zero_()
                if bias is not None:
                    target += bias.to(y.dtype).view(1, -1, 1, 1)
                continue
            # one launch per phase, written in place: the kernel's epilogue scatters its rows into the phase's pixels
            ops.ternary_conv2d_into(target, x, nw, (1, 1), ((pt, pb), (pl, pr)), (geo_h[2], geo_w[2]), scale=scale, bias=bias,
                                    first=(skip_h, skip_w))
        return y

    def _phase_weights(self, cin, cout, ky, kx, sy, sx, dy, dx):
        """The transposed convolution as sy * sx ordinary stride-1 convolutions, one per phase
        (r_h, r_w) = ((oh + py) mod sy, (ow + px) mod sx) of the output grid: an output row oh = sy q + r - py is
        reached from input row ih = q - e by exactly the taps i with i dy = r (mod sy), e = (i dy - r) / sy. In
        terms of q that is a convolution of x with those taps in reverse order, dilation (step of e), left padding
        (largest e). Returns {(r_h, r_w): (native weights of the sub-kernel or None when it is empty,
        (taps, largest e, step of e) along h, the same along w)}; cached with the weights."""
        key = self._weight_key("phases", sy, sx, dy, dx)
        if self._native is not None and self._native[0] == key:
            return self._native[1]
        full = ops.expand_ternary(self.weight.data, [cin, cout, ky, kx])          # [Cin, Cout, ky, kx]

        def taps(k, s, d, r):
            idx = [i for i in range(k) if (i * d - r) % s == 0 and i * d >= r]
            if not idx:
                return idx, 0, 1
            e = [(i * d - r) // s for i in idx]
            step = e[1] - e[0] if len(e) > 1 else 1
            assert all(b - a == step for a, b in zip(e, e[1:]))
            return idx, e[-1], step

        phases = {}
        for rh in range(sy):
            ih, eh, dh = taps(ky, sy, dy, rh)
            for rw in range(sx):
                iw, ew, dw = taps(kx, sx, dx, rw)
                nw = None
                if ih and iw:
                    sub = full[:, :, ih][:, :, :, iw].flip(2, 3).permute(1, 0, 2, 3).contiguous()   # [Cout, Cin, Th, Tw]
                    nw = ops.NativeWeights(ops.compactify_ternary(sub), cout, (len(ih), len(iw)))
                phases[(rh, rw)] = (nw, (len(ih), eh, dh), (len(iw), ew, dw))
        self._native = (key, phases)
        return phases

    @classmethod
    def from_transconv2d(cls, source: nn.ConvTranspose2d, name: str, ctrl: QuantizationControl):
        assert ctrl, "Controller required"
        obj = cls(source.in_channels, source.out_channels, source.kernel_size, stride=source.stride,
                  padding=source.padding, output_padding=source.output_padding, groups=source.groups,
                  dilation=source.dilation, bias=source.bias is not None, device=ctrl.device, ctrl=ctrl,
                  quant_mode=ctrl.quantization, post_scale=ctrl.post_scale)
        obj.layer_name = name
        ctrl.register_node(name, obj)
        return obj


# ---- model / state utilities (tmq/tmq.py:1090-1319) -------------------------------------------------------
def _tmq_layers(module: nn.Module, prefix=""):
    """(qualified name, parent, child name, layer) for every TMQ layer below `module`, depth first
    in registration order; does not descend into TMQ layers."""
    for name, sub in module.named_children():
        full = prefix + "." + name if prefix != "" else name
        if isinstance(sub, TMQLayer):
            yield full, module, name, sub
        else:
            yield from _tmq_layers(sub, full)


def quantize_weights(module: nn.Module):
    """Snap the fp32 weights of every TMQ layer to integers in place (tmq/tmq.py:1090-1111)."""
    for name, sub in module.named_children():
        if isinstance(sub, TMQLayer):
            if sub.weight.data.dtype == torch.float16:
                raise Exception("FP16 data is currently not supported")
            if sub.weight.data.dtype == torch.float32:
                _require_gpu_weight(sub.weight.data, "quantize_weights")
                rounded = ops.ternarize_(sub.weight.data.contiguous().clone())
                sub.weight = nn.Parameter(rounded, requires_grad=sub.weight.requires_grad)
        quantize_weights(sub)


def quantize_model(module: nn.Module, ctrl: QuantizationControl, prefix="", exclude=[]):
    """Swap nn.Linear / nn.Conv2d / nn.ConvTranspose2d for their quantization-aware versions in
    place (tmq/tmq.py:1114-1180). `exclude` holds qualified names or '*' wildcards. The original
    parameters are discarded and re-initialised U(-1, 1)."""
    assert ctrl, "Must supply a quantization control instance"
    exact = [p for p in exclude if "*" not in p]
    globs = [p for p in exclude if "*" in p]
    _swap_layers(module, ctrl, prefix, exact, globs)


_FACTORIES = ((nn.Linear, lambda s, n, c: Linear.from_linear(s, n, c)),
              (nn.Conv2d, lambda s, n, c: Conv2d.from_conv2d(s, n, c)),
              (nn.ConvTranspose2d, lambda s, n, c: ConvTranspose2d.from_transconv2d(s, n, c)))


def _swap_layers(module, ctrl, prefix, exact, globs):
    for name, sub in module.named_children():
        if sub is module:
            continue
        path = prefix + "." + name if prefix != "" else name
        if path in exact:
            print("Skipping excluded layer %s" % path)
            continue                                   # an exactly excluded module is not descended into
        if any(fnmatch.fnmatch(path, g) for g in globs):
            print("Skipping excluded layer %s" % path)
        else:
            for kind, make in _FACTORIES:
                if isinstance(sub, kind):
                    # registered under prefix + "." + name: a leading dot for an empty prefix, as in
                    # the reference (tmq/tmq.py:1171)
                    sub = make(sub, prefix + "." + name, ctrl)
                    setattr(module, name, sub)
        _swap_layers(sub, ctrl, path, exact, globs)


def compressed_state_dict(module: nn.Module, strong=False, remove_prefix=""):
    """State dict with TMQ weights bit-stuffed (2 bit / weight) or, with strong=True, range coded;
    the layers are switched to compact inference as a side effect (tmq/tmq.py:1183-1248)."""
    for _, _, _, layer in _tmq_layers(module):
        if not hasattr(layer, "tensor_type"):
            continue
        if getattr(layer, "original_shape", None) is None:
            layer.original_shape = layer.weight.shape
        if not strong and layer.tensor_type != TensorType.COMPACT_TERNARY_32BIT:
            layer.weight = nn.Parameter(_b.compactify_ternary(layer.weight.data), requires_grad=False)
            layer.tensor_type = TensorType.COMPACT_TERNARY_32BIT
        elif strong and layer.tensor_type != TensorType.COMPRESSED_TERNARY_32BIT:
            from_compact = layer.tensor_type == TensorType.COMPACT_TERNARY_32BIT
            stream = _b.compress_ternary(layer.weight.data, layer.original_shape, from_compact)
            layer._stream_device = layer.weight.device
            layer.weight = nn.Parameter(stream, requires_grad=False)
            layer.tensor_type = TensorType.COMPRESSED_TERNARY_32BIT
        layer._native = None
    state = module.state_dict()
    for full, _, _, layer in _tmq_layers(module):
        layer.compact_inference_mode()
        meta = state._metadata[full]
        meta["tmq.tensor_type"] = layer.tensor_type.value
        meta["tmq.shape"] = layer.original_shape
        meta["tmq.quant"] = layer.quantization.value
        if layer.tensor_type == TensorType.COMPRESSED_TERNARY_32BIT:
            # keep the model usable right away: back to the compact form in memory
            dev = getattr(layer, "_stream_device", layer.weight.device)
            layer.weight = nn.Parameter(_b.decompress_ternary(layer.weight.data.cpu(), layer.original_shape).to(dev),
                                        requires_grad=False)
            layer.tensor_type = TensorType.COMPACT_TERNARY_32BIT
    return state


def prepare_compressed_load(module: nn.Module, state_dict):
    """tmq/tmq.py:1251-1252"""
    _presize_weights(module, state_dict, "")


def load_compressed_state_dict(module: nn.Module, state_dict):
    """Load a compact / compressed state dict; entropy-coded weights end up in the compact form
    in memory (tmq/tmq.py:1256-1268)."""
    _presize_weights(module, state_dict)
    module.load_state_dict(state_dict, strict=False)


def _presize_weights(module: nn.Module, state_dict, prefix=""):
    """Give every TMQ layer an empty weight of the stored shape and dtype so that load_state_dict
    accepts the packed tensors (tmq/tmq.py:1271-1293)."""
    meta = state_dict._metadata
    for full, _, _, layer in _tmq_layers(module, prefix):
        layer.layer_name = full
        if full not in meta or "tmq.tensor_type" not in meta[full]:
            continue
        kind = TensorType(meta[full]["tmq.tensor_type"])
        if kind in (TensorType.COMPACT_TERNARY_32BIT, TensorType.COMPRESSED_TERNARY_32BIT):
            stored = state_dict[full + ".weight"]
            layer.weight = nn.Parameter(torch.empty(stored.shape, dtype=stored.dtype, device=layer.weight.device),
                                        requires_grad=False)
        else:
            layer.compact = False


@torch.no_grad()
def fold_batchnorm(module: nn.Module, pairs=None):
    """Fold eval-mode BatchNorm layers into the epilogue of the compact TMQ layer that feeds them (the
    reference's README lists this fusion as future work, README.md:150-155): the layer then computes
    gamma * (y - mean) / sqrt(var + eps) + beta in its own per-channel scale / bias and the BatchNorm
    module is replaced by nn.Identity. For inference only; call it after the layers went compact
    (compressed_state_dict / load_compressed_state_dict).

    pairs: [(qualified layer name, qualified BatchNorm name), ...]. None = every BatchNorm that is
    registered right after a compact Linear / Conv2d in the same parent and has as many features as
    that layer has outputs (the conv1 / bn1, Sequential(conv, bn) idiom) -- pass explicit pairs when
    registration order is not execution order. Returns the list of folded pairs."""
    def fits(layer, bn):
        # a layer with a BatchNorm of its own (Linear.implicit_bn) applies it after the kernel's epilogue: an
        # affine map folded into that epilogue would come before it instead of after
        return (isinstance(layer, (Linear, Conv2d)) and not isinstance(layer, ConvTranspose2d) and layer.compact and
                getattr(layer, "bn", None) is None and
                isinstance(bn, (nn.BatchNorm1d, nn.BatchNorm2d)) and bn.track_running_stats and
                bn.num_features == int(layer.original_shape[0]))

    todo = []
    if pairs is None:
        for pname, parent in module.named_modules():
            kids = list(parent.named_children())
            for (ln, layer), (bname, bn) in zip(kids, kids[1:]):
                if fits(layer, bn) and layer._fold is None:
                    todo.append((parent, bname, layer, bn, (pname + "." if pname else "") + ln, (pname + "." if pname else "") + bname))
    else:
        mods = dict(module.named_modules())
        for ln, bname in pairs:
            layer, bn = mods[ln], mods[bname]
            if not fits(layer, bn):
                raise RuntimeError(f"fold_batchnorm: {ln} / {bname} is not a compact TMQ layer followed by a matching BatchNorm")
            parent = mods[bname.rpartition(".")[0]] if "." in bname else module
            todo.append((parent, bname.rpartition(".")[2], layer, bn, ln, bname))
    done = []
    for parent, child, layer, bn, ln, bname in todo:
        if bn.training:
            raise RuntimeError("fold_batchnorm: BatchNorm layers must be in eval mode")
        inv = (bn.running_var.float() + bn.eps).rsqrt()
        g = inv * bn.weight.float() if bn.affine else inv
        h = (bn.bias.float() if bn.affine else 0.0) - bn.running_mean.float() * g
        layer._fold = (g.contiguous(), h.contiguous())
        setattr(parent, child, nn.Identity())
        done.append((ln, bname))
    return done


class _FusedEpilogue(nn.Module):
    """A compact layer called with its residual input and / or a ReLU in the kernel's epilogue; `pool`: the
    3 x 3 / stride 2 / pad 1 max-pool module that followed the ReLU, taken into the same call when the layer
    hands on fp16 (set_compact_output_dtype) and applied as it was otherwise."""

    def __init__(self, layer, relu, pool=None):
        super().__init__()
        self.layer = layer
        self.relu = bool(relu)
        self.pool = pool

    def forward(self, x, residual=None):
        if self.pool is None:
            return self.layer.compact_forward(x, residual, self.relu)
        if _compact_out == torch.float16 and x.is_cuda and x.dim() == 4:
            return self.layer.compact_forward(x, None, True, pool=True)
        return self.pool(self.layer.compact_forward(x, None, True))


class _FusedHead(nn.Module):
    """linear(flatten(global_average_pool(x), 1)) as one launch when x is an fp16 channels_last feature map of up to
    512 channels (the means stay in LDS and are the product's only activation row per image); the three modules as
    they were otherwise."""

    def __init__(self, pool, layer):
        super().__init__()
        self.pool = pool
        self.layer = layer

    @torch.no_grad()
    def forward(self, x):
        layer = self.layer
        if (x.is_cuda and x.dim() == 4 and x.dtype == torch.float16 and x.is_contiguous(memory_format=torch.channels_last)
                and not layer.training and layer.compact and layer.bn is None):
            layer._update_scale()
            nw = layer._native_weights()
            scale, bias = layer._epilogue(nw.N, x.device)
            return ops.avgpool_linear(x, nw, scale=scale, bias=bias, out_dtype=_compact_out)
        return layer(torch.flatten(self.pool(x), 1))


def fuse_epilogues(model: nn.Module):
    """Move the ReLU and the residual addition that follow a compact Conv2d / Linear in the model's forward
    into that layer's kernel epilogue (the reference's README lists this fusion as future work,
    README.md:150-155). The model is traced with torch.fx (TMQ layers are leaves); recognised are, with any
    number of nn.Identity modules (what fold_batchnorm leaves behind) in between,

        relu(layer(x))      layer(x) + r      relu(layer(x) + r)      maxpool(relu(conv(x)))
        linear(flatten(avgpool(x), 1))

    where `relu` is torch.relu / F.relu / x.relu() / an nn.ReLU module, `+` is +, += or torch.add, the
    layer is a compact Conv2d or Linear without a BatchNorm of its own, `maxpool` is an nn.MaxPool2d(3, 2, 1)
    module (a ResNet's opening; one kernel once the layers hand on fp16), `avgpool` an nn.AdaptiveAvgPool2d(1) module
    (a network's head: pooling and classifier in one launch on fp16 feature maps), and the intermediate values have no
    other use. Everything else stays as traced. For inference, after the layers went compact and after
    fold_batchnorm. Returns (GraphModule sharing the model's parameters, number of fused sites)."""
    import operator
    import torch.fx as fx

    class Tracer(fx.Tracer):
        def is_leaf_module(self, m, qualname):
            # this module's own layers and wrappers branch on their input: never trace into them
            return isinstance(m, TMQLayer) or type(m).__module__ == __name__ or super().is_leaf_module(m, qualname)

    graph = Tracer().trace(model)
    mods = dict(model.named_modules())

    def is_relu(n):
        if n.op == "call_function":
            return n.target in (torch.relu, nn.functional.relu, torch.relu_) and len(n.args) >= 1
        if n.op == "call_method":
            return n.target in ("relu", "relu_")
        return n.op == "call_module" and isinstance(mods.get(n.target), nn.ReLU)

    def is_add(n):
        if n.op == "call_function":
            return n.target in (operator.add, operator.iadd, torch.add) and len(n.args) == 2 and not n.kwargs
        return n.op == "call_method" and n.target in ("add", "add_") and len(n.args) == 2 and not n.kwargs

    def only_user(n):
        users = list(n.users)
        return users[0] if len(users) == 1 else None

    gm = fx.GraphModule(model, graph)
    fused = 0
    for node in list(graph.nodes):
        if node.op != "call_module":
            continue
        layer = mods.get(node.target)
        if not (isinstance(layer, (Linear, Conv2d)) and not isinstance(layer, ConvTranspose2d) and layer.compact
                and getattr(layer, "bn", None) is None and len(node.args) == 1 and not node.kwargs):
            continue
        # follow the value through Identity modules
        last = node
        while True:
            nxt = only_user(last)
            if nxt is not None and nxt.op == "call_module" and isinstance(mods.get(nxt.target), nn.Identity):
                last = nxt
            else:
                break
        nxt = only_user(last)
        if nxt is None:
            continue
        residual, end, relu = None, None, False
        if is_add(nxt) and nxt.args[0] is not nxt.args[1] and isinstance(nxt.args[0], fx.Node) and isinstance(nxt.args[1], fx.Node):
            residual = nxt.args[1] if nxt.args[0] is last else nxt.args[0]
            end = nxt
            after = only_user(nxt)
            if after is not None and is_relu(after) and after.args[0] is nxt:
                end, relu = after, True
        elif is_relu(nxt) and nxt.args[0] is last:
            end, relu = nxt, True
        if end is None:
            continue
        # relu(conv(x)) handed only to a 3 x 3 / stride 2 / pad 1 max-pool (a ResNet's opening): the pool joins the call
        pool = None
        if relu and residual is None and isinstance(layer, Conv2d) and layer.groups == 1:
            after = only_user(end)
            if after is not None and after.op == "call_module" and len(after.args) == 1 and after.args[0] is end and not after.kwargs:
                m = mods.get(after.target)
                inner = m.inner if isinstance(m, _MaxPool2dNHWC) else m
                if (isinstance(inner, nn.MaxPool2d) and _pair(inner.kernel_size) == (3, 3) and _pair(inner.stride) == (2, 2)
                        and _pair(inner.padding) == (1, 1) and _pair(inner.dilation) == (1, 1) and not inner.ceil_mode
                        and not inner.return_indices):
                    pool, end = m, after
        name = "_fused_" + node.target.replace(".", "_")
        k = 0
        while hasattr(gm, name + (str(k) if k else "")):
            k += 1
        name += str(k) if k else ""
        gm.add_submodule(name, _FusedEpilogue(layer, relu, pool))
        with graph.inserting_before(end):
            args = (node.args[0],) if residual is None else (node.args[0], residual)
            new = graph.call_module(name, args)
        end.replace_all_uses_with(new)
        # erase the replaced chain, consumers first
        chain, cur = [end], end
        while cur is not node:
            cur = cur.args[0] if (cur.args[0] is not residual or not is_add(cur)) else cur.args[1]
            chain.append(cur)
        for n in chain:
            graph.erase_node(n)
        fused += 1
    # a network's head: linear(flatten(avgpool(x), 1)) with a global average pool becomes one call
    for node in list(graph.nodes):
        if node.op != "call_module":
            continue
        layer = mods.get(node.target)
        if not (isinstance(layer, Linear) and layer.compact and getattr(layer, "bn", None) is None and len(node.args) == 1
                and not node.kwargs and isinstance(node.args[0], fx.Node)):
            continue
        fl = node.args[0]
        flat = ((fl.op == "call_function" and fl.target is torch.flatten) or (fl.op == "call_method" and fl.target == "flatten"))
        if not (flat and len(fl.users) == 1 and len(fl.args) >= 1 and isinstance(fl.args[0], fx.Node)
                and (tuple(fl.args[1:]) == (1,) or (len(fl.args) == 1 and dict(fl.kwargs) == {"start_dim": 1}))):
            continue
        pl = fl.args[0]
        pm = mods.get(pl.target) if pl.op == "call_module" else None
        inner = pm.inner if isinstance(pm, _GlobalAvgPoolNHWC) else pm
        if not (isinstance(inner, nn.AdaptiveAvgPool2d) and inner.output_size in (1, (1, 1)) and len(pl.users) == 1
                and len(pl.args) == 1 and not pl.kwargs):
            continue
        name = "_fused_" + node.target.replace(".", "_")
        k = 0
        while hasattr(gm, name + (str(k) if k else "")):
            k += 1
        name += str(k) if k else ""
        gm.add_submodule(name, _FusedHead(pm, layer))
        with graph.inserting_before(node):
            new = graph.call_module(name, (pl.args[0],))
        node.replace_all_uses_with(new)
        for n in (node, fl, pl):
            graph.erase_node(n)
        fused += 1
    graph.lint()
    gm.recompile()
    return gm, fused


class _MaxPool2dNHWC(nn.Module):
    """nn.MaxPool2d for fp16 channels_last GPU tensors (anything else goes to the module it replaced)."""

    def __init__(self, inner: nn.MaxPool2d):
        super().__init__()
        self.inner = inner

    def forward(self, x):
        if x.is_cuda and x.dim() == 4 and x.dtype == torch.float16 and x.is_contiguous(memory_format=torch.channels_last):
            return ops.maxpool2d_nhwc(x, self.inner.kernel_size, self.inner.stride, self.inner.padding)
        return self.inner(x)


class _GlobalAvgPoolNHWC(nn.Module):
    """nn.AdaptiveAvgPool2d(1) for fp16 channels_last GPU tensors (anything else goes to the module it replaced)."""

    def __init__(self, inner: nn.AdaptiveAvgPool2d):
        super().__init__()
        self.inner = inner

    def forward(self, x):
        if x.is_cuda and x.dim() == 4 and x.dtype == torch.float16 and x.is_contiguous(memory_format=torch.channels_last):
            return ops.avgpool_global_nhwc(x, out_dtype=torch.float16).view(x.shape[0], x.shape[1], 1, 1)
        return self.inner(x)


def use_native_pooling(module: nn.Module):
    """Replace the nn.MaxPool2d (no dilation, no ceil_mode, no indices) and nn.AdaptiveAvgPool2d(1) modules
    below `module` by fp16 NHWC kernels of this library; they act only on fp16 channels_last GPU tensors --
    what compact layers hand on after set_compact_output_dtype(torch.float16) -- and defer to the original
    module otherwise. For inference. Returns the qualified names of the replaced modules."""
    done = []
    for pname, parent in list(module.named_modules()):
        if isinstance(parent, (_MaxPool2dNHWC, _GlobalAvgPoolNHWC)):
            continue                                     # already wrapped by an earlier call
        for cname, child in list(parent.named_children()):
            name = (pname + "." if pname else "") + cname
            if (isinstance(child, nn.MaxPool2d) and child.dilation in (1, (1, 1)) and not child.ceil_mode
                    and not child.return_indices):
                setattr(parent, cname, _MaxPool2dNHWC(child))
                done.append(name)
            elif isinstance(child, nn.AdaptiveAvgPool2d) and child.output_size in (1, (1, 1)):
                setattr(parent, cname, _GlobalAvgPoolNHWC(child))
                done.append(name)
    return done


class GraphedForward:
    """A model's inference forward as one HIP graph: record it once for a given input shape, replay it with one launch.
    The compact layers' kernels take 3-30 us each, and a Python loop that launches 20-odd of them per forward spends as
    long on the launches as the GPU on the work (ResNet-18 after fuse_epilogues, batch 64: 0.46 ms per forward from
    Python, 0.43 replayed). The graph holds its own input and output tensors: a call copies the input in and returns the
    output tensor, which the next call overwrites (clone it to keep it). A new input shape or dtype records a new graph.
    For inference only (recorded under torch.no_grad()).

    A recorded graph replays raw device addresses: the layers' kernel-native weight buffers, folded scale / bias
    vectors, the dtype the layers hand on. Every call therefore compares a stamp of the model -- each TMQ layer's
    weight tensor (address, shape, version counter), its native-weight cache, folded BatchNorm and post-scale, and the
    global output-dtype and fp32-prescale switches -- with the one the graphs were recorded under, and records anew
    when it moved (load_state_dict, invalidate_native(), expand_compact_layers, fold_batchnorm,
    set_compact_output_dtype after the recording). What the stamp cannot see -- weights overwritten in place through
    `.data`, submodules swapped, other modules' parameters changed -- needs reset()."""

    def __init__(self, model, warmup: int = 2):
        self.model = model
        self.warmup = int(warmup)
        self._graphs = {}
        self._stamp = None
        self._layers = None

    def reset(self):
        """Forget every recorded graph (and the list of the model's TMQ layers); the next call records again."""
        self._graphs.clear()
        self._stamp = None
        self._layers = None

    def _model_stamp(self):
        if self._layers is None:
            self._layers = [m for m in self.model.modules() if isinstance(m, TMQLayer)]
        # addresses, not object identities: a buffer rebuilt at the address the graph already reads is as good
        def where(t):
            return t.data_ptr() if isinstance(t, torch.Tensor) else 0

        def native(entry):
            held = entry[1] if entry is not None else None
            if isinstance(held, ops.NativeWeights):
                return held.buf.data_ptr()
            if isinstance(held, dict):          # ConvTranspose2d: one sub-kernel per phase of the output grid
                return tuple(v[0].buf.data_ptr() if isinstance(v[0], ops.NativeWeights) else 0 for v in held.values())
            return 0

        return (_compact_out, ops._fp32_prescale) + tuple(
            (m._weight_key(), native(m._native),
             (where(m._fold[0]), where(m._fold[1])) if m._fold is not None else 0,
             where(m._scale_vec[1]) if m._scale_vec is not None else 0, where(getattr(m, "bias", None)),
             m.post_scale_imm, m.compact) for m in self._layers)

    def _record(self, x):
        static_in = x.clone()
        stream = torch.cuda.Stream(device=x.device)
        stream.wait_stream(torch.cuda.current_stream(x.device))
        with torch.cuda.stream(stream), torch.no_grad():
            for _ in range(self.warmup):                 # native weight caches, lazy initialisation: outside the graph
                self.model(static_in)
            stream.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                static_out = self.model(static_in)
        torch.cuda.current_stream(x.device).wait_stream(stream)
        if not isinstance(static_out, torch.Tensor):
            raise RuntimeError("GraphedForward: the model must return one tensor")
        return graph, static_in, static_out

    def __call__(self, x):
        if not (isinstance(x, torch.Tensor) and x.is_cuda):
            raise RuntimeError("GraphedForward: expected one GPU tensor")
        key = (tuple(x.shape), x.dtype, x.device, x.stride())
        stamp = self._model_stamp()
        if stamp != self._stamp:
            self._graphs.clear()                         # recorded against buffers that may be gone
        entry = self._graphs.get(key)
        if entry is None:
            entry = self._graphs[key] = self._record(x)
            self._stamp = self._model_stamp()            # the warm-up built the native-weight caches
        graph, static_in, static_out = entry
        static_in.copy_(x)
        graph.replay()
        return static_out


def expand_compact_layers(module: nn.Module, for_training=False):
    """Expand compact TMQ layers back to fp32 weights in place (tmq/tmq.py:1296-1319)."""
    for name, sub in module.named_children():
        if isinstance(sub, TMQLayer) and hasattr(sub, "tensor_type") and getattr(sub, "original_shape", None) is not None:
            if sub.tensor_type in (TensorType.COMPRESSED_TERNARY_32BIT, TensorType.COMPACT_TERNARY_32BIT):
                if sub._fold is not None:
                    raise RuntimeError("expand_compact_layers: a BatchNorm was folded into this layer (fold_batchnorm); "
                                       "reload the model instead")
                entropy = sub.tensor_type == TensorType.COMPRESSED_TERNARY_32BIT
                full = _b.expand_ternary(sub.weight.data, sub.original_shape, entropy)
                sub.weight = nn.Parameter(full, requires_grad=for_training)
                sub.tensor_type = TensorType.FLOAT_32BIT
                sub.compact = False
                sub._native = None
        expand_compact_layers(sub, for_training)
