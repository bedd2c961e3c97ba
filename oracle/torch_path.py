"""TEST INFRASTRUCTURE ONLY -- op-for-op torch restatement of the reference's CPU path.

Nothing in the shipped package imports this module. It issues the same sequence of torch CPU
ops, in the same association, as the CPU branches of the reference, so on CPU tensors it is
bit-identical to them by construction and costs what they cost (it is the timed "port" CPU
baseline of bench.py). It is a second, independent restatement next to oracle/tmq_oracle.c;
tests require the two to agree bit for bit.

Each function cites the reference lines it follows (paths relative to the reference root).
"""
import torch


# --- SoftStep helpers, tmq/tmq.py:353-391 -------------------------------------------------
def sigmoid(inp: torch.Tensor) -> torch.Tensor:
    """tmq/tmq.py:353-360"""
    x = torch.clamp(inp, -3.0, 3.0)
    x2 = x * x
    return x * (x2 + 27.0) / (27.0 + x2 * 9.0)


def dsigmoid(inp: torch.Tensor) -> torch.Tensor:
    """tmq/tmq.py:363-370"""
    x = torch.clamp(inp, -3.0, 3.0)
    x2 = x * x
    return ((x2 - 9) * (x2 - 9)) / (9 * (3 + x2) * (3 + x2))


def d2sigmoid(inp: torch.Tensor) -> torch.Tensor:
    """tmq/tmq.py:373-381"""
    x = torch.clamp(inp, -3.0, 3.0)
    x2 = x * x
    a = (x2 + 3)
    return 16 * x * (x2 - 9) / (3 * a * a * a)


def scalar_sigmoid(inp: float) -> float:
    """tmq/tmq.py:384-391"""
    x = min(3.0, max(-3.0, inp))
    x2 = x * x
    return x * (x2 + 27.0) / (27.0 + x2 * 9.0)


# --- SoftStep, tmq/tmq.py:404-438 ---------------------------------------------------------
def softstep_fwd(weight: torch.Tensor, digamma: float) -> torch.Tensor:
    """CPU branch of SoftStep.forward, tmq/tmq.py:417-419"""
    fw = torch.floor(weight)
    arg = digamma * (weight - fw) - digamma / 2.0
    return sigmoid(arg) / (2.0 * scalar_sigmoid(digamma / 2.0)) + 0.5 + fw


def softstep_bwd(weight: torch.Tensor, digamma: float, scale: float, grad_output: torch.Tensor) -> torch.Tensor:
    """CPU branch of SoftStep.backward, tmq/tmq.py:434-438"""
    frac = weight - torch.floor(weight)
    arg = digamma * frac - digamma / 2
    grad = digamma * dsigmoid(arg) / (2.0 * scalar_sigmoid(digamma / 2.0))
    return scale * grad_output * grad


# --- SoftStepDerivative, tmq/tmq.py:456-493 -----------------------------------------------
def deriv_fwd(weight: torch.Tensor, digamma: float, strength: float) -> torch.Tensor:
    """CPU branch of SoftStepDerivative.forward, tmq/tmq.py:469-473"""
    fw = torch.floor(weight)
    frac = weight - fw
    arg = digamma * frac - digamma / 2
    return strength * digamma * dsigmoid(arg) / (2.0 * scalar_sigmoid(digamma / 2.0))


def deriv_bwd(weight: torch.Tensor, digamma: float, strength: float, grad_output: torch.Tensor) -> torch.Tensor:
    """CPU branch of SoftStepDerivative.backward, tmq/tmq.py:488-493"""
    fw = torch.floor(weight)
    frac = weight - fw
    arg = digamma * frac - digamma / 2
    grad = strength * digamma * digamma * d2sigmoid(arg) / (2.0 * scalar_sigmoid(digamma / 2.0))
    return grad_output * grad


# --- SoftStep.map / dmap, ternarise, clamp ------------------------------------------------
def softstep_map(weight: torch.Tensor, digamma: float) -> torch.Tensor:
    """SoftStep.map, tmq/tmq.py:335-338"""
    fw = torch.floor(weight)
    arg = digamma * weight - digamma * fw - digamma / 2.0
    return sigmoid(arg) / (2.0 * scalar_sigmoid(digamma / 2)) + 0.5 + fw


def softstep_dmap(weight: torch.Tensor, digamma: float) -> torch.Tensor:
    """SoftStep.dmap, tmq/tmq.py:348-350"""
    arg = weight * digamma - digamma * torch.floor(weight) - digamma / 2
    return digamma * dsigmoid(arg) / (2.0 * scalar_sigmoid(digamma / 2))


def ternarize(weight: torch.Tensor, digamma: float) -> torch.Tensor:
    """QuantizationControl.quantize, tmq/tmq.py:293-295"""
    return torch.round(softstep_map(weight, digamma))


def clamp(weight: torch.Tensor, lo: float, hi: float) -> torch.Tensor:
    """Linear.clamp / Conv2d.clamp, tmq/tmq.py:696, 879"""
    return torch.clamp(weight, lo, hi)


def quantization_loss(weights, strength: float, sharpness: float):
    """QuantizationControl.quantization_loss + per-layer mean, tmq/tmq.py:298-310, 698-699."""
    total = None
    for w in weights:
        nloss = torch.mean(deriv_fwd(w, sharpness, strength))
        total = nloss if total is None else total + nloss
    return total


def fused_step(weight, grad_output, digamma, sharpness, strength, gl, lo, hi):
    """One QAT pass over a flat tensor with the reference's separate CPU op chains:
    forward, quantization-loss integrand + mean, both backward contributions summed the way
    autograd accumulates them, and the post-step clamp. This is what bench.py times as the
    CPU baseline for the fused GPU pass."""
    y = softstep_fwd(weight, digamma)
    q = deriv_fwd(weight, sharpness, strength)
    loss = torch.mean(q)
    t1 = softstep_bwd(weight, digamma, 1.0, grad_output)
    t2 = deriv_bwd(weight, sharpness, strength, torch.full_like(weight, gl))
    dw = t1 + t2
    wc = clamp(weight, lo, hi)
    return y, dw, wc, loss
