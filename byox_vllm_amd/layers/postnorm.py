"""A sublayer with the norm on its OUTPUT, a gate that reads the residual, and an input convolution:

    y = f(x + conv(x)),   x <- x + mult * rms_norm(y * sigmoid(W_r x + b_r)) * w

``GatedPostNorm`` owns w, W_r, b_r and the convolution (a per-channel causal convolution over time whose last
taps - 1 inputs are a request's state, layers/conv.py).  The update of the residual is deferred: ``begin`` first folds
the PREVIOUS sublayer's pending result into the fp32 residual (one launch: gate, norm, scaled add, and a copy of the new
rows in the model dtype for the gate's product), then hands out the sublayer's input and the gate logits; the caller
runs f and passes (y, gate logits, this module) on as the next pending result.  All of it is fp32
(csrc/rowops.hip: nv_gated_postnorm_add); eps sits inside the root."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.conv import CausalConv1d
from byox_vllm_amd.layers.linear import DenseLinear


def fold(x: torch.Tensor, pending, out_dtype=None):
    """Adds a pending sublayer result (y, gate logits or None, its GatedPostNorm[, a bias still to be added to y]) to the
    fp32 residual ``x`` in place;
    -> the new rows in ``out_dtype`` (None: no copy)."""
    if pending is None:
        return kernels.gated_postnorm_add(x, None, None, 0.0, 0.0, out_dtype=out_dtype) if out_dtype is not None else None
    y, logits, norm = pending[:3]
    y_bias = pending[3] if len(pending) > 3 else None          # a bias the sublayer's last product left to be added here
    return kernels.gated_postnorm_add(x, y, norm.weight.data, norm.eps, norm.mult, gate=logits,
                                      gate_bias=norm.gate.bias.data if norm.gate is not None else None,
                                      out_dtype=out_dtype, y_bias=y_bias)


class GatedPostNorm(nn.Module):
    def __init__(self, width: int, eps: float, mult: float = 1.0, taps: int = 0, gated: bool = True):
        super().__init__()
        self.eps, self.mult = float(eps), float(mult)
        self.weight = nn.Parameter(torch.ones(width), requires_grad=False)
        self.gate = DenseLinear(width, width, bias=True) if gated else None
        self.conv = CausalConv1d(width, taps, bias=False, residual=True) if taps else None

    def state_modules(self):
        return [self.conv] if self.conv is not None else []

    def begin(self, x: torch.Tensor, pending):
        """-> (the sublayer's input in the model dtype, fp32 gate logits [T, width] without their bias, or None)."""
        dtype = self.weight.dtype
        rows = fold(x, pending, dtype if (self.gate is not None or self.conv is None) else None)
        logits = kernels.linear(rows, self.gate.weight.data, out_dtype=torch.float32) if self.gate is not None else None
        h = self.conv(x, want_f32=False, want_t=True)[1] if self.conv is not None else rows
        return h, logits
