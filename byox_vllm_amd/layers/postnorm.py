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
from byox_vllm_amd.utils.context import get_context


def fold(x: torch.Tensor, pending, out_dtype=None, conv=None):
    """Adds a pending sublayer result (y, gate logits or None, its GatedPostNorm[, a bias still to be added to y]) to the
    fp32 residual ``x`` in place; -> the new rows in ``out_dtype`` (None: no copy).  ``conv`` (kernels.gated_postnorm_add):
    the same launch also runs the next sublayer's input convolution -> (rows, x + conv(x))."""
    if pending is None:
        if conv is not None:
            return kernels.gated_postnorm_add(x, None, None, 0.0, 0.0, out_dtype=out_dtype, conv=conv)
        return kernels.gated_postnorm_add(x, None, None, 0.0, 0.0, out_dtype=out_dtype) if out_dtype is not None else None
    y, logits, norm = pending[:3]
    y_bias = pending[3] if len(pending) > 3 else None          # a bias the sublayer's last product left to be added here
    return kernels.gated_postnorm_add(x, y, norm.weight.data, norm.eps, norm.mult, gate=logits,
                                      gate_bias=norm.gate.bias.data if norm.gate is not None else None,
                                      out_dtype=out_dtype, y_bias=y_bias, conv=conv)


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
        ctx = get_context()
        conv = self.conv
        if (conv is not None and ctx.max_seqlen_q == 1
                and kernels.lib().nv_gated_postnorm_add_conv_ok(x.data_ptr(), x.size(1), conv.taps)):
            # one token per request: every row a tap reads is in the request's slot, the folding launch convolves too
            rows, h = fold(x, pending, dtype if self.gate is not None else None,
                           conv=(conv.weight.data, conv.state, ctx.state_slots, ctx.past_lens))
        else:
            rows = fold(x, pending, dtype if (self.gate is not None or conv is None) else None)
            h = conv(x, want_f32=False, want_t=True)[1] if conv is not None else rows
        logits = kernels.linear(rows, self.gate.weight.data, out_dtype=torch.float32) if self.gate is not None else None
        return h, logits
