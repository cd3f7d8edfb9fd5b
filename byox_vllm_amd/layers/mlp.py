"""Feed-forward with one up-projection and an element-wise activation, W_down act(W_up h) (both products with a bias
when ``bias``); the activation runs in the up-projection's epilogue.  ``xielu`` is the activation with two learned numbers p, q:

    z > 0:  softplus(p) z^2 + z / 2;        z <= 0:  (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2

whose coefficients are evaluated once after loading (fp32, on the device) and read by the kernel."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.linear import DenseLinear

UNARY = {"silu": kernels.ACT_SILU, "gelu_tanh": kernels.ACT_GELU_TANH, "xielu": kernels.ACT_XIELU}


class UnaryMLP(nn.Module):
    def __init__(self, width: int, ff: int, act: str, bias: bool = False):
        super().__init__()
        self.act = UNARY[act]
        self.up = DenseLinear(width, ff, bias=bias)
        self.down = DenseLinear(ff, width, bias=bias)
        if act == "xielu":
            self.act_params = nn.Parameter(torch.zeros(2, dtype=torch.float32), requires_grad=False)
            self.act_params.weight_loader = lambda p, t: p.data.copy_(t.reshape(2).to(torch.float32))
        self.coef = None

    def finalize(self) -> None:
        """The activation's coefficients from its stored numbers (softplus in float64, then fp32)."""
        if self.act == kernels.ACT_XIELU:
            sp = torch.nn.functional.softplus(self.act_params.data.to(torch.float64))
            self.coef = torch.stack([sp[0], 0.5 + sp[1]]).to(torch.float32).contiguous()

    def forward(self, h, defer_bias: bool = False):
        """-> fp32 [T, width]; with ``defer_bias`` -> (the down-projection without its bias, that bias or None): a caller
        that adds the bias where it consumes the result keeps the product free of an epilogue."""
        if self.act == kernels.ACT_XIELU and self.coef is None:
            self.finalize()
        hidden = self.up(h, epilogue=kernels.EPI_ACT, act=self.act, gate=self.coef)
        if defer_bias:
            return kernels.linear(hidden, self.down.weight.data, out_dtype=torch.float32), \
                (self.down.bias.data if self.down.bias is not None else None)
        return self.down(hidden, out_dtype=torch.float32)
