"""Minimal gated recurrent unit (minGRU): a gated recurrence whose gates read the current token only, so a prompt is
a composition of affine maps of the state:

    z = sigmoid(W_z h + b_z),   u = W_x h + b_x,   c(u) = u + 1/2 for u >= 0, sigmoid(u) for u < 0
    S_t = (1 - z) S_(t-1) + z c(u),   y = W_o (S_t * silu(W_g h))

The state S (fp32 [width], zero before a request's first token) lives in a request's state slot.  z | x | g are one
merged projection left in fp32 (its biases are added where it is consumed); gates, candidate and recurrence are fp32
(csrc/scan.hip: nv_mingru_scan)."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.linear import DenseLinear
from byox_vllm_amd.utils.context import get_context


class MinGRU(nn.Module):
    def __init__(self, width: int, channels: int):
        super().__init__()
        self.channels = channels
        self.inp = DenseLinear(width, shards={"z": channels, "x": channels, "g": channels})
        self.z_bias = nn.Parameter(torch.zeros(channels), requires_grad=False)
        self.x_bias = nn.Parameter(torch.zeros(channels), requires_grad=False)
        self.o = DenseLinear(channels, width)
        self.state = torch.tensor([])          # fp32 [slots, channels], bound by the runner

    def state_spec(self) -> dict:
        return {"shape": (self.channels,)}

    def state_modules(self):
        return [self]

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        C = self.channels
        proj = self.inp(h, out_dtype=torch.float32)
        gated = torch.empty(h.size(0), C, dtype=h.dtype, device=h.device)
        kernels.mingru_scan(proj, (0, C, 2 * C), self.z_bias.data, self.x_bias.data, self.state, ctx.cu_seqlens_q,
                            ctx.past_lens, ctx.state_slots, C, gated)
        return self.o(gated, out_dtype=torch.float32)
