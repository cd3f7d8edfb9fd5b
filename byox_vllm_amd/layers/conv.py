"""Short causal convolution per channel, out[t] = act(b + sum_j w[:, j] x[t - (taps - 1 - j)]), with zeros before a
sequence's start.  The last taps - 1 inputs are a request's state (fp32 [taps - 1, channels] in a state slot), so a
prompt may arrive in pieces of any size and decoding continues from it (csrc/scan.hip).  ``residual``: the token's own
input is added, out[t] = x[t] + conv(x)[t] (a sublayer that reads its input through such a convolution).  ``shards``
names row blocks of the weight that a checkpoint stores as separate tensors (one convolution over the concatenated
channels of several projections)."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.utils.context import get_context


class CausalConv1d(nn.Module):
    def __init__(self, channels: int, taps: int, activation: str | None = None, bias: bool = True,
                 residual: bool = False, shards: dict[str, int] | None = None):
        super().__init__()
        assert not (residual and activation)
        self.channels, self.taps = channels, taps
        self.act = 2 if residual else {None: 0, "silu": 1}[activation]
        self.weight = nn.Parameter(torch.empty(channels, taps), requires_grad=False)
        if bias:
            self.bias = nn.Parameter(torch.zeros(channels), requires_grad=False)
        else:
            self.register_parameter("bias", None)
        self.row_of, at = {}, 0
        for name, rows in (shards or {}).items():
            self.row_of[name] = (at, rows)
            at += rows
        assert not shards or at == channels
        self.weight.weight_loader = self._load
        self.state = torch.tensor([])          # fp32 [slots, taps - 1, channels], bound by the runner

    def _load(self, param, tensor, shard: str | None = None):
        at, rows = self.row_of[shard] if shard is not None else (0, self.channels)
        assert tensor.shape == (rows, self.taps), f"{tuple(tensor.shape)} for {rows} channels of {self.taps} taps"
        param.data[at:at + rows].copy_(tensor)

    def state_spec(self) -> dict:
        return {"shape": (self.taps - 1, self.channels)}

    def forward(self, x: torch.Tensor, want_f32: bool = True, want_t: bool = False, x_bias: torch.Tensor | None = None):
        """``x`` fp32 [T, channels] (a column slice of a wider buffer is fine; ``x_bias`` is added to it first)
        -> (fp32 rows, rows in the model dtype)."""
        ctx = get_context()
        return kernels.causal_conv(x, self.weight.data, self.bias.data if self.bias is not None else None, self.state,
                                   ctx.cu_seqlens_q, ctx.past_lens,
                                   ctx.state_slots, ctx.seq_of_token, act=self.act, want_f32=want_f32, want_t=want_t, x_bias=x_bias)
