"""Feed-forward blocks on nv_linear: the gated unit W_down(act(W_gate h) * (W_up h)) as two launches (gate and up rows
share one product whose epilogue applies the activation and the multiplication), and a mixture of such units.

Mixture: fp32 router logits, the ``top`` largest per token, softmax over the chosen logits only; the (token, choice)
pairs are ordered by expert on the device, the experts' two products run as grouped launches over the gathered rows
(one weight per group, no host synchronisation: the grid covers the worst case and empty tiles leave at once), and the
rows are summed per token in the order of its choices.  An optional shared expert runs for every token and is added
multiplied by sigmoid(w_sg . h), one number per token; its gate row rides in the router's product.

Variants a design may choose: ``route="all"`` takes the softmax over every expert and divides the chosen scores by their
sum (+ 1e-20); the activation ``"clamped"`` is the unit g sigmoid(1.702 g) (u + 1) with g = min(gate, limit) and
u = clamp(up, -limit, limit); ``forward(h, add)`` folds another fp32 result of the same rows (a mixer that runs beside
the feed-forward) into the combining launch; with ``own_router=False`` the layer has no router matrix and takes fp32
logits from the caller, whose own projection of the same rows carries the router's rows (one launch and one read of
the input fewer)."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.linear import DenseLinear

ACTIVATIONS = {"silu": kernels.ACT_SILU, "gelu_tanh": kernels.ACT_GELU_TANH, "clamped": kernels.GLU_CLAMPED}
ROUTES = {"chosen": kernels.ROUTE_CHOSEN, "all": kernels.ROUTE_ALL}


class GatedMLP(nn.Module):
    def __init__(self, width: int, ff: int, act: str):
        super().__init__()
        self.act = ACTIVATIONS[act]
        self.gate_up = DenseLinear(width, shards={"gate": ff, "up": ff})
        self.down = DenseLinear(ff, width)

    def forward(self, h):
        hidden = self.gate_up(h, epilogue=kernels.EPI_GLU, act=self.act)
        return self.down(hidden, out_dtype=torch.float32)


class MixtureOfExperts(nn.Module):
    def __init__(self, width: int, experts: int, top: int, ff: int, act: str = "silu", shared_ff: int | None = None,
                 route: str = "chosen", limit: float = 0.0, own_router: bool = True):
        super().__init__()
        self.experts, self.top, self.ff, self.width, self.act = experts, top, ff, width, ACTIVATIONS[act]
        self.route, self.limit = ROUTES[route], float(limit)
        assert act != "clamped" or self.limit > 0.0
        shards = {"router": experts}
        if shared_ff:
            shards["sg"] = 1
        assert own_router or not shared_ff
        self.router = DenseLinear(width, shards=shards) if own_router else None
        self.gate_up = nn.Parameter(torch.empty(experts, 2 * ff, width), requires_grad=False)
        self.down = nn.Parameter(torch.empty(experts, width, ff), requires_grad=False)
        self.gate_up.weight_loader = self._load_gate_up
        self.down.weight_loader = lambda p, t, e: p.data[e].copy_(t)
        self.shared = GatedMLP(width, shared_ff, act) if shared_ff else None

    def _load_gate_up(self, param, tensor, shard):
        e, part = shard
        at = 0 if part == "gate" else self.ff
        param.data[e, at: at + self.ff].copy_(tensor)

    def forward(self, h, add=None, logits=None):
        T, E, top = h.size(0), self.experts, self.top
        if logits is None:
            logits = self.router(h, out_dtype=torch.float32)
        assert logits.dtype == torch.float32 and logits.shape == (T, E + (1 if self.shared is not None else 0))
        idx, weights = kernels.moe_route(logits, E, top, self.route)
        offsets, sorted_token, slot_of = kernels.moe_sort(idx, E)
        hidden = kernels.linear(h, self.gate_up.data, rows=T * top, a_rows=sorted_token, batch=E,
                                w_batch_stride=2 * self.ff * self.width, group_offsets=offsets, max_group_rows=T,
                                epilogue=kernels.EPI_GLU, act=self.act, cap=self.limit)
        y = kernels.linear(hidden, self.down.data, out_dtype=torch.float32, rows=T * top, batch=E,
                           w_batch_stride=self.width * self.ff, group_offsets=offsets, max_group_rows=T)
        if self.shared is None:
            return kernels.moe_combine(y, slot_of, weights, add)
        assert add is None, "a shared expert and an addend share one input of the combining launch"
        return kernels.moe_combine(y, slot_of, weights, self.shared(h), logits[:, E:])
