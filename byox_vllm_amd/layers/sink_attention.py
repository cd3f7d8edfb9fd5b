"""Causal softmax attention with grouped key/value heads whose VALUES ARE THE KEYS, a sink in the softmax, a query
temperature that grows with the position, and a sigmoid output gate:

    q = (W_q h + b_q) * (1 + coef ln(floor((p + 1) / every) + 1)),   k = W_k h + b_k,   v = k
    w_ij = exp(q_i . k_j * scale) / (exp(sink_h) + sum_(j' <= i) exp(q_i . k_j' * scale))
    y = W_o (concat_h(sum_j w_ij k_j) * sigmoid(W_g h)) + b_o

The sink is one learned logit per query head that takes part in the normalisation only: nothing is attended to through
it, and the score scale does not apply to it.  There is no rotation; positions enter through the temperature alone.  Cache rows hold the keys of the G
key/value heads, [G * dim] per token in the model dtype, in pages of the engine's BlockManager, and are read twice (as
keys and as values).  Scores, softmax, sink and gate are fp32 (csrc/window_attn.hip: nv_qk_store, nv_paged_softmax_attn).
q | k | g (and the rows of ``riders``: other consumers of the same input, such as a router beside the mixer) come from
one merged projection that is left in fp32; its biases are added where it is consumed.  A mixer
whose layer runs several times per token keeps one cache per run."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.linear import DenseLinear
from byox_vllm_amd.utils.context import get_context


class CacheRun:
    """The paged cache of one run of a mixer: [pages * block_size, width] in the model dtype, bound by the runner."""

    def __init__(self, width: int):
        self.width = width
        self.cache = torch.tensor([])
        self.block_size = 0

    def page_spec(self) -> dict:
        return {"width": self.width}


class SinkAttention(nn.Module):
    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, scale: float, temp_coef: float = 0.0,
                 temp_every: int = 0, runs: int = 1, riders: dict | None = None):
        super().__init__()
        assert heads % kv_heads == 0
        self.heads, self.kv_heads, self.dim, self.scale = heads, kv_heads, dim, float(scale)
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        shards = {"q": heads * dim, "k": kv_heads * dim, "g": heads * dim}
        shards.update(riders or {})               # rows of other consumers of the same input (a router)
        self.inp = DenseLinear(width, bias=True, shards=shards)
        self.inp.bias.data.zero_()                # the gate rows have no bias
        self.at = {name: self.inp.offset(name) for name in shards}
        self.sink = nn.Parameter(torch.zeros(heads), requires_grad=False)
        self.o = DenseLinear(heads * dim, width, bias=True)
        self.runs = [CacheRun(kv_heads * dim) for _ in range(runs)]

    def project(self, h: torch.Tensor) -> torch.Tensor:
        """The merged input projection, fp32 [T, q | k | g | ...], biases not yet added."""
        return kernels.linear(h, self.inp.weight.data, out_dtype=torch.float32)

    def rider(self, proj: torch.Tensor, name: str) -> torch.Tensor:
        at, rows = self.inp.row_of[name]
        return proj[:, at:at + rows]

    def forward(self, h: torch.Tensor, run: int = 0, positions=None, proj: torch.Tensor | None = None) -> torch.Tensor:
        ctx = get_context()
        own = self.runs[run]
        if proj is None:
            proj = self.project(h)
        q = kernels.qk_store(proj, (self.at["q"], self.at["k"]), positions, self.scale, ctx.slot_mapping, own.cache,
                             self.heads, self.kv_heads, self.dim, bias=self.inp.bias.data, temp_coef=self.temp_coef,
                             temp_every=self.temp_every)
        out = torch.empty(h.size(0), self.heads * self.dim, dtype=h.dtype, device=h.device)
        g = self.at["g"]
        kernels.paged_softmax_attn(q, own.cache, ctx.block_tables, ctx.cu_seqlens_q, ctx.past_lens, ctx.seq_of_token,
                                   ctx.max_seqlen_q, self.heads, self.kv_heads, self.dim, self.dim, own.block_size, out,
                                   values_are_keys=True, sink=self.sink.data, gate=proj[:, g:g + self.heads * self.dim])
        return self.o(out, out_dtype=torch.float32)
