"""Mixers built on a matrix memory with one decay per head and token (csrc/memory.hip): per head a state S [dim, vdim],

    S_t = keep_t S_(t-1) + take_t k_t v_t^T,   o_t = S_t^T q_t.

``LightningAttention``: keep is a constant of the head (``decay``), take is 1, and q, k, v pass through SiLU; the
concatenated heads are RMS-normed TOGETHER (plain weight), multiplied by sigmoid(W_g h) and projected.

``MLSTM`` (the matrix memory of xLSTM, Beck et al.): per head a log input gate i = cap tanh(z_i / cap) and a log forget
gate f = logsigmoid(cap tanh(z_f / cap)), z = W h + b, stabilised by a running maximum m_t = max(f + m_(t-1), i) that starts
at 0: keep = exp(f + m_(t-1) - m_t), take = exp(i - m_t); a normaliser n_t follows the same recurrence with k alone and
o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6) with q = W_q h / sqrt(dim).  EACH head's o is divided by its own
root mean square; then weight over all heads, sigmoid(W_g h), projection.

Both read one merged input projection (q | k | v | g [| i | f], then the rows of ``riders``: other consumers of the same
input, such as a router beside the mixer) and leave it in fp32: activations, gates, the
recurrence, the norm and the output gate are fp32.  What a request keeps between steps lives in fp32 slots that the
engine's StateSlotManager hands out; a request's first tokens start from zero instead of reading the slot.  A mixer whose
layer runs several times per token (a looped span of layers) keeps one state per run: ``runs`` holders, each bound to
its own pool by the runner."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.linear import DenseLinear
from byox_vllm_amd.utils.context import get_context


class MemoryRun:
    """The state of one run of a mixer: fp32 [slots, heads, numbers per head], bound by the runner."""

    def __init__(self, heads: int, per_head: int):
        self.shape = (heads, per_head)
        self.state = torch.tensor([])

    def state_spec(self) -> dict:
        return {"shape": self.shape}


class _MatrixMemoryMixer(nn.Module):
    mode = kernels.MEM_CONST
    extra_shards: tuple = ()

    def __init__(self, width: int, heads: int, dim: int, vdim: int, eps: float, runs: int = 1, riders: dict | None = None):
        super().__init__()
        self.heads, self.dim, self.vdim, self.eps = heads, dim, vdim, eps
        shards = {"q": heads * dim, "k": heads * dim, "v": heads * vdim, "g": heads * vdim}
        shards.update({name: heads for name in self.extra_shards})
        shards.update(riders or {})               # rows of other consumers of the same input (a router)
        self.inp = DenseLinear(width, bias=bool(self.extra_shards), shards=shards)
        if self.inp.bias is not None:
            self.inp.bias.data.zero_()            # only the gate rows have a bias; the others keep zero
            self.inp.bias.keep_init = True        # ... also under random initialisation
        self.at = {name: self.inp.offset(name) for name in shards}
        self.norm = nn.Parameter(torch.ones(heads * vdim), requires_grad=False)
        self.o = DenseLinear(heads * vdim, width)
        per_head = kernels.matrix_memory_state_size(self.mode, dim, vdim)
        self.runs = [MemoryRun(heads, per_head) for _ in range(runs)]

    def state_modules(self):
        return list(self.runs)

    def _memory(self, proj, state, ctx):
        raise NotImplementedError

    norm_groups = 1

    def project(self, h: torch.Tensor) -> torch.Tensor:
        """The merged input projection, fp32 [T, q | k | v | g | ...]; ``rider(proj, name)`` is a rider's slice of it."""
        return kernels.linear(h, self.inp.weight.data, out_dtype=torch.float32)

    def rider(self, proj: torch.Tensor, name: str) -> torch.Tensor:
        at, rows = self.inp.row_of[name]
        return proj[:, at:at + rows]

    def forward(self, h: torch.Tensor, run: int = 0, positions=None, proj: torch.Tensor | None = None) -> torch.Tensor:
        ctx = get_context()
        if proj is None:
            proj = self.project(h)
        o = self._memory(proj, self.runs[run].state, ctx)
        g = self.at["g"]
        y = kernels.group_rms_norm_f32(o, self.norm.data, self.norm_groups, self.eps,
                                       gate=proj[:, g:g + self.heads * self.vdim])
        return self.o(y, out_dtype=torch.float32)


class LightningAttention(_MatrixMemoryMixer):
    mode = kernels.MEM_CONST

    def __init__(self, width: int, heads: int, dim: int, vdim: int, decay, eps: float, runs: int = 1, riders=None):
        super().__init__(width, heads, dim, vdim, eps, runs, riders)
        assert len(decay) == heads, f"{len(decay)} decays for {heads} heads"
        self.register_buffer("decay", torch.tensor([float(a) for a in decay], dtype=torch.float32), persistent=False)

    def _memory(self, proj, state, ctx):
        return kernels.matrix_memory(proj, (self.at["q"], self.at["k"], self.at["v"]), state, ctx.cu_seqlens_q,
                                     ctx.past_lens, ctx.state_slots, self.heads, self.dim, self.vdim, self.mode,
                                     decay=self.decay, silu=True)


class MLSTM(_MatrixMemoryMixer):
    mode = kernels.MEM_EXPGATE
    extra_shards = ("i", "f")

    def __init__(self, width: int, heads: int, dim: int, vdim: int, gate_cap: float, eps: float, runs: int = 1,
                 riders=None):
        super().__init__(width, heads, dim, vdim, eps, runs, riders)
        self.gate_cap = float(gate_cap)
        self.norm_groups = heads

    def _memory(self, proj, state, ctx):
        return kernels.matrix_memory(proj, (self.at["q"], self.at["k"], self.at["v"]), state, ctx.cu_seqlens_q,
                                     ctx.past_lens, ctx.state_slots, self.heads, self.dim, self.vdim, self.mode,
                                     bias=self.inp.bias.data, gate_offsets=(self.at["i"], self.at["f"]),
                                     cap=self.gate_cap, q_scale=self.dim ** -0.5)
