"""Softmax attention with grouped key/value heads inside chunks of the sequence, over a paged cache:

    q, k, v = conv(W_q h), conv(W_k h), conv(W_v h)         a short causal convolution per channel (layers/conv.py)
    q, k    = rms_norm(q) * w_q, rms_norm(k) * w_k          ONE norm over all heads of a token, a weight per number
    q, k    = rotate(q), rotate(k)                          the first rot_dims numbers of every head, i with i + dims/2
    v       = (1 - lam) v + lam v_first                     values of the first layer that shares its values (optional)
    s_ij    = q_i . k_j * scale  for j <= i with floor(i / chunk) == floor(j / chunk)   (chunk 0: every j <= i)
    y       = W_o concat_h(sigmoid(W_g h)[h] * sum_j softmax(s)_ij v_j)                 one gate number per head

Chunks are counted from a sequence's first position, wherever a prompt was cut for processing.  Cache rows
[k: G * dim | v: G * vdim] (the blended values) live in pages of the engine's BlockManager in the model dtype; the last
taps - 1 projected rows of q | k | v are a request's state.  q | k | v | g are one merged projection left in fp32;
convolution, norm, rotation, scores and softmax are fp32 (csrc/scan.hip, csrc/window_attn.hip)."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.conv import CausalConv1d
from byox_vllm_amd.layers.linear import DenseLinear
from byox_vllm_amd.layers.rotary_embedding import scaled_inv_freq
from byox_vllm_amd.utils.context import get_context


class ChunkedAttention(nn.Module):
    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, chunk: int, taps: int,
                 rot_dims: int, rot_base: float, rot_scaling: dict | None, eps: float, qk_norm: bool = True,
                 v_source: "ChunkedAttention | None" = None, keeps_values: bool = False):
        super().__init__()
        assert heads % kv_heads == 0 and rot_dims % 2 == 0 and rot_dims <= dim
        self.heads, self.kv_heads, self.dim, self.vdim = heads, kv_heads, dim, vdim
        self.scale, self.chunk, self.rot_dims, self.eps = float(scale), int(chunk), int(rot_dims), eps
        sizes = {"q": heads * dim, "k": kv_heads * dim, "v": kv_heads * vdim}
        self.channels = sum(sizes.values())
        self.inp = DenseLinear(width, shards=dict(sizes, g=heads))
        self.conv = CausalConv1d(self.channels, taps, bias=False, shards=sizes) if taps else None
        if qk_norm:
            self.q_norm = nn.Parameter(torch.ones(heads * dim), requires_grad=False)
            self.k_norm = nn.Parameter(torch.ones(kv_heads * dim), requires_grad=False)
        else:
            self.q_norm = self.k_norm = None
        # lam of the value blend; a layer that only lends its values keeps the number a checkpoint stores for it unused
        self.vmix = nn.Parameter(torch.zeros(1), requires_grad=False) if (v_source is not None or keeps_values) else None
        if self.vmix is not None:
            self.vmix.weight_loader = lambda p, t: p.data.copy_(t.reshape(1))
        object.__setattr__(self, "v_source", v_source)       # a reference, not a submodule
        if v_source is not None:
            assert v_source.kv_heads * v_source.vdim == kv_heads * vdim, "blended values have one size"
        self.keeps_values = keeps_values
        self.values = None                      # fp32 [T, G * vdim] of the current step, for the layers that blend them in
        self.o = DenseLinear(heads * vdim, width)
        if rot_dims:
            inv_freq, self.magnitude = scaled_inv_freq(rot_dims, rot_base, rot_scaling)
            self.register_buffer("inv_freq", inv_freq.to(torch.float32), persistent=False)
        else:
            self.inv_freq, self.magnitude = None, 1.0
        self.cache = torch.tensor([])          # [pages * block_size, G * (dim + vdim)], bound by the runner
        self.block_size = 0

    def page_spec(self) -> dict:
        return {"width": self.kv_heads * (self.dim + self.vdim)}

    def state_modules(self):
        return [self.conv] if self.conv is not None else []

    def forward(self, h: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        H, G, d, dv = self.heads, self.kv_heads, self.dim, self.vdim
        proj = self.inp(h, out_dtype=torch.float32)
        qkv = self.conv(proj[:, :self.channels])[0] if self.conv is not None else proj
        v_at = (H + G) * d
        if self.keeps_values:
            self.values = qkv[:, v_at:v_at + G * dv]
        inv_freq = self.inv_freq
        if inv_freq is not None and inv_freq.dtype != torch.float32:
            inv_freq = inv_freq.float()
        src = self.v_source
        q = kernels.qk_rotate_store(qkv, (0, H * d, v_at), positions, self.scale, ctx.slot_mapping, self.cache, H, G, d, dv,
                                    q_norm=self.q_norm.data if self.q_norm is not None else None,
                                    k_norm=self.k_norm.data if self.k_norm is not None else None, eps=self.eps,
                                    inv_freq=inv_freq, rot_dims=self.rot_dims, mscale=self.magnitude,
                                    v_first=src.values if src is not None else None,
                                    vmix=self.vmix.data if src is not None else None)
        out = torch.empty(h.size(0), H * dv, dtype=h.dtype, device=h.device)
        g = self.inp.offset("g")
        kernels.paged_softmax_attn(q, self.cache, ctx.block_tables, ctx.cu_seqlens_q, ctx.past_lens, ctx.seq_of_token,
                                   ctx.max_seqlen_q, H, G, d, dv, self.block_size, out, chunk=self.chunk,
                                   gate=proj[:, g:g + H], gate_per_head=True)
        return self.o(out, out_dtype=torch.float32)
