"""Latent attention mixer: keys and values of all heads are up-projections of one low-rank latent per token, so the
cache holds per token only that latent c (kv_rank numbers, RMS-normed) and one rotated key part (rot_dim numbers)
shared by the heads (the multi-head latent attention of DeepSeek-V2).  Scores of head h:

    s = (q_nope[h] . (W_uk[h] c) + q_rot[h] . k_rot) * scale

The up-projections never run over cached tokens: W_uk[h] is folded into the query (q_abs[h] = W_uk[h]^T q_nope[h], one
small product per head and step token) and W_uv[h] is applied to the attention-weighted sum of latents.  Attention is
then multi-query attention over rows [c | k_rot] with a sliding window: position i sees j with 0 <= i - j < window
(window 0: every j <= i).  Queries go through a latent of their own (RMS-normed).  The output gate sigmoid(W_g h) has
one number per head (``gate`` "head") or one per output number (``gate`` "channel", W_g [heads * vdim, width]).  The
rotated parts turn dimension i with i + dims/2, or with ``interleaved`` dimension 2i with 2i + 1.

A layer built with ``kv_source`` has no key/value down-projection: it reads the cache rows another layer wrote in the
same step (same kv_rank, rot_dim and rotation), with its own W_uk, W_uv, queries and window.

Cache rows live in pages of the engine's BlockManager ([pages * block_size, kv_rank + rot_dim] in the model dtype);
scores, softmax and the weighted sum are fp32 (csrc/latent_attn.hip)."""

import torch
from torch import nn

from byox_vllm_amd import kernels
from byox_vllm_amd.layers.linear import DenseLinear
from byox_vllm_amd.layers.rotary_embedding import scaled_inv_freq
from byox_vllm_amd.utils.context import get_context


class LatentAttention(nn.Module):
    def __init__(self, width: int, heads: int, dim: int, rot_dim: int, vdim: int, q_rank: int, kv_rank: int, scale: float,
                 window: int, rot_dims: int, rot_base: float, rot_scaling: dict | None, eps: float,
                 kv_source: "LatentAttention | None" = None, interleaved: bool = False, gate: str = "head"):
        super().__init__()
        self.heads, self.dim, self.rot_dim, self.vdim = heads, dim, rot_dim, vdim
        self.q_rank, self.kv_rank, self.scale, self.window, self.rot_dims, self.eps = q_rank, kv_rank, scale, window, rot_dims, eps
        assert rot_dims <= rot_dim and rot_dims % 2 == 0 and gate in ("head", "channel")
        self.interleaved, self.gate_per_number = bool(interleaved), gate == "channel"
        self.own_kv = kv_source is None
        object.__setattr__(self, "kv_source", kv_source)      # a reference, not a submodule
        if kv_source is not None:
            assert (kv_source.kv_rank, kv_source.rot_dim, kv_source.own_kv) == (kv_rank, rot_dim, True)
        shards = {"dq": q_rank}
        if self.own_kv:
            shards["dkv"] = kv_rank + rot_dim
        shards["g"] = heads * vdim if self.gate_per_number else heads
        self.down = DenseLinear(width, shards=shards)
        self.dq_norm = nn.Parameter(torch.ones(q_rank), requires_grad=False)
        self.uq = DenseLinear(q_rank, heads * (dim + rot_dim))
        if self.own_kv:
            self.dkv_norm = nn.Parameter(torch.ones(kv_rank), requires_grad=False)
        # W_uk per head, stored transposed ([heads, kv_rank, dim]) so that folding it into the query is a plain product
        self.uk_t = nn.Parameter(torch.empty(heads, kv_rank, dim), requires_grad=False)
        self.uk_t.weight_loader = lambda p, t: p.data.copy_(t.view(heads, dim, kv_rank).transpose(1, 2))
        self.uv = DenseLinear(kv_rank, heads * vdim)
        self.o = DenseLinear(heads * vdim, width)
        inv_freq, self.magnitude = scaled_inv_freq(rot_dims, rot_base, rot_scaling)
        self.register_buffer("inv_freq", inv_freq.to(torch.float32), persistent=False)
        self.cache = torch.tensor([])          # [pages * block_size, kv_rank + rot_dim], bound by the runner
        self.block_size = 0

    def page_spec(self) -> dict | None:
        return {"width": self.kv_rank + self.rot_dim} if self.own_kv else None

    def forward(self, h: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        ctx = get_context()
        H, d, r, R = self.heads, self.dim, self.rot_dim, self.kv_rank
        inv_freq = self.inv_freq if self.inv_freq.dtype == torch.float32 else self.inv_freq.float()
        dn = self.down(h, out_dtype=torch.float32)
        q = self.uq(kernels.rms_norm_f32(dn[:, :self.q_rank], self.dq_norm.data, self.eps))
        if self.own_kv:
            at = self.down.offset("dkv")
            kernels.latent_kv_store(dn[:, at: at + R + r], self.dkv_norm.data, positions, inv_freq, self.magnitude,
                                    ctx.slot_mapping, self.cache, R, r, self.rot_dims, self.eps, self.interleaved)
        src = self if self.own_kv else self.kv_source
        T = h.size(0)
        if self._expands(ctx, h):
            return self.o(self._expanded(ctx, src, q, dn, positions, inv_freq), out_dtype=torch.float32)
        qa = torch.empty(T, H * (R + r), dtype=torch.float32, device=h.device)
        kernels.linear(q, self.uk_t.data, out=qa, out_dtype=torch.float32, batch=H, a_batch_stride=d + r,
                       w_batch_stride=R * d, out_batch_stride=R + r, n=R)
        kernels.latent_q_rope(q, positions, inv_freq, self.magnitude, qa, H, d, r, self.rot_dims, R, self.interleaved)
        mix = kernels.latent_attn(qa, src.cache, ctx.block_tables, ctx.cu_seqlens_q, ctx.past_lens, ctx.seq_of_token,
                                  H, R, r, src.block_size, self.window, self.scale, max_q=ctx.max_seqlen_q)
        o = kernels.linear(mix, self.uv.weight.data, batch=H, a_batch_stride=R, w_batch_stride=self.vdim * R,
                           out_batch_stride=self.vdim, n=self.vdim, epilogue=kernels.EPI_ROW_GATE,
                           act=kernels.GATE_PER_NUMBER if self.gate_per_number else 0,
                           gate=dn[:, self.down.offset("g"):], gate_stride=dn.stride(0))
        return self.o(o, out_dtype=torch.float32)

    # ------------------------------------------------------------------ long prompt portions
    EXPAND_FROM = 32          # tokens of one request in a step from which the expanded form is taken

    def _expands(self, ctx, h) -> bool:
        """Steps that bring a long portion write out keys and values of every head for the contexts of the step's
        requests (one product over the gathered latents) and run ordinary paged attention over them: a tile of keys
        then serves 64 tokens of a head instead of one token's heads.  16-bit caches with 16-byte-aligned heads only;
        single tokens and short portions keep the absorbed form, which never up-projects a cached token."""
        d, r, dv, R = self.dim, self.rot_dim, self.vdim, self.kv_rank
        return (h.dtype == torch.bfloat16 and ctx.cu_context is not None and ctx.max_seqlen_q >= self.EXPAND_FROM
                and (d + r) % 8 == 0 and dv % 8 == 0 and d % 8 == 0 and R % 8 == 0 and d + r <= 256 and dv <= 256)

    def _expanded(self, ctx, src, q, dn, positions, inv_freq):
        H, d, r, dv, R = self.heads, self.dim, self.rot_dim, self.vdim, self.kv_rank
        if getattr(self, "_up", None) is None:      # [W_uk; W_uv] over the latent, built once
            self._up = torch.cat([self.uk_t.data.transpose(1, 2).reshape(H * d, R), self.uv.weight.data]).contiguous()
        bs = src.block_size
        rows = kernels.latent_expand(src.cache, ctx.block_tables, ctx.cu_context, ctx.cu_seqlens_q, ctx.past_lens, bs,
                                     ctx.context_rows, self._up, H, d, r, dv, R)
        B = ctx.past_lens.numel()
        cols = ctx.context_rows // bs          # at most: one request owns every block
        tables = (torch.div(ctx.cu_context[:B], bs, rounding_mode="floor")[:, None]
                  + torch.arange(cols, dtype=torch.int32, device=q.device)[None]).to(torch.int32).contiguous()
        qf = kernels.latent_q_rows(q, positions, inv_freq, self.magnitude, H, d, r, self.rot_dims, self.scale,
                                   self.interleaved)
        out = torch.empty(q.size(0), H * dv, dtype=q.dtype, device=q.device)
        g = self.down.offset("g")
        if self.gate_per_number:
            gate, per_head = dn[:, g:g + H * dv], False
        else:
            gate, per_head = dn[:, g:g + H], True
        kernels.paged_softmax_attn(qf, rows, tables, ctx.cu_seqlens_q, ctx.past_lens, ctx.seq_of_token, ctx.max_seqlen_q,
                                   H, H, d + r, dv, bs, out, window=self.window, gate=gate, gate_per_head=per_head)
        return out
