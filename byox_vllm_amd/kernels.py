"""Tensor-level wrappers over the C ABI (include/nv_hip.h).

Each function checks shapes on the host (the kernels trust their arguments),
passes raw device pointers plus the current HIP stream, and raises on error.
Outputs are allocated with torch.empty unless an ``out`` buffer is given, so
every call is capturable in a hipGraph (torch.cuda.graph) once warmed up.
"""

import os

import torch

from byox_vllm_amd import _C
from byox_vllm_amd._C import check, dtype_code, lib, ptr, require_gpu, stream

_workspaces: dict[tuple, torch.Tensor] = {}
_retired: list[torch.Tensor] = []   # outgrown buffers stay alive: captured graphs may still point at them


def workspace(nbytes: int, device, tag: str = "main") -> torch.Tensor:
    """Grow-only scratch buffer per (device, tag).  Size it before graph capture."""
    # one buffer per stream: micro-batches captured on parallel streams must not share scratch space
    key = (device.index if isinstance(device, torch.device) else torch.device(device).index, tag, stream())
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            _retired.append(ws)
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


class Partials:
    """Split-K output of nv_gemm left as fp32 slabs [n, M, N] in the GEMM workspace, plus the bias still to add.
    Valid until the next gemm() that writes slabs; consumed by add_rms_norm / rope_kv_store."""

    def __init__(self, slabs, n, rows, cols, bias, dtype):
        self.slabs, self.n, self.rows, self.cols, self.bias, self.dtype = slabs, n, rows, cols, bias, dtype


class PendingReduce:
    """Output of a row-parallel linear that still has to be summed over the tensor-parallel ranks: ``value`` is this
    rank's contribution (a tensor or the Partials of its split-K GEMM).  Consumed by RMSNorm, which runs the
    all-reduce fused with its residual add and normalisation (layers/comm.py)."""

    def __init__(self, value):
        self.value = value


class result_policy:
    """``with result_policy(1):`` — launches made inside write the results the next launch reads through to the memory
    side (include/nv_hip.h nv_set_result_policy; a captured launch keeps the policy it was captured under).  The
    setting is one word per process, so it is restored on the way out: runners with different policies can share a
    process."""

    def __init__(self, write_through: int):
        self.mask = int(write_through)

    def __enter__(self):
        self.previous = lib().nv_get_result_policy()
        check(lib().nv_set_result_policy(self.mask), "nv_set_result_policy")

    def __exit__(self, *exc):
        check(lib().nv_set_result_policy(self.previous), "nv_set_result_policy")


def _require_device_weight(w, what: str) -> None:
    """A LinearWeight built from host tensors would hand the kernel a host pointer (a GPU memory fault, not an error
    code): refuse it here."""
    if not w.data.is_cuda or (w.scales is not None and not w.scales.is_cuda):
        raise RuntimeError(f"{what}: the weight's data/scales are on {w.data.device}; they must be device memory")


def rms_norm(x, weight, eps, out=None):
    require_gpu(x, "rms_norm")
    hidden = x.size(-1)
    assert x.is_contiguous() and weight.numel() == hidden and weight.dtype == x.dtype
    out = torch.empty_like(x) if out is None else out
    rows = x.numel() // hidden
    check(lib().nv_rmsnorm(ptr(x), ptr(weight), ptr(out), rows, hidden, hidden, hidden, eps,
                           dtype_code(x.dtype), stream()), "nv_rmsnorm")
    return out


def add_rms_norm(x, residual, weight, eps, out=None, residual_out=None):
    if isinstance(x, Partials):
        assert x.bias is None and residual.is_contiguous() and residual.shape == (x.rows, x.cols)
        out = torch.empty_like(residual) if out is None else out
        residual_out = residual if residual_out is None else residual_out
        check(lib().nv_add_rmsnorm_splitk(ptr(x.slabs), x.n, ptr(residual), ptr(weight), ptr(out), ptr(residual_out),
                                          x.rows, x.cols, eps, dtype_code(residual.dtype), stream()),
              "nv_add_rmsnorm_splitk")
        return out, residual_out
    require_gpu(x, "add_rms_norm")
    hidden = x.size(-1)
    assert x.is_contiguous() and residual.is_contiguous() and x.shape == residual.shape
    assert weight.numel() == hidden and weight.dtype == x.dtype == residual.dtype
    out = torch.empty_like(x) if out is None else out
    residual_out = torch.empty_like(x) if residual_out is None else residual_out
    check(lib().nv_add_rmsnorm(ptr(x), ptr(residual), ptr(weight), ptr(out), ptr(residual_out),
                               x.numel() // hidden, hidden, eps, dtype_code(x.dtype), stream()), "nv_add_rmsnorm")
    return out, residual_out


def rope_kv_store(qkv, positions, cos_sin, num_heads, num_kv_heads, head_dim, slot_mapping=None,
                  k_cache=None, v_cache=None, q_norm_w=None, k_norm_w=None, eps=1e-6):
    """Rotate q and k inside ``qkv`` [T, (H+2Hkv)*D] in place; optionally store k/v into the paged cache.
    ``qkv`` may be the QKV GEMM's Partials: the summed, biased qkv row is then materialised first."""
    partials = None
    if isinstance(qkv, Partials):
        partials = qkv
        assert partials.cols == (num_heads + 2 * num_kv_heads) * head_dim
        qkv = torch.empty(partials.rows, partials.cols, dtype=partials.dtype, device=partials.slabs.device)
    require_gpu(qkv, "rope_kv_store")
    T = qkv.size(0)
    assert qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.size(1) >= (num_heads + 2 * num_kv_heads) * head_dim
    assert positions.dtype == torch.int64 and positions.numel() == T and positions.is_contiguous()
    assert cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.size(-1) == head_dim
    if k_cache is not None:
        assert slot_mapping is not None and slot_mapping.dtype == torch.int32 and slot_mapping.numel() == T
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == qkv.dtype
        assert k_cache.size(-1) == head_dim and k_cache.size(-2) == num_kv_heads
    if partials is not None:
        check(lib().nv_rope_kv_store_splitk(ptr(partials.slabs), partials.n, ptr(partials.bias), ptr(qkv),
                                            qkv.stride(0), ptr(positions), ptr(cos_sin), ptr(slot_mapping),
                                            ptr(k_cache), ptr(v_cache), ptr(q_norm_w), ptr(k_norm_w), eps, T,
                                            num_heads, num_kv_heads, head_dim, dtype_code(qkv.dtype), stream()),
              "nv_rope_kv_store_splitk")
        return qkv
    check(lib().nv_rope_kv_store(ptr(qkv), qkv.stride(0), ptr(positions), ptr(cos_sin), ptr(slot_mapping),
                                 ptr(k_cache), ptr(v_cache), ptr(q_norm_w), ptr(k_norm_w), eps, T,
                                 num_heads, num_kv_heads, head_dim, dtype_code(qkv.dtype), stream()),
          "nv_rope_kv_store")
    return qkv


def gemm_rope_kv_store(x, w, bias, positions, cos_sin, num_heads, num_kv_heads, head_dim, slot_mapping=None,
                       k_cache=None, v_cache=None, q_norm_w=None, k_norm_w=None, eps=1e-6, out=None):
    """qkv projection + bias + [head norms] + RoPE + KV-cache store in one launch -> qkv [T, (H+2Hkv)*D]
    (q and k rotated, v as projected).  ``w``: LinearWeight of the packed q|k|v rows."""
    require_gpu(x, "gemm_rope_kv_store")
    _require_device_weight(w, "gemm_rope_kv_store")
    T, K = x.shape
    N = (num_heads + 2 * num_kv_heads) * head_dim
    assert K == w.in_features and N == w.out_features and x.stride(1) == 1 and x.dtype == w.dtype
    assert positions.dtype == torch.int64 and positions.numel() == T and positions.is_contiguous()
    assert cos_sin.dtype == torch.float32 and cos_sin.is_contiguous() and cos_sin.size(-1) == head_dim
    if bias is not None:
        assert bias.numel() == N and bias.dtype == x.dtype
    if k_cache is not None:
        assert slot_mapping is not None and slot_mapping.dtype == torch.int32 and slot_mapping.numel() == T
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == x.dtype
        assert k_cache.size(-1) == head_dim and k_cache.size(-2) == num_kv_heads
    if out is None:
        out = torch.empty(T, N, dtype=x.dtype, device=x.device)
    check(lib().nv_gemm_rope_kv_store(ptr(x), x.stride(0), ptr(w.data), ptr(w.scales), ptr(bias), ptr(out), out.stride(0),
                                      T, K, w.fmt, ptr(positions), ptr(cos_sin), ptr(slot_mapping), ptr(k_cache),
                                      ptr(v_cache), ptr(q_norm_w), ptr(k_norm_w), eps, num_heads, num_kv_heads,
                                      head_dim, dtype_code(x.dtype), stream()), "nv_gemm_rope_kv_store")
    return out


def kv_store(key, value, k_cache, v_cache, slot_mapping):
    """store_kvcache: key/value [T, Hkv, D] (may be strided views of a qkv buffer)."""
    require_gpu(key, "kv_store")
    T, hkv, d = key.shape
    row = hkv * d
    assert key.stride(-1) == 1 and value.stride(-1) == 1 and key.stride(1) == d and value.stride(1) == d
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.size(-1) * k_cache.size(-2) == row
    assert slot_mapping.dtype == torch.int32 and slot_mapping.numel() == T
    check(lib().nv_kv_store(ptr(key), key.stride(0), ptr(value), value.stride(0), ptr(k_cache), ptr(v_cache),
                            ptr(slot_mapping), T, row, dtype_code(key.dtype), stream()), "nv_kv_store")


def pick_decode_splits(batch, num_kv_heads, max_context):
    return lib().nv_paged_attn_decode_pick_splits(batch, num_kv_heads, max_context)


def paged_attn_decode(q, k_cache, v_cache, context_lens, block_tables, scale, out=None, num_splits=1):
    """q [B, H, D] (row-strided ok); caches [NB, bs, Hkv, D]; returns [B, H, D]."""
    require_gpu(q, "paged_attn_decode")
    B, H, D = q.shape
    nb, bs, hkv, d2 = k_cache.shape
    assert d2 == D and q.stride(2) == 1 and q.stride(1) == D
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and v_cache.shape == k_cache.shape
    assert context_lens.dtype == torch.int32 and context_lens.numel() == B and context_lens.is_contiguous()
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.size(0) >= B
    assert block_tables.stride(1) == 1
    out = torch.empty(B, H, D, dtype=q.dtype, device=q.device) if out is None else out
    assert out.stride(2) == 1 and out.stride(1) == D
    nbytes = lib().nv_paged_attn_decode_workspace_bytes(B, H, D, num_splits)
    ws = workspace(nbytes, q.device, "attn") if nbytes else None
    check(lib().nv_paged_attn_decode(ptr(q), q.stride(0), ptr(k_cache), ptr(v_cache), ptr(block_tables),
                                     block_tables.stride(0), ptr(context_lens), ptr(out), out.stride(0),
                                     ptr(ws), ws.numel() if ws is not None else 0, B, H, hkv, D, bs, scale,
                                     num_splits, dtype_code(q.dtype), stream()), "nv_paged_attn_decode")
    return out


def paged_attn_decode_static(q, k_cache, v_cache, context_lens, block_tables, scale, out, num_splits=1):
    """paged_attn_decode through the entry point that allocates nothing: ``out`` is required and the split partials
    live in the library's own per-GPU array (nv_paged_attn_decode_static)."""
    require_gpu(q, "paged_attn_decode_static")
    B, H, D = q.shape
    nb, bs, hkv, d2 = k_cache.shape
    assert d2 == D and q.stride(2) == 1 and q.stride(1) == D and out.shape == q.shape
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and v_cache.shape == k_cache.shape
    assert context_lens.dtype == torch.int32 and context_lens.numel() == B and context_lens.is_contiguous()
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.size(0) >= B
    assert block_tables.stride(1) == 1 and out.stride(2) == 1 and out.stride(1) == D
    check(lib().nv_paged_attn_decode_static(ptr(q), q.stride(0), ptr(k_cache), ptr(v_cache), ptr(block_tables),
                                            block_tables.stride(0), ptr(context_lens), ptr(out), out.stride(0),
                                            B, H, hkv, D, bs, scale, num_splits, dtype_code(q.dtype), stream()),
          "nv_paged_attn_decode_static")
    return out


def attn_prefill(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, scale, block_tables=None, out=None):
    """Causal varlen attention.  Packed k/v [Tk, Hkv, D] or, with block_tables, paged caches [NB, bs, Hkv, D]."""
    require_gpu(q, "attn_prefill")
    Tq, H, D = q.shape
    assert q.stride(2) == 1 and q.stride(1) == D
    assert cu_seqlens_q.dtype == torch.int32 and cu_seqlens_k.dtype == torch.int32
    n = cu_seqlens_q.numel() - 1
    if block_tables is None:
        hkv = k.size(1)
        assert k.stride(2) == 1 and k.stride(1) == D and v.stride(1) == D and k.stride(0) == v.stride(0)
        kv_stride, bs, bt_stride = k.stride(0), 0, 0
    else:
        assert k.is_contiguous() and v.is_contiguous() and k.dim() == 4
        hkv, bs = k.size(2), k.size(1)
        assert block_tables.dtype == torch.int32 and block_tables.size(0) >= n and block_tables.stride(1) == 1
        kv_stride, bt_stride = hkv * D, block_tables.stride(0)
    out = torch.empty(Tq, H, D, dtype=q.dtype, device=q.device) if out is None else out
    check(lib().nv_attn_prefill(ptr(q), q.stride(0), ptr(k), ptr(v), kv_stride, ptr(cu_seqlens_q), ptr(cu_seqlens_k),
                                ptr(block_tables), bt_stride, ptr(out), out.stride(0), n, max_seqlen_q, H, hkv, D, bs,
                                scale, dtype_code(q.dtype), stream()), "nv_attn_prefill")
    return out


def silu_mul(x, out=None):
    require_gpu(x, "silu_mul")
    assert x.is_contiguous() and x.dim() == 2 and x.size(1) % 2 == 0
    T, two_i = x.shape
    out = torch.empty(T, two_i // 2, dtype=x.dtype, device=x.device) if out is None else out
    check(lib().nv_silu_mul(ptr(x), ptr(out), T, two_i // 2, dtype_code(x.dtype), stream()), "nv_silu_mul")
    return out


def pick_split_k(M, N, K, wfmt=_C.W_INT4):
    """The library's own choice of split-K for this shape (see nv_gemm_pick_split_k)."""
    return lib().nv_gemm_pick_split_k(M, N, K, wfmt)


# Rows from which a product goes through the vendor library (nv_gemm_lt) instead of nv_gemm's decode-shaped tiles:
# prefill steps.  Measured on the layer shapes of Qwen3-0.6B, Qwen2-0.5B and Qwen2-7B, weight expansion included
# (scripts/r03_dense_prefill_gemm.py): at 1024 rows nv_gemm wins everywhere, at 2048 the two trade places by shape,
# from 4096 on the library wins or ties (1.3-1.7 times faster from 8192).  NV_GEMM_LT_ROWS=0 switches the path off.
MANY_ROWS = int(os.environ.get("NV_GEMM_LT_ROWS", "4096"))
LT_WORKSPACE_BYTES = 128 << 20


def expand_weight(w, gate_up_rows=False, out=None):
    """Row-major [N, K] copy, in the model dtype, of a LinearWeight in any format (nv_weight_expand)."""
    _require_device_weight(w, "expand_weight")
    N, K = w.out_features, w.in_features
    out = torch.empty(N, K, dtype=w.dtype, device=w.data.device) if out is None else out
    assert out.is_contiguous() and out.shape == (N, K) and out.dtype == w.dtype
    check(lib().nv_weight_expand(ptr(w.data), ptr(w.scales), w.fmt, N, K, int(gate_up_rows), dtype_code(w.dtype), ptr(out),
                                 stream()), "nv_weight_expand")
    return out


def gemm_many_rows(x, w, bias=None, out=None, silu_mul=False):
    """gemm() for prefill-sized x: the weight written out row-major into scratch, one vendor-library product, and for
    gate/up weights the SiluAndMul pass over its result (same roundings as the fused epilogue: the product rounded to
    the model dtype, silu rounded, the product with up rounded)."""
    M, K = x.shape
    N = w.out_features
    dev = x.device
    if w.fmt == _C.W_DENSE and not silu_mul:
        wr = w.data
    else:
        wr = workspace(N * K * x.element_size(), dev, "gemm_lt_weight")[:N * K * x.element_size()].view(x.dtype).view(N, K)
        expand_weight(w, gate_up_rows=silu_mul, out=wr)
    if silu_mul:
        y = workspace(M * N * x.element_size(), dev, "gemm_lt_gate_up")[:M * N * x.element_size()].view(x.dtype).view(M, N)
    else:
        y = torch.empty(M, N, dtype=x.dtype, device=dev) if out is None else out
        assert y.stride(1) == 1 and y.shape == (M, N)
    ws = workspace(LT_WORKSPACE_BYTES, dev, "gemm_lt")
    check(lib().nv_gemm_lt(ptr(x), x.stride(0), ptr(wr), ptr(bias), ptr(y), y.stride(0), M, N, K, dtype_code(x.dtype),
                           ptr(ws), LT_WORKSPACE_BYTES, stream()), "nv_gemm_lt")
    if not silu_mul:
        return y
    out = torch.empty(M, N // 2, dtype=x.dtype, device=dev) if out is None else out
    assert out.is_contiguous() and out.shape == (M, N // 2)
    check(lib().nv_silu_mul(ptr(y), ptr(out), M, N // 2, dtype_code(x.dtype), stream()), "nv_silu_mul")
    return out


_many_rows_blocked = 0


def block_many_rows(on: bool) -> None:
    """Keep products off the vendor-library route while ``on`` (counted: callers pair True with False).  For jobs whose
    ranks SHARE a GPU (rehearsals of the tensor-parallel runtime): the library's persistent stream-K workgroups and the
    peer-memory all-reduce's workgroups both wait for partners that must be resident at the same time, and with eight
    processes on one device the all-reduce's bounded wait has been seen to run out."""
    global _many_rows_blocked
    _many_rows_blocked = max(0, _many_rows_blocked + (1 if on else -1))


def use_many_rows_path(M, K, N) -> bool:
    return bool(MANY_ROWS) and M >= MANY_ROWS and not _many_rows_blocked and K % 128 == 0 and N % 16 == 0 \
        and lib().nv_gemm_lt_available() == 1 and not torch.cuda.is_current_stream_capturing()


def gemm(x, w, bias=None, out=None, split_k=None, silu_mul=False, partial_out=False):
    """x [M, K] @ w^T where ``w`` is a layers.quant.LinearWeight (dense, int8 or int4).

    silu_mul: ``w`` holds gate/up rows interleaved (LinearWeight.interleave_gate_up); returns silu(gate)*up [M, N/2].
    partial_out: return the split-K slabs as a Partials for a fused consumer instead of reducing them here."""
    require_gpu(x, "gemm")
    _require_device_weight(w, "gemm")
    M, K = x.shape
    assert K == w.in_features and x.stride(1) == 1 and x.dtype == w.dtype
    N = w.out_features
    if bias is not None:
        assert bias.numel() == N and bias.dtype == x.dtype
    if split_k is None:
        if use_many_rows_path(M, K, N) and (out is None or out.is_contiguous() or not silu_mul):
            return gemm_many_rows(x, w, bias, out, silu_mul)
        split_k = 1 if silu_mul else pick_split_k(M, N, K, w.fmt)
    split_k = max(1, min(split_k, K // 128))
    if split_k == 1:
        partial_out = False   # nothing to fuse: the GEMM epilogue writes the finished rows itself
    flags = (_C.GEMM_SILU_MUL if silu_mul else 0) | (_C.GEMM_PARTIAL_OUT if partial_out else 0)
    ws = None
    if split_k > 1 or partial_out:
        ws = workspace(lib().nv_gemm_workspace_bytes(M, N, split_k), x.device, "gemm")
    if partial_out:
        out_ptr, out_stride = None, N
    else:
        out = torch.empty(M, N // 2 if silu_mul else N, dtype=x.dtype, device=x.device) if out is None else out
        assert out.stride(1) == 1 and out.size(1) == (N // 2 if silu_mul else N)
        out_ptr, out_stride = ptr(out), out.stride(0)
    check(lib().nv_gemm(ptr(x), x.stride(0), ptr(w.data), ptr(w.scales), None if partial_out else ptr(bias), out_ptr,
                        out_stride, M, N, K, w.fmt, split_k, ptr(ws), ws.numel() if ws is not None else 0, flags,
                        dtype_code(x.dtype), stream()), "nv_gemm")
    if partial_out:
        return Partials(ws, split_k, M, N, bias, x.dtype)
    return out


def embed(ids, weight, vocab_start=0, out=None):
    require_gpu(weight, "embed")
    assert ids.dtype == torch.int64 and ids.is_contiguous() and weight.is_contiguous()
    T, hidden = ids.numel(), weight.size(1)
    out = torch.empty(T, hidden, dtype=weight.dtype, device=weight.device) if out is None else out
    check(lib().nv_embed(ptr(ids), ptr(weight), ptr(out), T, hidden, vocab_start, weight.size(0),
                         dtype_code(weight.dtype), stream()), "nv_embed")
    return out


def sample(logits, temperatures, noise=None, seed=0, out=None, seed_offset=None):
    require_gpu(logits, "sample")
    B, V = logits.shape
    assert logits.stride(1) == 1 and temperatures.dtype == torch.float32 and temperatures.numel() == B
    if noise is not None:
        assert noise.dtype == torch.float32 and noise.shape == logits.shape and noise.is_contiguous()
    out = torch.empty(B, dtype=torch.int64, device=logits.device) if out is None else out
    ws = workspace(lib().nv_sample_workspace_bytes(B, V), logits.device, "sample")
    check(lib().nv_sample(ptr(logits), logits.stride(0), ptr(temperatures), ptr(noise), ptr(out), ptr(ws), ws.numel(),
                          B, V, seed & 0xFFFFFFFFFFFFFFFF, ptr(seed_offset), dtype_code(logits.dtype), stream()),
          "nv_sample")
    return out


def lm_head_sample(x, w, temperatures, seed=0, out=None, seed_offset=None, logits=None):
    """LM head and sampler chained (embed_head.py:54-66 + sampler.py:11-15 of the reference): x [M, K] against the
    vocabulary matrix ``w`` (an unquantised LinearWeight) -> (tokens [M], logits [M, V]).  The GEMM's epilogue hands
    the sampler its statistics, so the logits are not read again; the tokens are those of ``sample(gemm(x, w), ...)``
    bit for bit, which is also what runs where the GEMM planner would split K (small vocabularies)."""
    require_gpu(x, "lm_head_sample")
    _require_device_weight(w, "lm_head_sample")
    M, K = x.shape
    V = w.out_features
    assert K == w.in_features and x.stride(1) == 1 and x.dtype == w.dtype and w.scales is None
    assert temperatures.dtype == torch.float32 and temperatures.numel() == M
    out = torch.empty(M, dtype=torch.int64, device=x.device) if out is None else out
    logits = torch.empty(M, V, dtype=x.dtype, device=x.device) if logits is None else logits
    assert logits.shape == (M, V) and logits.stride(1) == 1
    if V % 16 or pick_split_k(M, V, K, w.fmt) != 1:
        gemm(x, w, out=logits)
        return sample(logits, temperatures, seed=seed, out=out, seed_offset=seed_offset), logits
    ws = workspace(lib().nv_lm_head_sample_workspace_bytes(M, V), x.device, "sample")
    check(lib().nv_lm_head_sample(ptr(x), x.stride(0), ptr(w.data), w.fmt, ptr(logits), logits.stride(0),
                                  ptr(temperatures), ptr(out), ptr(ws), ws.numel(), M, V, K,
                                  seed & 0xFFFFFFFFFFFFFFFF, ptr(seed_offset), dtype_code(x.dtype), stream()),
          "nv_lm_head_sample")
    return out, logits


def stage_decode_inputs(ids, positions, slots, context_lens, block_tables, g):
    """Copy one step's metadata into the static buffers ``g`` of a captured graph (padding the tail)."""
    bs, padded = ids.numel(), g["padded_bs"]
    cols = block_tables.size(1)
    assert block_tables.is_contiguous() and cols <= g["block_tables"].size(1)
    check(lib().nv_stage_decode_inputs(ptr(ids), ptr(positions), ptr(slots), ptr(context_lens), ptr(block_tables),
                                       cols, ptr(g["input_ids"]), ptr(g["positions"]), ptr(g["slot_mapping"]),
                                       ptr(g["context_lens"]), ptr(g["block_tables"]), g["block_tables"].size(1),
                                       bs, padded, stream()), "nv_stage_decode_inputs")


STAGE_ADVANCE = 0x40000000   # header word 1 of the packed buffer: continue the previous step on the device
STAGE_STEP_BACK = 0x20000000  # header word 1: the previous launch was discarded, take its step count back first


def stage_decode_packed(packed, bs, bt_cols, g, prev_tokens=None, block_size=0):
    """Unpack one step's host buffer (already copied to the device) into the static graph buffers ``g``.
    ``prev_tokens`` (header form only): the launch also honours the STAGE_ADVANCE flag of the header."""
    if prev_tokens is not None:
        assert bs < 0 and prev_tokens.dtype == torch.int64 and block_size > 0
        check(lib().nv_stage_decode_packed_advance(
            ptr(packed), g["padded_bs"], ptr(g["input_ids"]), ptr(g["positions"]), ptr(g["slot_mapping"]),
            ptr(g["context_lens"]), ptr(g["block_tables"]), g["block_tables"].size(1), ptr(g.get("temperatures")),
            ptr(g.get("step")), ptr(prev_tokens), block_size, stream()), "nv_stage_decode_packed_advance")
        return
    check(lib().nv_stage_decode_packed(ptr(packed), bs, g["padded_bs"], bt_cols, ptr(g["input_ids"]),
                                       ptr(g["positions"]), ptr(g["slot_mapping"]), ptr(g["context_lens"]),
                                       ptr(g["block_tables"]), g["block_tables"].size(1), ptr(g.get("temperatures")),
                                       ptr(g.get("step")), stream()), "nv_stage_decode_packed")


# ---------------------------------------------------------------------------------------------------------------
# Kernels of models with an fp32 residual stream (bf16 or true fp32 storage): nv_linear and its row-wise companions.

EPI_NONE, EPI_GLU, EPI_SOFTCAP, EPI_ROW_GATE, EPI_ACT = 0, 1, 2, 3, 4
ACT_SILU, ACT_GELU_TANH, ACT_XIELU, ACT_SCALE = 0, 1, 2, 3
GATE_PER_NUMBER = 1  # EPI_ROW_GATE only (as ``act``): one gate logit per output number instead of one per row and batch
GLU_CLAMPED = 2      # EPI_GLU only: g sigmoid(1.702 g) (u + 1) with g = min(gate, cap), u = clamp(up, -cap, cap)
ROUTE_CHOSEN, ROUTE_ALL = 0, 1   # softmax over the chosen logits / over every expert, renormalised over the chosen


def _code32(dt) -> int:
    return dtype_code(dt, allow_f32=True)


def linear(x, w, bias=None, out=None, out_dtype=None, *, rows=None, a_rows=None, batch=1, a_batch_stride=0,
           w_batch_stride=0, out_batch_stride=0, group_offsets=None, max_group_rows=None, epilogue=EPI_NONE,
           act=ACT_SILU, gate=None, gate_stride=0, cap=0.0, n=None):
    """nv_linear.  ``x`` [M, >=K] (row stride free) in the model dtype, ``w`` [.., K] rows of the same dtype.
    Plain: w [N, K] -> out [M, N].  ``batch`` > 1: per-batch element strides select the operands (heads).
    ``group_offsets`` [batch + 1]: batch b owns output rows [off[b], off[b+1]) (experts), ``a_rows`` maps an output row to
    its row of x, ``max_group_rows`` bounds a group.  GLU: w holds n gate rows then n up rows per batch."""
    require_gpu(x, "linear")
    assert x.dim() == 2 and x.stride(1) == 1 and w.stride(-1) == 1 and w.dtype == x.dtype and w.is_cuda
    K = w.size(-1)
    if n is None:
        n = w.size(-2) // (2 if epilogue == EPI_GLU else 1)
    M = x.size(0) if rows is None else rows
    # prefill-sized plain products of a 16-bit model go where the engine sends its other many-row products: the vendor
    # library, here with the result left in fp32
    if (epilogue in (EPI_NONE, EPI_GLU, EPI_ACT) and batch == 1 and group_offsets is None and a_rows is None
            and (bias is None or (epilogue == EPI_ACT and (out_dtype or x.dtype) == x.dtype)) and out is None
            and rows is None and x.dtype == torch.bfloat16 and (out_dtype or x.dtype) in (torch.float32, torch.bfloat16)
            and w.dim() == 2 and w.is_contiguous() and x.stride(0) % 8 == 0 and use_many_rows_path(M, K, n) and K % 8 == 0
            and n % 8 == 0 and x.data_ptr() % 16 == 0):
        if epilogue == EPI_GLU:      # [gate | up] rows from the library, activation and product in one pass over them
            y = _linear_many_rows(x, w, M, 2 * n, K, torch.float32)
            out = torch.empty(M, n, dtype=out_dtype or x.dtype, device=x.device)
            check(lib().nv_act_mul_f32(ptr(y), ptr(out), M, n, act, cap, _code32(out.dtype), stream()), "nv_act_mul_f32")
            return out
        if epilogue == EPI_ACT:      # the element-wise function in one pass over the library's fp32 result
            y = _linear_many_rows(x, w, M, n, K, torch.float32)
            out = torch.empty(M, n, dtype=out_dtype or x.dtype, device=x.device)
            assert bias is None or (bias.dtype == x.dtype and bias.numel() == n and bias.is_contiguous())
            check(lib().nv_bias_act_f32(ptr(y), ptr(bias), n, ptr(out), M * n, act, ptr(gate), cap, _code32(out.dtype),
                                        stream()), "nv_bias_act_f32")
            return out
        return _linear_many_rows(x, w, M, n, K, out_dtype or x.dtype)
    grid_rows = M if group_offsets is None else (max_group_rows if max_group_rows is not None else M)
    out_dtype = out_dtype or x.dtype
    if out is None:
        cols = n * batch if (batch > 1 and group_offsets is None) else n
        out = torch.empty(M, cols, dtype=out_dtype, device=x.device)
        if batch > 1 and group_offsets is None and out_batch_stride == 0:
            out_batch_stride = n
    assert out.stride(-1) == 1 and out.dtype == out_dtype
    if bias is not None:
        assert bias.dtype == x.dtype and bias.is_contiguous()
    if gate is not None:
        assert gate.dtype == torch.float32
    if group_offsets is not None:
        assert group_offsets.dtype == torch.int32 and group_offsets.numel() == batch + 1
    if a_rows is not None:
        assert a_rows.dtype == torch.int32
    check(lib().nv_linear(ptr(x), x.stride(0), ptr(a_rows), ptr(w), w.stride(-2), ptr(bias), ptr(out), out.stride(0),
                          _code32(out_dtype), grid_rows, n, K, batch, a_batch_stride, w_batch_stride, out_batch_stride,
                          n if bias is not None and batch > 1 else 0, ptr(group_offsets), epilogue, act, ptr(gate),
                          gate_stride, cap, _code32(x.dtype), stream()), "nv_linear")
    return out


def _linear_many_rows(x, w, M, N, K, out_dtype):
    ws = workspace(LT_WORKSPACE_BYTES, x.device, "gemm_lt")
    out = torch.empty(M, N, dtype=out_dtype, device=x.device)
    if out_dtype == torch.float32:
        check(lib().nv_gemm_lt_f32out(ptr(x), x.stride(0), ptr(w), ptr(out), N, M, N, K, dtype_code(x.dtype), ptr(ws),
                                      LT_WORKSPACE_BYTES, stream()), "nv_gemm_lt_f32out")
    else:
        check(lib().nv_gemm_lt(ptr(x), x.stride(0), ptr(w), None, ptr(out), N, M, N, K, dtype_code(x.dtype), ptr(ws),
                               LT_WORKSPACE_BYTES, stream()), "nv_gemm_lt")
    return out


def embed_scale(ids, table, scale, out=None):
    require_gpu(table, "embed_scale")
    assert ids.dtype == torch.int64 and ids.is_contiguous() and table.is_contiguous()
    T, width = ids.numel(), table.size(1)
    out = torch.empty(T, width, dtype=torch.float32, device=table.device) if out is None else out
    check(lib().nv_embed_scale(ptr(ids), ptr(table), ptr(out), T, width, table.size(0), scale, _code32(table.dtype),
                               stream()), "nv_embed_scale")
    return out


def dyt_norm(x, alpha, w, b, delta=None, rows_idx=None, out=None):
    """Dynamic Tanh of the fp32 residual rows ``x`` (updated in place by ``delta`` first when given)."""
    require_gpu(x, "dyt_norm")
    n = x.size(-1)
    assert x.dtype == torch.float32 and x.is_contiguous() and alpha.dtype == torch.float32 and w.dtype == b.dtype
    assert w.numel() == n and b.numel() == n
    rows = x.size(0) if rows_idx is None else rows_idx.numel()
    if delta is not None:
        assert delta.dtype == torch.float32 and delta.stride(1) == 1 and delta.shape == x.shape
    if rows_idx is not None:
        assert rows_idx.dtype == torch.int32
    out = torch.empty(rows, n, dtype=w.dtype, device=x.device) if out is None else out
    check(lib().nv_dyt_norm(ptr(x), ptr(delta), delta.stride(0) if delta is not None else 0, ptr(rows_idx), ptr(alpha),
                            ptr(w), ptr(b), ptr(out), rows, n, _code32(w.dtype), stream()), "nv_dyt_norm")
    return out


def rms_norm_f32(x, w, eps, out=None):
    """RMS norm of fp32 rows (a column slice of a wider buffer is fine) -> rows in the dtype of ``w``."""
    require_gpu(x, "rms_norm_f32")
    assert x.dim() == 2 and x.dtype == torch.float32 and x.stride(1) == 1 and w.numel() == x.size(1)
    out = torch.empty(x.shape, dtype=w.dtype, device=x.device) if out is None else out
    check(lib().nv_rmsnorm_f32(ptr(x), x.stride(0), ptr(w), ptr(out), out.stride(0), x.size(0), x.size(1), eps,
                               _code32(w.dtype), stream()), "nv_rmsnorm_f32")
    return out


def sample_f32(logits, temperatures, seed=0, out=None):
    """Tokens from fp32 logits [B, V]: argmax where the temperature is 0, Gumbel-max otherwise."""
    require_gpu(logits, "sample_f32")
    B, V = logits.shape
    assert logits.dtype == torch.float32 and logits.stride(1) == 1
    assert temperatures.dtype == torch.float32 and temperatures.numel() == B
    out = torch.empty(B, dtype=torch.int64, device=logits.device) if out is None else out
    check(lib().nv_sample_f32(ptr(logits), logits.stride(0), ptr(temperatures), ptr(out), B, V,
                              seed & 0xFFFFFFFFFFFFFFFF, stream()), "nv_sample_f32")
    return out


def gla_recurrent(proj, offsets, z, state, cu_q, past_lens, state_slots, norm_w, heads, dim, vdim, tau, q_scale, eps,
                  out=None):
    """Gated linear attention over the step's tokens; ``proj`` fp32 [T, *] holds q | k | v | g at ``offsets``; ``state``
    fp32 [slots, heads, dim, vdim] is read (unless the request starts) and written back."""
    require_gpu(proj, "gla_recurrent")
    T = proj.size(0)
    assert proj.dtype == z.dtype == state.dtype == torch.float32 and proj.stride(1) == 1 and z.stride(1) == 1
    assert state.is_contiguous() and state.shape[1:] == (heads, dim, vdim) and norm_w.numel() == vdim
    assert cu_q.dtype == past_lens.dtype == state_slots.dtype == torch.int32
    B = past_lens.numel()
    assert cu_q.numel() == B + 1 and state_slots.numel() == B
    out = torch.empty(T, heads * vdim, dtype=norm_w.dtype, device=proj.device) if out is None else out
    q_off, k_off, v_off, g_off = offsets
    check(lib().nv_gla_recurrent(ptr(proj), proj.stride(0), q_off, k_off, v_off, g_off, ptr(z), z.stride(0), ptr(state),
                                 ptr(cu_q), ptr(past_lens), ptr(state_slots), ptr(norm_w), ptr(out), B, heads, dim, vdim,
                                 tau, q_scale, eps, _code32(norm_w.dtype), stream()), "nv_gla_recurrent")
    return out


MEM_CONST, MEM_EXPGATE = 0, 1


def matrix_memory_state_size(mode, dim, vdim) -> int:
    """fp32 numbers one head keeps between steps: the matrix, and in the gated form the normaliser and the maximum, once
    per slice of 64 value columns (each slice is walked by a workgroup of its own).  Mirrors nv_matrix_memory_state_size."""
    return dim * vdim + (-(-vdim // 64) * (dim + 1) if mode == MEM_EXPGATE else 0)


def matrix_memory(proj, offsets, state, cu_q, past_lens, state_slots, heads, dim, vdim, mode, *, decay=None, bias=None,
                  gate_offsets=(0, 0), cap=0.0, silu=False, q_scale=1.0, out=None):
    """Matrix memory with one decay per head and token over the step's tokens; ``proj`` fp32 [T, *] holds q | k | v at
    ``offsets`` (and, MEM_EXPGATE, one input-gate and one forget-gate logit per head at ``gate_offsets``, to which
    ``bias`` over proj's columns is added); ``state`` fp32 [slots, heads, state size] is read (unless the request
    starts) and written back.  -> fp32 [T, heads * vdim]."""
    require_gpu(proj, "matrix_memory")
    T = proj.size(0)
    assert proj.dtype == state.dtype == torch.float32 and proj.stride(1) == 1 and state.is_contiguous()
    assert state.shape[1:] == (heads, matrix_memory_state_size(mode, dim, vdim))
    assert cu_q.dtype == past_lens.dtype == state_slots.dtype == torch.int32
    B = past_lens.numel()
    assert cu_q.numel() == B + 1 and state_slots.numel() == B
    q_off, k_off, v_off = offsets
    i_off, f_off = gate_offsets
    cols = proj.size(1)
    assert max(q_off + heads * dim, k_off + heads * dim, v_off + heads * vdim) <= cols
    dt = torch.float32
    if mode == MEM_CONST:
        assert decay is not None and decay.dtype == torch.float32 and decay.numel() == heads and decay.is_cuda
    else:
        assert max(i_off, f_off) + heads <= cols and cap > 0
        if bias is not None:
            assert bias.is_contiguous() and bias.numel() >= max(i_off, f_off) + heads and bias.is_cuda
            dt = bias.dtype
    out = torch.empty(T, heads * vdim, dtype=torch.float32, device=proj.device) if out is None else out
    assert out.dtype == torch.float32 and out.stride(1) == 1 and out.size(0) == T and out.size(1) >= heads * vdim
    check(lib().nv_matrix_memory(ptr(proj), proj.stride(0), q_off, k_off, v_off, i_off, f_off, ptr(bias), ptr(decay),
                                 ptr(state), ptr(cu_q), ptr(past_lens), ptr(state_slots), ptr(out), out.stride(0), B, heads,
                                 dim, vdim, mode, int(silu), q_scale, cap, _code32(dt), stream()), "nv_matrix_memory")
    return out


def residual_pair(x, x0, dtype, delta=None):
    """[x | x0] rows in ``dtype`` for the projection that re-enters a block of layers; the fp32 rows ``x`` take ``delta``
    in place first."""
    require_gpu(x, "residual_pair")
    assert x.dtype == x0.dtype == torch.float32 and x.is_contiguous() and x0.is_contiguous() and x.shape == x0.shape
    assert x.dim() == 2
    if delta is not None:
        assert delta.dtype == torch.float32 and delta.stride(1) == 1 and delta.shape == x.shape
    out = torch.empty(x.size(0), 2 * x.size(1), dtype=dtype, device=x.device)
    check(lib().nv_residual_pair(ptr(x), ptr(delta), delta.stride(0) if delta is not None else 0, ptr(x0), ptr(out),
                                 x.size(0), x.size(1), _code32(dtype), stream()), "nv_residual_pair")
    return out


def latent_kv_store(kv, norm_w, positions, inv_freq, mscale, slot_mapping, cache, rank, rot_dim, rot_dims, eps,
                    interleaved=False):
    """``interleaved``: dimension 2i turns with 2i + 1 instead of i with i + rot_dims / 2."""
    require_gpu(kv, "latent_kv_store")
    assert kv.dtype == torch.float32 and kv.stride(1) == 1 and kv.size(1) == rank + rot_dim
    assert positions.dtype == torch.int64 and slot_mapping.dtype == torch.int32 and inv_freq.dtype == torch.float32
    assert cache.is_contiguous() and cache.size(-1) == rank + rot_dim and cache.dtype == norm_w.dtype
    assert positions.numel() == slot_mapping.numel() == kv.size(0) and inv_freq.numel() * 2 >= rot_dims
    check(lib().nv_latent_kv_store(ptr(kv), kv.stride(0), ptr(norm_w), ptr(positions), ptr(inv_freq), mscale,
                                   ptr(slot_mapping), ptr(cache), kv.size(0), rank, rot_dim, rot_dims, int(interleaved),
                                   eps, _code32(cache.dtype), stream()), "nv_latent_kv_store")


def latent_q_rope(q, positions, inv_freq, mscale, qa, heads, dim, rot_dim, rot_dims, rank, interleaved=False):
    require_gpu(q, "latent_q_rope")
    assert q.stride(1) == 1 and q.size(1) == heads * (dim + rot_dim) and qa.dtype == torch.float32 and qa.is_contiguous()
    assert qa.numel() == q.size(0) * heads * (rank + rot_dim) and positions.dtype == torch.int64
    check(lib().nv_latent_q_rope(ptr(q), q.stride(0), ptr(positions), ptr(inv_freq), mscale, ptr(qa), q.size(0), heads,
                                 dim, rot_dim, rot_dims, int(interleaved), rank, _code32(q.dtype), stream()),
          "nv_latent_q_rope")


def latent_q_rows(q, positions, inv_freq, mscale, heads, dim, rot_dim, rot_dims, factor, interleaved=False):
    """q [T, heads * (dim + rot_dim)] -> fp32 rows of the same layout, the rotated part turned, everything times
    ``factor``."""
    require_gpu(q, "latent_q_rows")
    assert q.stride(1) == 1 and q.size(1) == heads * (dim + rot_dim) and positions.dtype == torch.int64
    out = torch.empty(q.size(0), heads * (dim + rot_dim), dtype=torch.float32, device=q.device)
    check(lib().nv_latent_q_rows(ptr(q), q.stride(0), ptr(positions), ptr(inv_freq), mscale, ptr(out), q.size(0), heads,
                                 dim, rot_dim, rot_dims, int(interleaved), dim, 1, factor, _code32(q.dtype), stream()),
          "nv_latent_q_rows")
    return out


def latent_expand(cache, block_tables, cu_k, cu_q, past_lens, block_size, rows, up_weight, heads, dim, rot_dim, vdim, rank):
    """The expanded keys and values of every request of a step: its cache rows [rank | rot_dim] gathered in order of
    position (request b at rows cu_k[b] .., padded to whole blocks; ``rows`` = cu_k[-1] on the host), multiplied by
    ``up_weight`` [heads * dim + heads * vdim, rank] -> [rows, heads * (dim + rot_dim) | heads * vdim] in the cache
    dtype, laid out like the rows of ordinary paged attention."""
    require_gpu(cache, "latent_expand")
    Dk = rank + rot_dim
    assert cache.is_contiguous() and cache.size(-1) == Dk and up_weight.shape == (heads * (dim + vdim), rank)
    assert block_tables.dtype == cu_k.dtype == cu_q.dtype == past_lens.dtype == torch.int32 and block_tables.is_contiguous()
    c = torch.empty(rows, Dk, dtype=cache.dtype, device=cache.device)
    check(lib().nv_latent_gather(ptr(cache), ptr(block_tables), block_tables.size(1), ptr(cu_k), ptr(cu_q), ptr(past_lens),
                                 past_lens.numel(), block_size, Dk, ptr(c), rows, _code32(cache.dtype), stream()),
          "nv_latent_gather")
    kv = linear(c[:, :rank], up_weight)
    out = torch.empty(rows, heads * (dim + rot_dim + vdim), dtype=cache.dtype, device=cache.device)
    check(lib().nv_latent_expand(ptr(kv), ptr(c), ptr(out), rows, heads, dim, rot_dim, vdim, rank, _code32(cache.dtype),
                                 stream()), "nv_latent_expand")
    return out


def latent_attn(qa, cache, block_tables, cu_q, past_lens, seq_of_token, heads, rank, rot_dim, block_size, window, scale,
                out=None, max_q=0):
    """Sliding-window attention of absorbed queries ``qa`` fp32 [T, heads, rank + rot_dim] over the paged latent cache
    -> [T, heads * rank] in the cache dtype (sum of softmax weights times latents).  ``max_q`` 1 says that every request
    brings one token: several workgroups may then share a token's keys."""
    require_gpu(qa, "latent_attn")
    T = qa.size(0)
    assert qa.dtype == torch.float32 and qa.is_contiguous() and cache.is_contiguous()
    assert block_tables.dtype == torch.int32 and block_tables.is_contiguous() and block_tables.dim() == 2
    assert cu_q.dtype == past_lens.dtype == seq_of_token.dtype == torch.int32 and seq_of_token.numel() == T
    out = torch.empty(T, heads * rank, dtype=cache.dtype, device=qa.device) if out is None else out
    # steps of one token per request: room for the shares of several workgroups per token (sized before graph capture
    # by the warm-up run of the same shape)
    nbytes = lib().nv_latent_attn_workspace_bytes(T, max_q, heads, rank) if cache.dtype == torch.bfloat16 else 0
    ws = workspace(nbytes, qa.device, "latent_attn") if nbytes else None
    check(lib().nv_latent_attn_split(ptr(qa), ptr(cache), ptr(block_tables), block_tables.size(1), ptr(cu_q),
                                     ptr(past_lens), ptr(seq_of_token), ptr(out), T, past_lens.numel(), heads, rank,
                                     rot_dim, block_size, window, scale, int(max_q), ptr(ws), nbytes,
                                     _code32(cache.dtype), stream()), "nv_latent_attn_split")
    return out


def moe_route(logits, experts, top, mode=ROUTE_CHOSEN):
    """fp32 router logits [T, >=experts] -> (chosen experts int32 [T, top], their weights fp32 [T, top]): the softmax
    over the chosen logits, or (ROUTE_ALL) scores of the softmax over all experts divided by the chosen ones' sum."""
    require_gpu(logits, "moe_route")
    assert logits.dtype == torch.float32 and logits.stride(1) == 1
    T = logits.size(0)
    idx = torch.empty(T, top, dtype=torch.int32, device=logits.device)
    wt = torch.empty(T, top, dtype=torch.float32, device=logits.device)
    check(lib().nv_moe_route(ptr(logits), logits.stride(0), ptr(idx), ptr(wt), T, experts, top, mode, stream()),
          "nv_moe_route")
    return idx, wt


def moe_sort(idx, experts):
    """-> (offsets int32 [experts + 1], token of every sorted row int32 [T * top], sorted row of every pair int32 [T, top])."""
    T, top = idx.shape
    dev = idx.device
    offsets = torch.empty(experts + 1, dtype=torch.int32, device=dev)
    sorted_token = torch.empty(T * top, dtype=torch.int32, device=dev)
    slot_of = torch.empty(T, top, dtype=torch.int32, device=dev)
    check(lib().nv_moe_sort(ptr(idx), T, experts, top, ptr(offsets), ptr(sorted_token), ptr(slot_of), stream()),
          "nv_moe_sort")
    return offsets, sorted_token, slot_of


def moe_combine(y, slot_of, weights, shared=None, shared_gate=None, out=None):
    T, top = slot_of.shape
    width = y.size(1)
    assert y.dtype == weights.dtype == torch.float32 and y.is_contiguous() and weights.is_contiguous()
    if shared is not None:
        assert shared.dtype == torch.float32 and shared.is_contiguous() and shared.shape == (T, width)
        assert shared_gate is None or shared_gate.dtype == torch.float32
    out = torch.empty(T, width, dtype=torch.float32, device=y.device) if out is None else out
    check(lib().nv_moe_combine(ptr(y), ptr(slot_of), ptr(weights), top, ptr(shared), ptr(shared_gate),
                               shared_gate.stride(0) if shared_gate is not None else 0, ptr(out), T, width, stream()),
          "nv_moe_combine")
    return out


# ---- residual streams, token shift, shaped-score attention, recurrences with state slots ----
def embed_sinusoid(ids, positions, table, inv_freq, streams, out=None):
    """fp32 streams [T, streams, width], each table[id] + (sin, cos) pairs of position * inv_freq (float64 [ceil(width/2)])."""
    require_gpu(table, "embed_sinusoid")
    T, width = ids.numel(), table.size(1)
    assert ids.dtype == positions.dtype == torch.int64 and ids.is_contiguous() and positions.is_contiguous()
    assert positions.numel() == T and table.is_contiguous()
    assert inv_freq.dtype == torch.float64 and inv_freq.is_cuda and inv_freq.numel() * 2 >= width
    out = torch.empty(T, streams, width, dtype=torch.float32, device=table.device) if out is None else out
    check(lib().nv_embed_sinusoid(ptr(ids), ptr(positions), ptr(table), ptr(inv_freq), ptr(out), T, streams, width,
                                  table.size(0), _code32(table.dtype), stream()), "nv_embed_sinusoid")
    return out


def hc_norm(x, w, eps, hc_in=None, delta=None, hc_prev=None, rows_idx=None, one_plus=True, out_dtype=None, out=None):
    """RMS norm of a weighted sum of the fp32 streams ``x`` [T, S, width].  ``delta`` [T, width] (the previous sublayer's
    output) is first folded into the streams with ``hc_prev`` = in | out | mix of that sublayer (None: added to every
    stream); ``hc_in`` [S] weighs the streams (None: their sum).  ``rows_idx`` gathers rows and leaves ``x`` alone."""
    require_gpu(x, "hc_norm")
    T, S, width = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous() and w.numel() == width and w.is_contiguous()
    if delta is not None:
        assert delta.dtype == torch.float32 and delta.stride(1) == 1 and delta.shape == (T, width)
    for t, n in ((hc_prev, 2 * S + S * S), (hc_in, S)):
        assert t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= n and t.is_cuda)
    rows = T if rows_idx is None else rows_idx.numel()
    if rows_idx is not None:
        assert rows_idx.dtype == torch.int32
    out_dtype = out_dtype or w.dtype
    out = torch.empty(rows, width, dtype=out_dtype, device=x.device) if out is None else out
    assert out.dtype == out_dtype and out.stride(1) == 1
    check(lib().nv_hc_norm(ptr(x), S, width, ptr(delta), delta.stride(0) if delta is not None else 0,
                           ptr(hc_prev) if delta is not None else None, ptr(hc_in), ptr(w), int(one_plus), eps,
                           ptr(rows_idx), ptr(out), out.stride(0), _code32(out_dtype), rows, _code32(w.dtype), stream()),
          "nv_hc_norm")
    return out


def token_shift(h, mu, state, cu_q, past_lens, state_slots, seq_of_token, out=None):
    """h fp32 [T, width] -> h + (previous row - h) * mu in the dtype of ``mu``; ``state`` fp32 [slots, width]."""
    require_gpu(h, "token_shift")
    T, width = h.shape
    assert h.dtype == state.dtype == torch.float32 and h.is_contiguous() and state.is_contiguous()
    assert state.size(-1) == width and mu.numel() == width
    assert cu_q.dtype == past_lens.dtype == state_slots.dtype == seq_of_token.dtype == torch.int32
    assert seq_of_token.numel() == T and cu_q.numel() == past_lens.numel() + 1 == state_slots.numel() + 1
    out = torch.empty(T, width, dtype=mu.dtype, device=h.device) if out is None else out
    check(lib().nv_token_shift(ptr(h), ptr(mu), ptr(state), ptr(cu_q), ptr(past_lens), ptr(state_slots),
                               ptr(seq_of_token), ptr(out), T, width, _code32(mu.dtype), stream()), "nv_token_shift")
    return out


def group_rms_norm_f32(x, w, groups, eps, out=None, gate=None):
    """fp32 rows [T, groups * n]: every part of n numbers by its own root mean square, times w (times sigmoid of the
    fp32 ``gate`` logits of the same layout, if given) -> rows in w's dtype."""
    require_gpu(x, "group_rms_norm_f32")
    assert x.dim() == 2 and x.dtype == torch.float32 and x.stride(1) == 1 and w.numel() == x.size(1)
    assert x.size(1) % groups == 0
    out = torch.empty(x.shape, dtype=w.dtype, device=x.device) if out is None else out
    assert gate is None or (gate.dtype == torch.float32 and gate.stride(1) == 1 and gate.shape == x.shape)
    check(lib().nv_group_rmsnorm_f32(ptr(x), x.stride(0), ptr(w), ptr(out), out.stride(0), x.size(0), groups,
                                     x.size(1) // groups, eps, ptr(gate), gate.stride(0) if gate is not None else 0,
                                     _code32(w.dtype), stream()), "nv_group_rmsnorm_f32")
    return out


def qk_norm_store(proj, offsets, q_norm, k_norm, temp, scale, eps, slot_mapping, cache, heads, kv_heads, dim, vdim,
                  bias=None):
    """fp32 projections [T, *] with q | k | v at ``offsets`` -> fp32 queries [T, heads * dim] (normalised, times scale and
    the head's temperature); normalised keys and values go to the cache rows [G * dim | G * vdim] of ``slot_mapping``.
    ``bias`` (a vector over the projection's columns) is added to the projections first."""
    require_gpu(proj, "qk_norm_store")
    T = proj.size(0)
    assert proj.dtype == torch.float32 and proj.stride(1) == 1 and slot_mapping.dtype == torch.int32
    assert slot_mapping.numel() == T and cache.is_contiguous() and cache.size(-1) == kv_heads * (dim + vdim)
    assert q_norm.numel() == k_norm.numel() == dim and q_norm.dtype == k_norm.dtype == cache.dtype
    assert temp is None or (temp.numel() == heads and temp.dtype == cache.dtype)
    q_off, k_off, v_off = offsets
    assert max(q_off + heads * dim, k_off + kv_heads * dim, v_off + kv_heads * vdim) <= proj.size(1)
    assert bias is None or (bias.dtype == cache.dtype and bias.is_contiguous() and bias.numel() <= proj.size(1)
                            and bias.numel() >= max(q_off + heads * dim, k_off + kv_heads * dim, v_off + kv_heads * vdim))
    q = torch.empty(T, heads * dim, dtype=torch.float32, device=proj.device)
    check(lib().nv_qk_norm_store(ptr(proj), ptr(bias), proj.stride(0), q_off, k_off, v_off, ptr(q_norm), ptr(k_norm), ptr(temp),
                                 scale, eps, ptr(slot_mapping), ptr(cache), ptr(q), T, heads, kv_heads, dim, vdim,
                                 _code32(cache.dtype), stream()), "nv_qk_norm_store")
    return q


def window_attn(q, cache, block_tables, cu_q, past_lens, seq_of_token, max_q, heads, kv_heads, dim, vdim, block_size,
                window, softcap, out, out_scale=1.0):
    """Attention of fp32 queries [T, heads * dim] over the paged cache; ``out`` [T, >= heads * vdim] (a column slice of a
    wider buffer is fine) in the cache dtype receives out_scale * the weighted values."""
    require_gpu(q, "window_attn")
    T = q.size(0)
    assert q.dtype == torch.float32 and q.is_contiguous() and q.size(1) == heads * dim and cache.is_contiguous()
    assert block_tables.dtype == torch.int32 and block_tables.is_contiguous() and block_tables.dim() == 2
    assert cu_q.dtype == past_lens.dtype == seq_of_token.dtype == torch.int32 and seq_of_token.numel() == T
    assert out.dtype == cache.dtype and out.stride(1) == 1 and out.size(0) == T and out.size(1) >= heads * vdim
    check(lib().nv_window_attn(ptr(q), ptr(cache), ptr(block_tables), block_tables.size(1), ptr(cu_q), ptr(past_lens),
                               ptr(seq_of_token), ptr(out), out.stride(0), T, max_q, heads, kv_heads, dim, vdim,
                               block_size, window, float(softcap or 0.0), out_scale, _code32(cache.dtype), stream()),
          "nv_window_attn")
    return out


def qk_rotate_store(proj, offsets, positions, scale, slot_mapping, cache, heads, kv_heads, dim, vdim, *, q_norm=None,
                    k_norm=None, eps=0.0, inv_freq=None, rot_dims=0, mscale=1.0, v_first=None, vmix=None, bias=None):
    """fp32 projections [T, *] with q | k | v at ``offsets`` -> fp32 queries [T, heads * dim] times ``scale``; keys and
    values go to cache rows [G * dim | G * vdim] of ``slot_mapping``.  ``q_norm`` [heads * dim] / ``k_norm``
    [kv_heads * dim]: one RMS norm over all of a token's query numbers (and all of its key numbers) with a weight per
    number.  ``rot_dims``: the first rot_dims numbers of every head turn by position * inv_freq[i], i with
    i + rot_dims / 2.  ``v_first`` fp32 [T, G * vdim] (a column slice is fine): the stored values are
    (1 - vmix) v + vmix v_first."""
    require_gpu(proj, "qk_rotate_store")
    T = proj.size(0)
    assert proj.dtype == torch.float32 and proj.stride(1) == 1 and slot_mapping.dtype == torch.int32
    assert slot_mapping.numel() == T and cache.is_contiguous() and cache.size(-1) == kv_heads * (dim + vdim)
    assert positions.dtype == torch.int64 and positions.numel() == T and positions.is_contiguous()
    q_off, k_off, v_off = offsets
    need = max(q_off + heads * dim, k_off + kv_heads * dim, v_off + kv_heads * vdim)
    assert need <= proj.size(1)
    assert bias is None or (bias.dtype == cache.dtype and bias.is_contiguous() and need <= bias.numel() <= proj.size(1))
    assert (q_norm is None) == (k_norm is None)
    if q_norm is not None:
        assert q_norm.numel() == heads * dim and k_norm.numel() == kv_heads * dim
        assert q_norm.dtype == k_norm.dtype == cache.dtype and q_norm.is_contiguous() and k_norm.is_contiguous()
    if rot_dims:
        assert rot_dims % 2 == 0 and rot_dims <= dim and inv_freq.dtype == torch.float32 and inv_freq.is_contiguous()
        assert inv_freq.numel() * 2 >= rot_dims and inv_freq.is_cuda
    if v_first is not None:
        assert v_first.dtype == torch.float32 and v_first.stride(1) == 1 and v_first.shape == (T, kv_heads * vdim)
        assert vmix.dtype == cache.dtype and vmix.numel() == 1 and vmix.is_cuda
    q = torch.empty(T, heads * dim, dtype=torch.float32, device=proj.device)
    check(lib().nv_qk_rotate_store(ptr(proj), ptr(bias), proj.stride(0), q_off, k_off, v_off, ptr(q_norm), ptr(k_norm),
                                   int(q_norm is not None), None, ptr(positions), 0.0, 0, ptr(inv_freq), int(rot_dims),
                                   float(mscale), ptr(v_first), v_first.stride(0) if v_first is not None else 0,
                                   ptr(vmix) if v_first is not None else None, scale, eps, ptr(slot_mapping), ptr(cache),
                                   ptr(q), T, heads, kv_heads, dim, vdim, _code32(cache.dtype), stream()),
          "nv_qk_rotate_store")
    return q


def qk_store(proj, offsets, positions, scale, slot_mapping, cache, heads, kv_heads, dim, bias=None, temp_coef=0.0,
             temp_every=0):
    """fp32 projections [T, *] with q | k at ``offsets`` (plus ``bias`` over the same columns) -> fp32 queries
    [T, heads * dim] times ``scale`` and the position temperature 1 + coef * ln(floor((p + 1) / every) + 1) (every 0:
    none); the keys go to cache rows [G * dim] of ``slot_mapping``: they are the values too."""
    require_gpu(proj, "qk_store")
    T = proj.size(0)
    assert proj.dtype == torch.float32 and proj.stride(1) == 1 and slot_mapping.dtype == torch.int32
    assert slot_mapping.numel() == T and cache.is_contiguous() and cache.size(-1) == kv_heads * dim
    assert positions.dtype == torch.int64 and positions.numel() == T and positions.is_contiguous()
    q_off, k_off = offsets
    need = max(q_off + heads * dim, k_off + kv_heads * dim)
    assert need <= proj.size(1)
    assert bias is None or (bias.dtype == cache.dtype and bias.is_contiguous() and need <= bias.numel() <= proj.size(1))
    q = torch.empty(T, heads * dim, dtype=torch.float32, device=proj.device)
    check(lib().nv_qk_store(ptr(proj), ptr(bias), proj.stride(0), q_off, k_off, 0, None, None, None, ptr(positions),
                            float(temp_coef), int(temp_every), scale, 0.0, ptr(slot_mapping), ptr(cache), ptr(q), T, heads,
                            kv_heads, dim, 0, _code32(cache.dtype), stream()), "nv_qk_store")
    return q


def paged_softmax_attn(q, cache, block_tables, cu_q, past_lens, seq_of_token, max_q, heads, kv_heads, dim, vdim, block_size,
                       out, window=0, softcap=0.0, out_scale=1.0, distance_term=False, values_are_keys=False, sink=None,
                       gate=None, chunk=0, gate_per_head=False):
    """window_attn with its options spelled out: no distance term unless asked for, cache rows that hold keys only and
    serve as values too, a sink logit per head in the denominator, a sigmoid gate (fp32 logits laid out like the
    output, or with ``gate_per_head`` one per head) folded into the store, and ``chunk`` > 0: a query sees the keys
    of its own chunk of the sequence only."""
    require_gpu(q, "paged_softmax_attn")
    T = q.size(0)
    assert q.dtype == torch.float32 and q.is_contiguous() and q.size(1) == heads * dim and cache.is_contiguous()
    assert cache.size(-1) == (kv_heads * dim if values_are_keys else kv_heads * (dim + vdim))
    assert block_tables.dtype == torch.int32 and block_tables.is_contiguous() and block_tables.dim() == 2
    assert cu_q.dtype == past_lens.dtype == seq_of_token.dtype == torch.int32 and seq_of_token.numel() == T
    assert out.dtype == cache.dtype and out.stride(1) == 1 and out.size(0) == T and out.size(1) >= heads * vdim
    assert sink is None or (sink.dtype == cache.dtype and sink.numel() == heads and sink.is_contiguous())
    assert gate is None or (gate.dtype == torch.float32 and gate.stride(1) == 1 and gate.size(0) == T
                            and gate.size(1) >= (heads if gate_per_head else heads * vdim))
    # steps of one token per request: room for the shares of several workgroups per token (sized before graph capture
    # by the warm-up run of the same shape)
    nbytes = lib().nv_paged_softmax_attn_workspace_bytes(T, max_q, heads, kv_heads, vdim) if cache.dtype == torch.bfloat16 else 0
    ws = workspace(nbytes, q.device, "paged_softmax_attn") if nbytes else None
    check(lib().nv_paged_softmax_attn(ptr(q), ptr(cache), ptr(block_tables), block_tables.size(1), ptr(cu_q),
                                      ptr(past_lens), ptr(seq_of_token), ptr(out), out.stride(0), T, max_q, heads, kv_heads,
                                      dim, vdim, block_size, window, int(chunk), float(softcap or 0.0), out_scale,
                                      int(distance_term), int(values_are_keys), ptr(sink), ptr(gate),
                                      gate.stride(0) if gate is not None else 0, int(gate_per_head), ptr(ws), nbytes,
                                      _code32(cache.dtype), stream()),
          "nv_paged_softmax_attn")
    return out


def causal_conv(x, w, bias, state, cu_q, past_lens, state_slots, seq_of_token, act=0, want_f32=True, want_t=False,
                x_bias=None):
    """Per-channel causal convolution of fp32 rows ``x`` [T, C] (a column slice is fine) with ``w`` [C, taps]; ``state``
    fp32 [slots, taps - 1, C].  ``act`` 0: none, 1: SiLU, 2: none, and the token's own input is added (x + conv(x)).
    -> (fp32 result or None, result in w's dtype or None)."""
    require_gpu(x, "causal_conv")
    T, C = x.shape
    taps = w.size(1)
    assert x.dtype == state.dtype == torch.float32 and x.stride(1) == 1 and w.shape == (C, taps) and w.is_contiguous()
    assert state.is_contiguous() and state.shape[1:] == (max(taps - 1, 0), C) and seq_of_token.numel() == T
    assert bias is None or (bias.numel() == C and bias.dtype == w.dtype)
    assert cu_q.dtype == past_lens.dtype == state_slots.dtype == seq_of_token.dtype == torch.int32
    of = torch.empty(T, C, dtype=torch.float32, device=x.device) if want_f32 else None
    ot = torch.empty(T, C, dtype=w.dtype, device=x.device) if want_t else None
    assert x_bias is None or (x_bias.numel() == C and x_bias.dtype == w.dtype and x_bias.stride(0) == 1)
    assert cu_q.numel() == past_lens.numel() + 1
    check(lib().nv_causal_conv_batch(ptr(x), ptr(x_bias), x.stride(0), ptr(w), ptr(bias), ptr(state), ptr(cu_q),
                                     ptr(past_lens), ptr(state_slots), ptr(seq_of_token), ptr(of), C, ptr(ot), C, T,
                                     past_lens.numel(), C, taps, act, _code32(w.dtype), stream()), "nv_causal_conv_batch")
    return of, ot


def rglru_scan(u, gates, y, lam, state, cu_q, past_lens, state_slots, block_width, out, c=8.0, out_scale=1.0,
               y_bias=None):
    """Real-gated linear recurrence over fp32 rows u [T, C]; ``gates`` fp32 [T, 2C] (per block: recurrence-gate logits,
    then input-gate logits); ``y`` fp32 [T, C] is the other branch before its GELU; ``state`` fp32 [slots, C];
    ``out`` [T, >= C] in lam's dtype."""
    require_gpu(u, "rglru_scan")
    T, C = u.shape
    assert u.dtype == gates.dtype == y.dtype == state.dtype == torch.float32
    assert u.stride(1) == gates.stride(1) == y.stride(1) == out.stride(1) == 1 and gates.shape == (T, 2 * C)
    assert y.shape == (T, C) and state.is_contiguous() and state.size(-1) == C and lam.numel() == C
    assert out.dtype == lam.dtype and out.size(0) == T and out.size(1) >= C and C % block_width == 0
    assert cu_q.dtype == past_lens.dtype == state_slots.dtype == torch.int32
    assert y_bias is None or (y_bias.numel() == C and y_bias.dtype == lam.dtype and y_bias.stride(0) == 1)
    check(lib().nv_rglru_scan(ptr(u), u.stride(0), ptr(gates), gates.stride(0), ptr(y), ptr(y_bias), y.stride(0), ptr(lam), ptr(state),
                              ptr(cu_q), ptr(past_lens), ptr(state_slots), ptr(out), out.stride(0), past_lens.numel(), C,
                              block_width, c, out_scale, _code32(lam.dtype), stream()), "nv_rglru_scan")
    return out


def ssd_scan(xbc, z, dt, dt_bias, A_log, D, state, cu_q, past_lens, state_slots, heads, groups, state_size, vdim, max_q=1):
    """Selective state-space recurrence over fp32 rows xbc [T, heads*vdim + 2*groups*state] -> fp32 [T, heads*vdim]
    (already multiplied by silu(z)); ``state`` fp32 [slots, heads, state, vdim].  ``max_q`` bounds the tokens one
    request brings (long prompts are walked in parallel runs through a workspace)."""
    require_gpu(xbc, "ssd_scan")
    T = xbc.size(0)
    inner = heads * vdim
    assert xbc.dtype == z.dtype == dt.dtype == state.dtype == torch.float32
    assert xbc.stride(1) == z.stride(1) == dt.stride(1) == 1 and xbc.size(1) == inner + 2 * groups * state_size
    assert z.shape == (T, inner) and dt.shape == (T, heads) and state.is_contiguous()
    assert state.shape[1:] == (heads, state_size, vdim) and dt_bias.numel() == A_log.numel() == D.numel() == heads
    assert dt_bias.dtype == A_log.dtype == D.dtype
    assert cu_q.dtype == past_lens.dtype == state_slots.dtype == torch.int32
    out = torch.empty(T, inner, dtype=torch.float32, device=xbc.device)
    B = past_lens.numel()
    nbytes = lib().nv_ssd_scan_workspace_bytes(B, heads, state_size, vdim, max_q)
    ws = workspace(nbytes, xbc.device, "ssd_scan") if nbytes else None
    check(lib().nv_ssd_scan(ptr(xbc), xbc.stride(0), ptr(z), z.stride(0), ptr(dt), dt.stride(0), ptr(dt_bias), ptr(A_log),
                            ptr(D), ptr(state), ptr(cu_q), ptr(past_lens), ptr(state_slots), ptr(out), B,
                            heads, groups, state_size, vdim, max_q, ptr(ws), nbytes, _code32(dt_bias.dtype), stream()),
          "nv_ssd_scan")
    return out


def mingru_scan(proj, offsets, z_bias, u_bias, state, cu_q, past_lens, state_slots, channels, out):
    """Minimal gated recurrent unit over fp32 projections ``proj`` [T, *] with update-gate logits | candidates |
    output-gate logits at ``offsets`` (``channels`` columns each; the biases of the first two, in out's dtype, are added
    here); ``state`` fp32 [slots, channels]; ``out`` [T, >= channels] receives S * silu(g)."""
    require_gpu(proj, "mingru_scan")
    T = proj.size(0)
    z_off, u_off, g_off = offsets
    assert proj.dtype == state.dtype == torch.float32 and proj.stride(1) == 1 and out.stride(1) == 1
    assert max(z_off, u_off, g_off) + channels <= proj.size(1) and out.size(0) == T and out.size(1) >= channels
    assert state.is_contiguous() and state.size(-1) == channels
    for b in (z_bias, u_bias):
        assert b is None or (b.numel() == channels and b.dtype == out.dtype and b.stride(0) == 1)
    assert cu_q.dtype == past_lens.dtype == state_slots.dtype == torch.int32
    check(lib().nv_mingru_scan(ptr(proj), proj.stride(0), z_off, u_off, g_off, ptr(z_bias), ptr(u_bias), ptr(state),
                               ptr(cu_q), ptr(past_lens), ptr(state_slots), ptr(out), out.stride(0), past_lens.numel(),
                               channels, _code32(out.dtype), stream()), "nv_mingru_scan")
    return out


def gated_postnorm_add(x, y, w, eps, mult, gate=None, gate_bias=None, out_dtype=None, y_bias=None, conv=None):
    """fp32 residual rows ``x`` [T, n] += mult * rms_norm((y + y_bias) * sigmoid(gate + gate_bias)) * w, in place
    (``gate`` None: no gate; ``y`` None: nothing is added); -> the new rows in ``out_dtype`` (None: no copy).
    ``conv`` = (weight [n, taps], state [slots, taps - 1, n], state_slots, past_lens), for steps in which row t is the
    only token of request t: -> (rows, x + conv(x) in the weight's dtype), the slots moved on by that token."""
    require_gpu(x, "gated_postnorm_add")
    T, n = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    if y is not None:
        assert y.dtype == torch.float32 and y.stride(1) == 1 and y.shape == (T, n) and w.numel() == n and w.is_contiguous()
        assert gate is None or (gate.dtype == torch.float32 and gate.stride(1) == 1 and gate.shape == (T, n))
        for b in (gate_bias, y_bias):
            assert b is None or (b.dtype == w.dtype and b.numel() == n and b.is_contiguous())
        assert out_dtype is None or out_dtype == w.dtype
    out = torch.empty(T, n, dtype=out_dtype, device=x.device) if out_dtype is not None else None
    if conv is not None:
        cw, state, slots, past = conv
        taps = cw.size(1)
        assert cw.shape == (n, taps) and cw.is_contiguous() and state.is_contiguous() and state.shape[1:] == (taps - 1, n)
        assert slots.dtype == past.dtype == torch.int32 and slots.numel() == past.numel() == T
        assert (y is None or cw.dtype == w.dtype) and (out_dtype is None or out_dtype == cw.dtype)
        hc = torch.empty(T, n, dtype=cw.dtype, device=x.device)
        check(lib().nv_gated_postnorm_add_conv(ptr(x), ptr(y), y.stride(0) if y is not None else 0,
                                               ptr(y_bias) if y is not None else None, ptr(gate),
                                               gate.stride(0) if gate is not None else 0, ptr(gate_bias),
                                               ptr(w) if y is not None else None, ptr(out), n, T, n, eps, mult, ptr(cw),
                                               taps, ptr(state), ptr(slots), ptr(past), ptr(hc), n, _code32(cw.dtype),
                                               stream()), "nv_gated_postnorm_add_conv")
        return out, hc
    code = _code32(out_dtype if out_dtype is not None else w.dtype)
    check(lib().nv_gated_postnorm_add(ptr(x), ptr(y), y.stride(0) if y is not None else 0,
                                      ptr(y_bias) if y is not None else None, ptr(gate),
                                      gate.stride(0) if gate is not None else 0, ptr(gate_bias),
                                      ptr(w) if y is not None else None, ptr(out), n, T, n, eps, mult, code, stream()),
          "nv_gated_postnorm_add")
    return out
