"""Zamusun on the GPU: every mechanism's kernel alone against the plain functions of oracle/zamusun.py, then the engine
(scheduler commit, pages, state slots, run_portions) against the oracle run on each request's whole token list."""

import math

import pytest
import torch

from oracle import zamusun as O
from zamusun_cases import (Engine, aligned_config, engine_config, looped_config, odd_config, plain_config,
                           random_checkpoint, row_error, row_errors, wide_config)

pytestmark = pytest.mark.gpu
DEV = "cuda"
F64 = torch.float64
F32_TOL, BF16_TOL = 2e-4, 6e-2          # engine logits against the float64 oracle (row_error)
SAME_TOL = 2e-5                         # fp32 engine against itself under another schedule


def _tol(dtype):
    return F32_TOL if dtype == torch.float32 else BF16_TOL


def _i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


def _steps(pieces, slot=0, past=0):
    """Single-request step arrays for consecutive pieces: (start, count, cu_q, past_lens, state_slots, seq_of_token)."""
    at = 0
    for n in pieces:
        yield at, n, _i32([0, n]), _i32([past + at]), _i32([slot]), _i32([0] * n)
        at += n


def _close(got, want, tol):
    scale = float(want.abs().max()) + 1e-30
    err = float((got.double().cpu() - want.double()).abs().max()) / scale
    assert err <= tol, err


# ------------------------------------------------------------------------------------------------ matrix memories
def _memory_inputs(T, H, d, dv, seed, gates=True):
    g = torch.Generator().manual_seed(seed)
    cols = 2 * H * d + H * dv + (2 * H if gates else 0)
    proj = torch.randn(T, cols + 3, generator=g)                  # three columns nobody reads in front
    offs = (3, 3 + H * d, 3 + 2 * H * d)
    return proj, offs, (3 + 2 * H * d + H * dv, 3 + 2 * H * d + H * dv + H)


def _memory_plain(proj, offs, goffs, H, d, dv, mode, decay=None, bias=None, cap=0.0):
    T = proj.shape[0]
    p = proj.double()
    q, k = p[:, offs[0]:offs[0] + H * d].view(T, H, d), p[:, offs[1]:offs[1] + H * d].view(T, H, d)
    v = p[:, offs[2]:offs[2] + H * dv].view(T, H, dv)
    if mode == 0:
        return O.lightning(O.silu(q), O.silu(k), O.silu(v), torch.tensor(decay, dtype=F64)).reshape(T, H * dv)
    zi, zf = p[:, goffs[0]:goffs[0] + H] + bias[0].double(), p[:, goffs[1]:goffs[1] + H] + bias[1].double()
    i_log = O.soft_bound(zi, cap)
    f_log = torch.nn.functional.logsigmoid(O.soft_bound(zf, cap))
    return O.mlstm(q * d ** -0.5, k, v, i_log, f_log).reshape(T, H * dv)


def _memory_run(proj, offs, goffs, pieces, H, d, dv, mode, state, slot=0, decay=None, bias=None, cap=0.0):
    from byox_vllm_amd import kernels
    pd = proj.to(DEV)
    outs = []
    bias_full = None
    if mode == 1:
        bias_full = torch.zeros(proj.shape[1], device=DEV)
        bias_full[goffs[0]:goffs[0] + H], bias_full[goffs[1]:goffs[1] + H] = bias[0].to(DEV), bias[1].to(DEV)
    dec = torch.tensor(decay, dtype=torch.float32, device=DEV) if decay is not None else None
    for a, n, cu, past, slots, _ in _steps(pieces, slot):
        outs.append(kernels.matrix_memory(pd[a:a + n], offs, state, cu, past, slots, H, d, dv, mode, decay=dec,
                                          bias=bias_full, gate_offsets=goffs, cap=cap, silu=mode == 0,
                                          q_scale=d ** -0.5 if mode == 1 else 1.0))
    return torch.cat(outs)


# value sizes above 64 are walked in slices of 64 columns by workgroups of their own; keys above 256 take the general kernel
SHAPES = [(3, 16, 24), (1, 12, 20), (2, 64, 64), (1, 128, 128), (2, 128, 32), (1, 256, 40), (5, 8, 130), (2, 40, 8),
          (1, 300, 20), (2, 256, 128), (1, 130, 300)]


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("H,d,dv", SHAPES)
@pytest.mark.parametrize("pieces", [[40], [1] * 40, [2, 2, 35, 1], [17, 16, 7]])
def test_matrix_memory_in_pieces(mode, H, d, dv, pieces):
    """A request's tokens in one step, one by one, and in uneven pieces (a chunk of sixteen, its neighbours, two
    tokens), from a slot that held something else before."""
    from byox_vllm_amd import kernels
    proj, offs, goffs = _memory_inputs(40, H, d, dv, seed=H * 100 + d)
    decay = [0.5 + 0.499 * i / max(H - 1, 1) for i in range(H)]
    bias = (torch.linspace(-1, 1, H), torch.linspace(3, 1, H))
    state = torch.full((3, H, kernels.matrix_memory_state_size(mode, d, dv)), float("nan"), device=DEV)
    got = _memory_run(proj, offs, goffs, pieces, H, d, dv, mode, state, slot=1, decay=decay, bias=bias, cap=7.0)
    want = _memory_plain(proj, offs, goffs, H, d, dv, mode, decay=decay, bias=bias, cap=7.0)
    _close(got, want, 2e-5)
    assert torch.isnan(state[0]).all() and torch.isnan(state[2]).all() and not torch.isnan(state[1]).any()


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("H,d,dv", [(2, 24, 16), (1, 64, 130)])
def test_matrix_memory_general_kernel_shares_the_slot_layout(mode, H, d, dv, monkeypatch):
    """The general kernel continues a state the fast kernel left, and the other way round."""
    from byox_vllm_amd import kernels
    assert kernels.matrix_memory_state_size(mode, d, dv) == kernels.lib().nv_matrix_memory_state_size(mode, d, dv)
    proj, offs, goffs = _memory_inputs(45, H, d, dv, seed=9)
    decay, bias = [0.9] * H, (torch.zeros(H), torch.ones(H))
    want = _memory_plain(proj, offs, goffs, H, d, dv, mode, decay=decay, bias=bias, cap=9.0)
    for first_general in (True, False):
        state = torch.full((1, H, kernels.matrix_memory_state_size(mode, d, dv)), float("nan"), device=DEV)
        outs = []
        for k, (a, b) in enumerate(((0, 20), (20, 21), (21, 45))):
            if (k % 2 == 0) == first_general:
                monkeypatch.setenv("NV_MATRIX_MEMORY_GENERIC", "1")
            else:
                monkeypatch.delenv("NV_MATRIX_MEMORY_GENERIC", raising=False)
            outs.append(_memory_run(proj[a:b], offs, goffs, [b - a], H, d, dv, mode, state, decay=decay, bias=bias, cap=9.0)
                        if a == 0 else _memory_continue(proj[a:b], offs, goffs, a, H, d, dv, mode, state, decay, bias, 9.0))
        monkeypatch.delenv("NV_MATRIX_MEMORY_GENERIC", raising=False)
        _close(torch.cat(outs), want, 2e-5)


@pytest.mark.parametrize("mode", [0, 1])
def test_matrix_memory_many_requests_take_whole_heads_and_few_take_slices(mode):
    """64 requests x 8 heads give one workgroup all 128 value columns of a head; the two requests that go on alone are
    then walked in slices of 64 columns, from the state the first launch left."""
    from byox_vllm_amd import kernels
    H, d, dv, B = 8, 16, 128, 64
    projs = [_memory_inputs(5, H, d, dv, seed=200 + i) for i in range(B)]
    offs, goffs = projs[0][1], projs[0][2]
    decay, bias = [0.8 + 0.02 * h for h in range(H)], (torch.zeros(H), torch.ones(H))
    state = torch.full((B, H, kernels.matrix_memory_state_size(mode, d, dv)), float("nan"), device=DEV)
    bias_full = torch.zeros(projs[0][0].shape[1], device=DEV)
    bias_full[goffs[1]:goffs[1] + H] = 1.0
    kw = dict(decay=torch.tensor(decay, device=DEV), bias=bias_full if mode else None, gate_offsets=goffs, cap=5.0,
              silu=mode == 0, q_scale=d ** -0.5 if mode else 1.0)
    batch = torch.cat([p[0][:3] for p in projs]).to(DEV)
    got1 = kernels.matrix_memory(batch, offs, state, _i32(list(range(0, 3 * B + 1, 3))), _i32([0] * B), _i32(list(range(B))),
                                 H, d, dv, mode, **kw)
    keep = [7, 50]
    batch = torch.cat([projs[r][0][3:] for r in keep]).to(DEV)
    got2 = kernels.matrix_memory(batch, offs, state, _i32([0, 2, 4]), _i32([3, 3]), _i32(keep), H, d, dv, mode, **kw)
    for k, r in enumerate(keep):
        want = _memory_plain(projs[r][0], offs, goffs, H, d, dv, mode, decay=decay, bias=bias, cap=5.0)
        _close(torch.cat([got1[3 * r:3 * r + 3], got2[2 * k:2 * k + 2]]), want, 2e-5)
    want = _memory_plain(projs[33][0][:3], offs, goffs, H, d, dv, mode, decay=decay, bias=bias, cap=5.0)
    _close(got1[99:102], want, 2e-5)


def _memory_continue(proj, offs, goffs, past, H, d, dv, mode, state, decay, bias, cap):
    from byox_vllm_amd import kernels
    n = proj.shape[0]
    bias_full = torch.zeros(proj.shape[1], device=DEV)
    bias_full[goffs[0]:goffs[0] + H], bias_full[goffs[1]:goffs[1] + H] = bias[0].to(DEV), bias[1].to(DEV)
    return kernels.matrix_memory(proj.to(DEV), offs, state, _i32([0, n]), _i32([past]), _i32([0]), H, d, dv, mode,
                                 decay=torch.tensor(decay, device=DEV), bias=bias_full if mode else None,
                                 gate_offsets=goffs, cap=cap, silu=mode == 0, q_scale=d ** -0.5 if mode else 1.0)


@pytest.mark.parametrize("mode", [0, 1])
def test_matrix_memory_batch_of_unequal_requests_and_a_reused_slot(mode):
    from byox_vllm_amd import kernels
    H, d, dv = 3, 24, 16
    lens = [19, 1, 33]
    projs = [_memory_inputs(n, H, d, dv, seed=50 + i) for i, n in enumerate(lens)]
    offs, goffs = projs[0][1], projs[0][2]
    decay, bias = [0.6, 0.9, 0.99], (torch.zeros(H), torch.ones(H))
    state = torch.full((4, H, kernels.matrix_memory_state_size(mode, d, dv)), float("nan"), device=DEV)
    dec = torch.tensor(decay, device=DEV)
    bias_full = torch.zeros(projs[0][0].shape[1], device=DEV)
    bias_full[goffs[1]:goffs[1] + H] = 1.0
    kw = dict(decay=dec, bias=bias_full if mode else None, gate_offsets=goffs, cap=5.0, silu=mode == 0,
              q_scale=d ** -0.5 if mode else 1.0)
    # step 1: the first 10 / 1 / 20 tokens of the three requests in slots 2, 0, 3; step 2: the rest of the first and the
    # third (the second has ended); step 3: a new request in the second's slot
    first = [10, 1, 20]
    batch = torch.cat([p[0][:n] for p, n in zip(projs, first)]).to(DEV)
    got1 = kernels.matrix_memory(batch, offs, state, _i32([0, 10, 11, 31]), _i32([0, 0, 0]), _i32([2, 0, 3]), H, d, dv,
                                 mode, **kw)
    batch = torch.cat([projs[0][0][10:], projs[2][0][20:]]).to(DEV)
    got2 = kernels.matrix_memory(batch, offs, state, _i32([0, 9, 22]), _i32([10, 20]), _i32([2, 3]), H, d, dv, mode, **kw)
    got3 = kernels.matrix_memory(projs[1][0].to(DEV), offs, state, _i32([0, 1]), _i32([0]), _i32([0]), H, d, dv, mode, **kw)
    want = [_memory_plain(p[0], offs, goffs, H, d, dv, mode, decay=decay, bias=bias, cap=5.0) for p in projs]
    _close(torch.cat([got1[:10], got2[:9]]), want[0], 2e-5)
    _close(got1[10:11], want[1], 2e-5)
    _close(got3, want[1], 2e-5)
    _close(torch.cat([got1[11:], got2[9:]]), want[2], 2e-5)
    assert torch.isnan(state[1]).all()


@pytest.mark.parametrize("pieces", [[400], [390] + [1] * 10, [5, 250, 145]])
def test_lightning_keeps_a_far_key_under_a_slow_decay_and_loses_it_under_a_fast_one(pieces):
    """Token 3 writes a large value under a key that only token 399 asks for: the head with decay 0.999 still returns it
    (times 0.999^396), the head with decay 0.5 has forgotten it."""
    H, d, dv, T = 2, 16, 8, 400
    g = torch.Generator().manual_seed(7)
    proj = torch.randn(T, 2 * H * d + H * dv, generator=g) * 0.1
    offs = (0, H * d, 2 * H * d)
    for h in range(H):
        proj[:, offs[1] + h * d] = -9.0                                   # silu(-9) ~ 0: nobody else writes channel 0
        proj[:, offs[0] + h * d] = -9.0
        proj[3, offs[1] + h * d] = 6.0
        proj[399, offs[0] + h * d] = 6.0
        proj[3, offs[2] + h * dv: offs[2] + (h + 1) * dv] = 50.0
    from byox_vllm_amd import kernels
    state = torch.zeros(1, H, kernels.matrix_memory_state_size(0, d, dv), device=DEV)
    got = _memory_run(proj, offs, (0, 0), pieces, H, d, dv, 0, state, decay=[0.999, 0.5])
    want = _memory_plain(proj, offs, (0, 0), H, d, dv, 0, decay=[0.999, 0.5])
    assert float(want[399, :dv].min()) > 1000 and float(want[399, dv:].abs().max()) < 1.0
    _close(got, want, 2e-5)


@pytest.mark.parametrize("pieces", [[320], [20] + [1] * 300, [2, 3, 315]])
def test_mlstm_first_tokens_start_from_a_maximum_of_zero_and_a_strong_input_survives_a_long_decode(pieces):
    """The first tokens arrive with very negative input gates: with the running maximum starting at 0 (not at minus
    infinity) they enter with weight exp(i - f), far below one.  Token 10 opens its input gate fully; forget gates stay
    near one, so 300 tokens later it still dominates."""
    H, d, dv, T, cap = 2, 16, 8, 320, 11.0
    g = torch.Generator().manual_seed(8)
    proj = torch.randn(T, 2 * H * d + H * dv + 2 * H, generator=g)
    offs, goffs = (0, H * d, 2 * H * d), (2 * H * d + H * dv, 2 * H * d + H * dv + H)
    proj[:, goffs[0]:goffs[0] + H] = -30.0
    proj[10, goffs[0]:goffs[0] + H] = 40.0
    proj[:, goffs[1]:goffs[1] + H] = 6.0
    bias = (torch.zeros(H), torch.full((H,), 2.0))
    from byox_vllm_amd import kernels
    state = torch.full((1, H, kernels.matrix_memory_state_size(1, d, dv)), 3.0, device=DEV)
    got = _memory_run(proj, offs, goffs, pieces, H, d, dv, 1, state, bias=bias, cap=cap)
    want = _memory_plain(proj, offs, goffs, H, d, dv, 1, bias=bias, cap=cap)
    # a start at minus infinity would give the first token weight 1 and an output of the order of v
    assert float(want[:10].abs().max()) < 1e-2 * float(want[10:].abs().max())
    _close(got[:10], want[:10], 2e-5)
    _close(got, want, 1e-4)                  # three hundred fp32 additions onto a state that hardly decays


# ------------------------------------------------------------------------------------------------ attention
def _attention_plain(proj, offs, H, G, d, scale, sink, coef, every, gate=None, bias=None):
    T = proj.shape[0]
    p = proj.double() + (bias.double() if bias is not None else 0.0)
    q, k = p[:, offs[0]:offs[0] + H * d].view(T, H, d), p[:, offs[1]:offs[1] + G * d].view(T, G, d)
    if every:
        q = q * O.query_temperature(T, coef, every)[:, None, None]
    o = O.sink_attention(q, k, scale, sink.double()).reshape(T, H * d)
    return o * torch.sigmoid(gate.double()) if gate is not None else o


def _paged_sink_attention(proj, offs, pieces, H, G, d, scale, sink, coef, every, dtype, block, gate=None, bias=None, seed=0):
    """The two kernels over one request cut into ``pieces``, on scattered pages."""
    from byox_vllm_amd import kernels
    T = proj.shape[0]
    nblocks = -(-T // block)
    g = torch.Generator().manual_seed(seed)
    pages = torch.randperm(nblocks + 3, generator=g)[:nblocks].tolist()
    cache = torch.full(((nblocks + 3) * block, G * d), float("nan"), dtype=dtype, device=DEV)
    table = _i32([pages])
    out = torch.zeros(T, H * d + 2, dtype=dtype, device=DEV)
    pd = proj.to(DEV)
    gd = gate.to(DEV) if gate is not None else None
    for a, n, cu, past, _, seq_of in _steps(pieces):
        slots = _i32([pages[p // block] * block + p % block for p in range(a, a + n)])
        pos = torch.arange(a, a + n, device=DEV)
        q = kernels.qk_store(pd[a:a + n], offs, pos, scale, slots, cache, H, G, d,
                             bias=bias.to(DEV).to(dtype) if bias is not None else None, temp_coef=coef, temp_every=every)
        kernels.paged_softmax_attn(q, cache, table, cu, past, seq_of, n, H, G, d, d, block, out[a:a + n, 2:],
                                   values_are_keys=True, sink=sink.to(DEV).to(dtype),
                                   gate=gd[a:a + n] if gd is not None else None)
    assert float(out[:, :2].float().abs().max()) == 0.0
    return out[:, 2:].float()


def _round(t, dtype):
    return t.to(dtype).float()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,block", [(6, 2, 16, 16), (1, 1, 20, 16), (3, 1, 12, 32), (8, 2, 32, 16), (8, 1, 128, 64),
                                         (4, 4, 8, 16), (2, 1, 256, 16)])
def test_sink_attention_prompt_pieces_and_single_tokens(dtype, H, G, d, block):
    T = 70
    g = torch.Generator().manual_seed(H * 10 + d)
    proj = _round(torch.randn(T, H * d + G * d + 5, generator=g), dtype)
    offs = (5, 5 + H * d)
    bias = _round(torch.randn(proj.shape[1], generator=g) * 0.3, dtype)
    sink = _round(torch.randn(H, generator=g), dtype)
    gate = torch.randn(T, H * d, generator=g)
    scale = d ** -0.5
    want = _attention_plain(proj, offs, H, G, d, scale, sink, 0.5, 16, gate, bias)
    if dtype == torch.bfloat16:      # the cache holds the keys (= values) rounded to the storage type
        pr = proj.clone()
        pr[:, offs[1]:] = _round(proj[:, offs[1]:offs[1] + G * d] + bias[offs[1]:offs[1] + G * d], dtype) - bias[offs[1]:offs[1] + G * d]
        want = _attention_plain(pr, offs, H, G, d, scale, sink, 0.5, 16, gate, bias)
    for pieces in ([T], [1] * T, [2, 2, 3, 9, 16, 1, 17, 2, 15, 3], [T - 1, 1], [33, 37]):
        got = _paged_sink_attention(proj, offs, pieces, H, G, d, scale, sink, 0.5, 16, dtype, block, gate, bias)
        _close(got, want, 2e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pieces", [[300], [150, 150], [299, 1], [250] + [1] * 50, [64, 64, 64, 108]])
def test_a_far_key_and_the_keys_at_a_page_border_stand_out(pieces, dtype):
    """Head 0 asks at the last position for key 5 (far back, among hundreds), head 1 for key 63 (the last row of a
    page), head 2 for key 64 (the first row of the next): each returns that key, almost alone."""
    H, G, d, T, block = 3, 1, 16, 300, 64
    g = torch.Generator().manual_seed(3)
    proj = torch.randn(T, H * d + G * d, generator=g) * 0.3
    k_off = H * d
    marks = {0: 5, 1: 63, 2: 64}
    for h, j in marks.items():
        proj[j, k_off:] = 0.0
        proj[j, k_off + h] = 6.0
        proj[j, k_off + 8 + h] = 1.0 + h                          # what the output must show
        proj[T - 1, h * d: (h + 1) * d] = 0.0
        proj[T - 1, h * d + h] = 6.0
    proj = _round(proj, dtype)
    sink = torch.zeros(H)
    want = _attention_plain(proj, (0, k_off), H, G, d, 1.0, sink, 0.0, 0)
    for h in marks:
        assert abs(float(want[T - 1, h * d + 8 + h]) - (1.0 + h)) < 1e-3        # 36 against scores of about 1
    got = _paged_sink_attention(proj, (0, k_off), pieces, H, G, d, 1.0, sink, 0.0, 0, dtype, block)
    _close(got, want, 2e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_sink_takes_its_share_of_the_softmax(dtype):
    """All scores are zero, so position i spreads (i + 1) / (i + 1 + exp(sink)) over its keys: a sink of ln 3 makes the
    first position return a quarter of its key, a very negative one changes nothing, a huge one leaves nothing."""
    H, G, d, T = 3, 1, 8, 40
    proj = torch.zeros(T, H * d + G * d)
    proj[:, H * d:] = 2.0
    sink = torch.tensor([math.log(3.0), -60.0, 60.0])
    for pieces in ([T], [1] * T, [7, 33]):
        got = _paged_sink_attention(proj, (0, H * d), pieces, H, G, d, 1.0, sink, 0.0, 0, dtype, 16)
        i = torch.arange(T, dtype=torch.float32)
        _close(got[:, 0], 2.0 * (i + 1) / (i + 4), 2e-6 if dtype == torch.float32 else 1e-2)
        _close(got[:, d], torch.full((T,), 2.0), 2e-6 if dtype == torch.float32 else 1e-2)
        assert float(got[:, 2 * d].abs().max()) < 1e-20


def test_the_query_temperature_follows_the_position_not_the_place_in_the_piece():
    from byox_vllm_amd import kernels
    H, G, d = 2, 1, 4
    proj = torch.ones(6, H * d + G * d, device=DEV)
    cache = torch.zeros(64, G * d, device=DEV)
    pos = torch.tensor([14, 15, 30, 31, 4094, 4095], device=DEV)
    q = kernels.qk_store(proj, (0, H * d), pos, 0.5, _i32([0, 1, 2, 3, -1, 5]), cache, H, G, d, temp_coef=0.5, temp_every=16)
    want = 0.5 * (1.0 + 0.5 * torch.log(torch.tensor([1.0, 2.0, 2.0, 3.0, 256.0, 257.0], dtype=F64)))
    _close(q[:, 0], want, 1e-6)
    assert float(cache[4].abs().max()) == 0.0 and float(cache[5].min()) == 1.0      # slot -1 writes nothing


def test_sink_attention_batch_of_unequal_requests():
    """Three requests in one launch: a prompt piece that continues 21 cached tokens, a single decoded token, a whole
    short prompt; block tables of different lengths."""
    from byox_vllm_amd import kernels
    for dtype in (torch.float32, torch.bfloat16):
        H, G, d, block = 4, 2, 16, 16
        g = torch.Generator().manual_seed(12)
        lens, past = [40, 37, 5], [21, 36, 0]
        projs = [_round(torch.randn(n, H * d + G * d, generator=g), dtype) for n in lens]
        sink = _round(torch.randn(H, generator=g), dtype)
        cache = torch.zeros(12 * block, G * d, dtype=dtype, device=DEV)
        tables = [[7, 2, 9], [4, 1, 8], [5]]
        slot = lambda r, p: tables[r][p // block] * block + p % block   # noqa: E731
        for r in (0, 1):     # what the earlier steps left in the cache
            pos = torch.arange(past[r], device=DEV)
            kernels.qk_store(projs[r][:past[r]].to(DEV), (0, H * d), pos, 0.25, _i32([slot(r, p) for p in range(past[r])]),
                             cache, H, G, d, temp_coef=0.3, temp_every=8)
        new = [projs[r][past[r]:] for r in range(3)]
        counts = [t.shape[0] for t in new]
        pos = torch.cat([torch.arange(past[r], lens[r]) for r in range(3)]).to(DEV)
        slots = _i32([slot(r, p) for r in range(3) for p in range(past[r], lens[r])])
        q = kernels.qk_store(torch.cat(new).to(DEV), (0, H * d), pos, 0.25, slots, cache, H, G, d, temp_coef=0.3,
                             temp_every=8)
        table = torch.full((3, 3), -1, dtype=torch.int32)
        for r, t in enumerate(tables):
            table[r, :len(t)] = torch.tensor(t)
        cu = [0, counts[0], counts[0] + counts[1], sum(counts)]
        seq_of = sum(([r] * c for r, c in enumerate(counts)), [])
        out = torch.zeros(sum(counts), H * d, dtype=dtype, device=DEV)
        kernels.paged_softmax_attn(q, cache, table.to(DEV), _i32(cu), _i32(past), _i32(seq_of), max(counts), H, G, d, d,
                                   block, out, values_are_keys=True, sink=sink.to(DEV).to(dtype))
        for r in range(3):
            want = _attention_plain(projs[r], (0, H * d), H, G, d, 0.25, sink, 0.3, 8)[past[r]:]
            _close(out[cu[r]:cu[r + 1]].float(), want, 2e-5 if dtype == torch.float32 else 2e-2)


# ------------------------------------------------------------------------------------------------ feed-forward, rows
@pytest.mark.parametrize("E,top", [(5, 2), (3, 1), (4, 4), (8, 3)])
def test_routing_over_all_experts(E, top):
    from byox_vllm_amd import kernels
    z = torch.randn(50, E + 2, generator=torch.Generator().manual_seed(E))
    idx, w = kernels.moe_route(z.to(DEV), E, top, kernels.ROUTE_ALL)
    want_idx, want_w = O.route(z[:, :E].double(), top)
    assert torch.equal(idx.cpu().long(), want_idx)
    _close(w, want_w, 1e-6)
    _, chosen = kernels.moe_route(z.to(DEV), E, top, kernels.ROUTE_CHOSEN)
    _close(chosen, want_w, 1e-6)            # the same numbers unless the chosen scores underflow


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M", [3, 100, 4096])
def test_clamped_gated_unit_in_every_route_of_the_product(dtype, M):
    """Few rows, the tiled kernel, and the vendor route with the activation as a pass of its own: gate and up values
    on both sides of the limit."""
    from byox_vllm_amd import kernels
    K, N, limit = 64, 24, 1.25
    g = torch.Generator().manual_seed(M)
    x = _round(torch.randn(M, K, generator=g), dtype)
    w = _round(torch.randn(2 * N, K, generator=g) * 0.3, dtype)
    got = kernels.linear(x.to(DEV).to(dtype), w.to(DEV).to(dtype), epilogue=kernels.EPI_GLU, act=kernels.GLU_CLAMPED,
                         cap=limit, out_dtype=torch.float32)
    gate, up = x.double() @ w[:N].double().T, x.double() @ w[N:].double().T
    assert float(gate.max()) > limit and float(up.min()) < -limit and float(up.max()) > limit
    gc, uc = gate.clamp(max=limit), up.clamp(-limit, limit)
    _close(got, gc * torch.sigmoid(1.702 * gc) * (uc + 1.0), 1e-5)


def test_mixture_layer_against_the_plain_mixture_with_an_addend():
    from byox_vllm_amd.layers.moe import MixtureOfExperts
    cfg = looped_config()
    spec = cfg["layers"][1]["mlp"]
    W = {k: v.float() for k, v in random_checkpoint(cfg, 5).items()}
    width, E, ff = cfg["width"], spec["router"]["experts"], spec["expert"]["ff"]
    torch.set_default_device(DEV)
    try:
        layer = MixtureOfExperts(width, E, spec["router"]["top"], ff, "clamped", route="all", limit=spec["expert"]["limit"])
    finally:
        torch.set_default_device(None)
    layer = layer.float()
    layer.router.weight.data.copy_(W["l1.mlp.router"])
    for e in range(E):
        layer.gate_up.data[e, :ff].copy_(W[f"l1.mlp.e{e}.gate"])
        layer.gate_up.data[e, ff:].copy_(W[f"l1.mlp.e{e}.up"])
        layer.down.data[e].copy_(W[f"l1.mlp.e{e}.down"])
    h = torch.randn(37, width, generator=torch.Generator().manual_seed(1)) * 2
    add = torch.randn(37, width, generator=torch.Generator().manual_seed(2))
    want = O.moe(h.double(), {k: v.double() for k, v in W.items()}, "l1.mlp.", spec)
    _close(layer(h.to(DEV)), want, 2e-5)
    _close(layer(h.to(DEV), add=add.to(DEV)), want + add.double(), 2e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("groups", [1, 3])
def test_group_norm_with_a_sigmoid_gate(dtype, groups):
    from byox_vllm_amd import kernels
    g = torch.Generator().manual_seed(groups)
    x, gate = torch.randn(9, groups * 20, generator=g) * 3, torch.randn(9, groups * 20 + 4, generator=g)
    w = _round(torch.randn(groups * 20, generator=g), dtype)
    got = kernels.group_rms_norm_f32(x.to(DEV), w.to(DEV).to(dtype), groups, 1e-5, gate=gate.to(DEV)[:, 4:])
    want = O.rms(x.double().view(9, groups, 20), 1e-5).reshape(9, -1) * w.double() * torch.sigmoid(gate[:, 4:].double())
    _close(got.float(), want, 1e-6 if dtype == torch.float32 else 8e-3)


def test_residual_pair_folds_the_pending_output_in():
    from byox_vllm_amd import kernels
    g = torch.Generator().manual_seed(0)
    x, x0, delta = (torch.randn(5, 12, generator=g) for _ in range(3))
    xd = x.to(DEV)
    pair = kernels.residual_pair(xd, x0.to(DEV), torch.float32, delta.to(DEV))
    assert torch.equal(xd.cpu(), x + delta) and torch.equal(pair.cpu(), torch.cat([x + delta, x0], 1))
    pair = kernels.residual_pair(xd, x0.to(DEV), torch.bfloat16)
    assert torch.equal(pair.cpu(), torch.cat([x + delta, x0], 1).to(torch.bfloat16)) and torch.equal(xd.cpu(), x + delta)


# ------------------------------------------------------------------------------------------------ the engine
CASES = {"looped": looped_config, "odd": odd_config, "plain": plain_config, "aligned": aligned_config, "wide": wide_config}


@pytest.fixture(scope="module", params=[(n, dt) for n in CASES for dt in (torch.float32, torch.bfloat16)],
                ids=lambda p: f"{p[0]}-{str(p[1])[6:]}")
def setup(request):
    name, dtype = request.param
    cfg = CASES[name]()
    weights = random_checkpoint(cfg, seed=11)
    torch.manual_seed(99)
    reqs = {"a": torch.randint(0, cfg["vocab"], (83,)).tolist(), "b": torch.randint(0, cfg["vocab"], (31,)).tolist(),
            "c": torch.randint(0, cfg["vocab"], (2,)).tolist(), "d": torch.randint(0, cfg["vocab"], (50,)).tolist()}
    want, clear = {}, {}
    for n, t in reqs.items():
        logits, gaps = _forward_with_router_gaps(t, weights, cfg)
        want[n] = logits.float()
        # tokens up to the first whose routers (any layer run) had a close call: no 16-bit rounding can change their experts
        close = (gaps < 0.05).nonzero()
        clear[n] = int(close[0]) if len(close) else len(t)
    engine = Engine(cfg, weights, dtype, blocks=12, slots=3)
    engine.clear = clear
    whole = engine.replay(reqs, [[(n, len(t))] for n, t in reqs.items()])
    return cfg, weights, dtype, reqs, want, engine, whole


def _forward_with_router_gaps(tokens, weights, cfg):
    """The oracle's logits and, per token, the smallest gap over all routers between the last chosen logit and the
    first one left out."""
    gaps, route = [], O.route

    def recording(z, top):
        ordered = z.sort(-1, descending=True).values
        gaps.append(ordered[:, top - 1] - ordered[:, top] if top < z.shape[1] else torch.full((z.shape[0],), math.inf,
                                                                                              dtype=F64))
        return route(z, top)
    O.route = recording
    try:
        logits = O.forward(tokens, weights, cfg)
    finally:
        O.route = route
    return logits, (torch.stack(gaps).min(0).values if gaps else torch.full((len(tokens),), math.inf, dtype=F64))


def _check(setup, got):
    cfg, weights, dtype, reqs, want, engine, whole = setup
    for n in got:
        if dtype == torch.float32:
            assert row_error(got[n], want[n]) < F32_TOL, (n, row_error(got[n], want[n]))
            assert row_error(got[n], whole[n]) < SAME_TOL, n
        else:
            # A router logit of random weights can lie inside the rounding of its 16-bit input; a token that takes
            # another expert is off by much more than rounding, and so, less, are the tokens after it (states and keys
            # carry it on).  Sharp where no router had a close call yet; after that a tenth of the rows may differ.
            err = row_errors(got[n], want[n])
            head = err[:engine.clear[n]]
            assert head.numel() == 0 or float(head.max()) < BF16_TOL, (n, engine.clear[n], head.max())
            assert float((err > BF16_TOL).float().mean()) <= 0.1 and float(err.median()) < BF16_TOL / 2, (n, err.max())


def test_whole_prompts_match_the_oracle(setup):
    _check(setup, setup[6])


def test_every_layer_run_matches_the_oracle(setup):
    """The residual after every layer run (a looped layer counts each time), for one request in one step (fp32 only: it
    is the sharp comparison)."""
    cfg, weights, dtype, reqs, want, engine, whole = setup
    if dtype != torch.float32:
        pytest.skip("layer by layer in fp32 only")
    from byox_vllm_amd.engine.sequence import Sequence
    trace, plain = [], []
    O.forward(reqs["b"], weights, cfg, trace=plain)
    model = engine.runner.model
    forward = model.forward
    model.forward = lambda ids, pos: forward(ids, pos, trace=trace)
    try:
        seq = Sequence(reqs["b"], engine.block_size)
        engine.scheduler.add(seq)
        plan = [(seq, len(reqs["b"]))]
        engine.scheduler.commit(plan)
        engine.runner.run_portions(plan, want=[[0]])
        engine.scheduler.finish(seq)
    finally:
        model.forward = forward
    assert len(trace) == len(plain) == len(O.layer_runs(cfg))
    for got, ref in zip(trace, plain):
        _close(got, ref, 2e-5)


def test_prompt_then_token_by_token(setup):
    reqs = setup[3]
    # the decoded stretch crosses page borders and several steps of the query temperature
    _check(setup, setup[5].replay({"a": reqs["a"]}, [[("a", 20)]] + [[("a", 1)]] * 63))
    _check(setup, setup[5].replay({"b": reqs["b"]}, [[("b", 1)]] * 31))           # from the very first token on


def test_portions_of_many_sizes(setup):
    reqs = setup[3]
    _check(setup, setup[5].replay({"a": reqs["a"]}, [[("a", n)] for n in (2, 2, 3, 9, 16, 1, 17, 2, 15, 14, 2)]))
    _check(setup, setup[5].replay({"d": reqs["d"]}, [[("d", n)] for n in (15, 1, 16, 2, 16)]))


def test_mixed_batches_reuse_pages_and_slots(setup):
    """Three slots, twelve pages of sixteen tokens: four requests only fit because the finished ones give theirs back.
    Prompt pieces run beside single tokens; requests sit out steps."""
    reqs = setup[3]
    schedule = [[("a", 30), ("b", 5)], [("a", 1), ("b", 20), ("c", 2)], [("a", 2), ("b", 1)], [("b", 1), ("d", 7), ("a", 1)],
                [("a", 40), ("d", 1), ("b", 4)], [("d", 30)], [("a", 1), ("d", 1)], [("a", 8), ("d", 11)]]
    _check(setup, setup[5].replay(reqs, schedule))
    # the same requests again, in slots and pages that the first pass has used
    _check(setup, setup[5].replay(reqs, [[("d", 50), ("c", 1)], [("c", 1), ("b", 31)], [("a", 83)]]))


def test_greedy_generation_through_the_engine(setup):
    """LLM.generate (scheduler's own portion policy, sampler at temperature 0) against the oracle's greedy run."""
    cfg, weights, dtype, reqs, want, engine, whole = setup
    from byox_vllm_amd import LLM, SamplingParams
    conf = engine_config(cfg, weights, dtype, blocks=12, slots=3)
    llm = LLM("synthetic", hf_config=conf.hf_config, state_dict=weights, kvcache_block_size=16, num_kvcache_blocks=12,
              max_num_seqs=3, num_state_slots=3, enforce_eager=True, max_num_batched_tokens=48, max_model_len=1 << 20)
    prompts = [reqs["b"], reqs["c"], reqs["d"][:20], reqs["a"][:40]]
    steps = 10
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True), use_tqdm=False)
    llm._exit()
    for prompt, out in zip(prompts, outs):
        tokens = list(prompt) + out["token_ids"]
        logits = O.forward(tokens, weights, cfg)
        spread = float(logits.std())
        for k, tok in enumerate(out["token_ids"]):
            row = logits[len(prompt) + k - 1]
            # the engine's choice is the oracle's argmax, or lies inside the rounding of the engine's dtype
            assert row.max().item() - row[tok].item() <= (1e-3 if dtype == torch.float32 else 0.1) * spread, (k, tok)
        assert len(out["token_ids"]) == steps


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_captured_decode_steps_equal_eager_ones(dtype):
    """Decode steps replayed from hipGraphs (padded batches, the spare state slot, one staging copy) give the tokens of
    the eager engine, step after step, with prompt portions running eagerly between the replays."""
    from byox_vllm_amd import LLM, SamplingParams
    cfg = looped_config()
    weights = random_checkpoint(cfg, seed=21)
    torch.manual_seed(5)
    prompts = [torch.randint(0, cfg["vocab"], (n,)).tolist() for n in (37, 3, 18, 25, 9)]
    params = [SamplingParams(temperature=0.0, max_tokens=n, ignore_eos=True) for n in (30, 41, 12, 25, 33)]
    outs = []
    for eager in (True, False):
        conf = engine_config(cfg, weights, dtype, blocks=24, slots=4)
        llm = LLM("synthetic", hf_config=conf.hf_config, state_dict=weights, kvcache_block_size=16, num_kvcache_blocks=24,
                  max_num_seqs=4, num_state_slots=4, enforce_eager=eager, max_num_batched_tokens=32, max_model_len=128)
        assert bool(llm.model_runner.graphs) == (not eager)
        outs.append([o["token_ids"] for o in llm.generate(prompts, params, use_tqdm=False)])
        llm._exit()
    assert outs[0] == outs[1]
    assert [len(t) for t in outs[0]] == [30, 41, 12, 25, 33]


def test_command_line_generation_and_trace_replay_from_a_model_folder(tmp_path):
    """A model folder (config.json + model.safetensors in bf16) through the two command-line entry points, each in a
    process of its own: `python -m byox_vllm_amd generate` against the oracle's greedy continuation, bin/trace_run
    against the oracle's logits for a replayed schedule with pieces, a pause and a request that ends early."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np
    from safetensors.torch import save_file
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = aligned_config()
    weights = random_checkpoint(cfg, seed=31)
    model = tmp_path / "model"
    model.mkdir()
    with open(model / "config.json", "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, str(model / "model.safetensors"))
    torch.manual_seed(3)
    a = torch.randint(0, cfg["vocab"], (70,)).tolist()
    b = torch.randint(0, cfg["vocab"], (9,)).tolist()

    run = subprocess.run([sys.executable, "-m", "byox_vllm_amd", "generate", "--model", str(model), "--dtype", "float32",
                          "--prompt-ids", ",".join(map(str, b)), "--max-tokens", "6", "--block-size", "16", "--eager"],
                         cwd=root, capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-3000:]
    line = json.loads([ln for ln in run.stdout.splitlines() if ln.startswith("{")][0])
    logits = O.forward(list(b) + line["token_ids"], weights, cfg)
    for k, tok in enumerate(line["token_ids"]):
        row = logits[len(b) + k - 1]
        assert row.max().item() - row[tok].item() <= 1e-3 * float(logits.std())
    assert len(line["token_ids"]) == 6

    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:40], "want": [0, 39]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[:2], "want": []}, {"id": "a", "tokens": a[40:41], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[2:], "want": [6]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[41:], "want": [0, 28]}, {"id": "c", "tokens": b, "want": [8]}], "end": ["a", "c"]}]
    wa, wb = O.forward(a, weights, cfg).float(), O.forward(b, weights, cfg).float()
    for dtype, tol in (("float32", F32_TOL), ("bfloat16", BF16_TOL)):
        out = tmp_path / ("out_" + dtype)
        run = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", str(model), "--dtype", dtype, "--out", str(out),
                              "--max-tokens", "192"], input="\n".join(json.dumps(s) for s in steps) + "\n", cwd=root,
                             capture_output=True, text=True, timeout=600)
        assert run.returncode == 0, run.stderr[-3000:]
        assert [ln for ln in run.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
        expect = {0: wa[[0, 39]], 1: wa[[40]], 2: wb[[8]], 3: torch.cat([wa[[41, 69]], wb[[8]]])}
        for i, want in expect.items():
            got = torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, cfg["vocab"]))
            assert got.shape == want.shape and row_error(got, want) < tol, (dtype, i)
